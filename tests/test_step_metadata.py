"""Host-side metadata of a step: the attention task lists and the sizes that captured programs pad to."""
import numpy as np

from runtime.engine.context import fill_tasks
from runtime.engine.runner import _bucket


def test_task_lists_cover_every_row_once_and_never_cross_a_segment():
    rng = np.random.default_rng(0)
    for _ in range(50):
        counts = rng.integers(1, 40, size=rng.integers(1, 6)).tolist()
        rows_per_tile = int(rng.choice([1, 2, 4, 5, 16, 64]))
        most = -(-sum(counts) // rows_per_tile) + len(counts)
        tasks = np.full((most, 4), -7, dtype=np.int32)
        n = fill_tasks(tasks, counts, rows_per_tile)
        assert n == sum(-(-c // rows_per_tile) for c in counts) <= most
        assert (tasks[n:] == -7).all()
        starts = np.concatenate(([0], np.cumsum(counts)))
        seen = []
        for seg, first, rows, zero in tasks[:n]:
            assert zero == 0 and 1 <= rows <= rows_per_tile
            assert starts[seg] <= first and first + rows <= starts[seg + 1]
            seen += list(range(first, first + rows))
        assert seen == list(range(sum(counts)))
        # with the segments' first positions: the same tiles, those with the most keys first
        seg_starts = rng.integers(0, 100, size=len(counts)).tolist()
        ordered = np.full((most, 4), -7, dtype=np.int32)
        assert fill_tasks(ordered, counts, rows_per_tile, seg_starts) == n
        assert sorted(map(tuple, ordered[:n, :3])) == sorted(map(tuple, tasks[:n, :3]))
        keys = [seg_starts[seg] + first - starts[seg] + rows for seg, first, rows, _ in ordered[:n]]
        assert keys == sorted(keys, reverse=True)
        # and the fourth entry is the position of the tile's first row, plus one (0 stands for "not given")
        assert [p for *_, p in ordered[:n]] == [seg_starts[seg] + first - starts[seg] + 1 for seg, first, _, _ in ordered[:n]]


def test_program_sizes_are_powers_of_two_then_multiples_of_64():
    assert [_bucket(n) for n in (0, 1, 2, 3, 5, 33, 64, 65, 128, 129, 2048)] == [0, 1, 2, 4, 8, 64, 64, 128, 128, 192, 2048]
    assert all(_bucket(n) >= n for n in range(1, 500))


def test_workspace_buffers_are_stable_for_programs_and_bounded_for_other_steps():
    import torch
    from runtime.engine.context import Workspace
    ws = Workspace(torch.device("cpu"))
    # captured programs: the same tensor for the same (name, shape, dtype), alive until its last owner goes
    a = ws.get("x", (4, 8), torch.float32, owner="p1")
    assert ws.get("x", (4, 8), torch.float32, owner="p1") is a
    assert ws.get("x", (4, 8), torch.float32, owner="p2") is a
    b = ws.get("x", (6, 8), torch.float32, owner="p2")
    assert b is not a and b.shape == (6, 8)
    ws.release("p1")
    assert ws.get("x", (4, 8), torch.float32, owner="p2") is a
    ws.release("p2")
    assert ws.bytes() == 0
    # other steps: one buffer per name that only grows; smaller requests are views of it
    big = ws.get("y", (10, 3), torch.float32)
    small = ws.get("y", (4, 3), torch.float32)
    assert small.shape == (4, 3) and small.is_contiguous() and small.data_ptr() == big.data_ptr()
    bigger = ws.get("y", (11, 3), torch.float32)
    assert bigger.shape == (11, 3) and ws.bytes() == 15 * 3 * 4      # grown by half, the old one dropped
    assert ws.get("y", (2, 5), torch.float32).shape == (2, 5)       # another trailing shape: another buffer
    assert ws.get("z", (7,), torch.int32, zeroed=True).sum() == 0
