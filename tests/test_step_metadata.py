"""Host-side metadata of a step: the attention task lists and the sizes that captured programs pad to."""
import numpy as np

from runtime.kernels.attention import RowsLongestFirst, SingleRows, TileTasks, fill_tasks
from runtime.engine.context import Batch
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


def test_step_arrays_of_the_attention_kernels():
    """The two lists that the attention kernels ask every step to carry, filled from a batch as the step function does:
    the rows of the one-token segments of a mixed step (when one of them has a long context), and the tiles of the
    other segments (which then leave the one-token segments out)."""
    singles = SingleRows(split_from=100)
    tiles = TileTasks(4, singles)
    counts, starts = [1, 6, 1, 3], [150, 0, 20, 7]
    first_row = np.array([0, 1, 7, 8], dtype=np.int32)
    batch = Batch(counts, starts, first_row, False, {})
    assert singles.launch_value(batch) == 2 and tiles.launch_value(batch) is None
    assert singles.launch_value(Batch([1, 1], [150, 3], None, True, {})) == 0          # a step of single tokens only
    assert singles.launch_value(Batch([1, 6], [50, 0], None, False, {})) == 0          # short contexts: they stay tiles
    batch.launch_values[singles] = 4                                                    # (rounded up, as a captured program does)
    rows = np.full(singles.words(16, 8), 99, dtype=np.int32)
    singles.fill(rows, batch, 4)
    assert rows.tolist() == [0, 7, -1, -1, -1, -1, -1, -1]
    tasks = np.full(tiles.words(16, 8), 99, dtype=np.int32)
    tiles.fill(tasks, batch, None)
    tasks = tasks.reshape(-1, 4)
    real = tasks[tasks[:, 0] >= 0]
    assert sorted(map(tuple, real[:, :3])) == [(1, 1, 4), (1, 5, 2), (3, 8, 3)]          # no tile for segments 0 and 2
    assert (tasks[len(real):] == (-1, 0, 0, 0)).all()
    batch.launch_values[singles] = 0
    tiles.fill(tasks.reshape(-1), batch, None)
    assert sorted(tasks[tasks[:, 0] >= 0][:, 0].tolist()) == [0, 1, 1, 2, 3]


def test_rows_of_a_decode_step_longest_first():
    """The order in which an unsplit decode launch hands out its blocks: rows by keys, most first, rows of equal
    length in their own order, then the padding rows of a captured program; a mixed step lists every row in place."""
    order = RowsLongestFirst()
    starts = [5, 900, 17, 900, 0, 300]
    batch = Batch([1] * 6, starts, np.arange(6, dtype=np.int32), True, {})
    assert order.launch_value(batch) is None and order.words(8, 8) == 8
    out = np.full(8, -9, dtype=np.int32)
    order.fill(out, batch, None)
    assert out.tolist() == [1, 3, 5, 2, 0, 4, 6, 7]
    mixed = Batch([1, 4], [50, 0], np.array([0, 1], dtype=np.int32), False, {})
    out = np.full(5, -9, dtype=np.int32)
    order.fill(out, mixed, None)
    assert out.tolist() == [0, 1, 2, 3, 4]
