"""What a step hands to the parts: the rows of the batch and where they live.

A step's batch is a list of segments, one per request in the step: `count`
new tokens at positions start..start+count-1.  Flattened, that gives T token
rows.  All per-row and per-segment metadata sits in int32 device tensors; parts
never look at request identities.
"""
from dataclasses import dataclass

import numpy as np
import torch

from ..kernels import ops


@dataclass
class GroupView:
    """A cache group as one step sees it."""
    slots: torch.Tensor       # int32 [T]: physical token slot each row's key/value is written to (-1: none)
    tables: torch.Tensor      # int32 [S, W]: block table of each segment's request
    page_size: int
    width: int


def fill_tasks(tasks, counts, rows_per_tile, starts=None, skip_single=False):
    """Write (segment, first row, rows, p) for tiles of at most `rows_per_tile` consecutive
    rows of one segment into the int32 array tasks[n, 4]; returns how many were written.
    With `starts` (the position of each segment's first row) p is the position of the tile's
    first row plus one (a segment's rows have consecutive positions, so a kernel that reads p need
    not wait for the positions array; p = 0 says "not given"), and the tiles are ordered by the
    number of keys they attend to, most first: blocks are handed out in this order, and the
    long ones must not be the last to start.  `skip_single`: segments of one row get no tile
    (they are attended to by a launch of their own)."""
    n = row = 0
    for seg, count in enumerate(counts):
        tiles = 0 if skip_single and count == 1 else -(-count // rows_per_tile)
        firsts = np.arange(tiles, dtype=np.int64) * rows_per_tile
        tasks[n:n + tiles, 0] = seg
        tasks[n:n + tiles, 1] = row + firsts
        tasks[n:n + tiles, 2] = np.minimum(rows_per_tile, count - firsts)
        tasks[n:n + tiles, 3] = 0 if starts is None else int(starts[seg]) + firsts + 1
        n += tiles
        row += count
    if starts is not None and n > 1:
        first_row = np.concatenate(([0], np.cumsum(counts)))[tasks[:n, 0]]
        keys = np.asarray(starts, dtype=np.int64)[tasks[:n, 0]] + (tasks[:n, 1] - first_row) + tasks[:n, 2]
        tasks[:n] = tasks[:n][np.argsort(-keys, kind="stable")]
    return n


class StepContext:
    def __init__(self, runner):
        self.runner = runner
        self.cache = runner.cache
        self.dtype = runner.model.dtype
        self.device = runner.device
        self.n_rows = self.n_segments = 0
        self.tokens = self.positions = self.seg_of_row = self.logit_rows = None
        self.seg_start = self.seg_first_pos = self.state_slots = None
        self.token_source = None  # int32 [T]: state slot whose device-side picked token a row takes, or -1
        self.kv = []
        self.segments = []        # host: [(request, start, count)]
        self.max_context = 0      # host: largest position + 1 among the rows
        self.decode_only = False  # host: every segment brings exactly one token
        self.span_hint = 0        # host: context length that sizes attention launches (a bucket under capture)
        self.tasks = {}           # rows per tile -> int32 [n, 4] task list on the device
        self.single_rows = None   # int32 [S]: the rows of the one-token segments of a mixed step, then -1
        self.n_single = 0         # host: how many entries of single_rows a launch of their own covers (0: none)
        # A product whose partial sums are still to be added to the residual stream: (rows tensor, partials), set by a
        # part that was told it may (`next_norm`), taken by the norm that reads the rows next (or settled)
        self.unfinished = None
        self.next_norm = None     # the norm that reads the residual stream after the block that runs now, if known
        self.capturing = False    # the step is being recorded into a graph: launches only
        self.owner = None         # key of the captured program this step belongs to, if any

    def buffer(self, name, shape, dtype):
        """A device buffer for an intermediate result of this step (stable across the replays of a
        captured program; otherwise valid until the next step)."""
        return self.runner.workspace.get(name, shape, dtype, owner=self.owner)

    def attention_tasks(self, rows_per_tile):
        """int32 [n, 4] on the device: (segment, first row, rows, 0) for tiles of at most
        `rows_per_tile` consecutive rows of one segment; entries with segment -1 are no tile.
        The step's metadata holds the list for every tiling asked for before; a new tiling
        is built and uploaded here once and travels with the metadata from the next step on."""
        tasks = self.tasks.get(rows_per_tile)
        if tasks is None:
            if self.capturing:
                raise RuntimeError(f"a task list of {rows_per_tile} rows a tile was first asked for under graph capture")
            counts = [count for _, _, count in self.segments]
            host = np.full((sum(-(-c // rows_per_tile) for c in counts), 4), -1, dtype=np.int32)
            fill_tasks(host, counts, rows_per_tile, [start for _, start, _ in self.segments], skip_single=self.n_single > 0)
            tasks = torch.from_numpy(host).to(self.device, non_blocking=False)
            self.tasks[rows_per_tile] = tasks
            if rows_per_tile not in self.runner.task_tilings:
                self.runner.task_tilings.append(rows_per_tile)
        return tasks

    def add_product(self, a, w, residual):
        """residual += a . w^T, in place.  Where the product is cut along its inner size and the norm that reads the
        residual next can add the slices itself (`next_norm`), they are left to it: one kernel fewer."""
        if getattr(self.next_norm, "adds_partials", False):
            partials = ops.gemm_unfinished(a, w, residual)
            if partials is not None:
                self.leave_unfinished(residual, partials)
                return residual
        return ops.gemm(a, w, residual, residual=residual)

    def leave_unfinished(self, rows, partials):
        """`rows` lack the partial sums `partials` (ops.gemm_unfinished); whoever reads them next adds them."""
        if self.unfinished is not None:
            raise RuntimeError("a second unfinished product before the first was added")
        self.unfinished = (rows, partials)

    def take_unfinished(self, rows):
        """The partial sums that `rows` lack, for a kernel that adds them itself; None if there are none."""
        if self.unfinished is None:
            return None
        if self.unfinished[0].data_ptr() != rows.data_ptr():
            raise RuntimeError("the unfinished product belongs to other rows")
        partials, self.unfinished = self.unfinished[1], None
        return partials

    def settle(self, rows):
        """Add what `rows` lack, if anything: before a reader that cannot do it itself."""
        partials = self.take_unfinished(rows)
        if partials is not None:
            ops.add_partials(rows, partials)

    def attend(self, q, q_row_stride, kcache, vcache, view, out, heads, kv_heads, head_dim, window, scale, defer_merge=None):
        """out[r] = attention of row r's queries over its request's cache.  With `defer_merge` (see
        ModelRunner.attention) the result may come back unmerged instead: (partial outputs, statistics, splits) for
        ops.gemm_merged, `out` untouched; None means `out` holds the result."""
        return self.runner.attention(self, q, q_row_stride, kcache, vcache, view, out, heads, kv_heads, head_dim, window, scale,
                                     defer_merge=defer_merge)


class Workspace:
    """Named device buffers for a step's intermediate results.

    A captured program needs buffers whose addresses never change: it asks with its key as `owner` and gets
    one buffer per (name, shape, dtype), shared with every other program that asks for the same; a buffer
    lives until its last owner is released.  Steps that are not captured (owner None) share one buffer per
    name that only grows, and get a view of its first rows."""

    def __init__(self, device):
        self.device = device
        self.owned = {}      # (name, shape, dtype) -> [tensor, set of owners]
        self.growing = {}    # (name, trailing shape, dtype) -> tensor

    def get(self, name, shape, dtype, owner=None, zeroed=False):
        shape = tuple(int(d) for d in shape)
        make = torch.zeros if zeroed else torch.empty
        if owner is not None:
            entry = self.owned.get((name, shape, dtype))
            if entry is None:
                entry = self.owned[(name, shape, dtype)] = [make(shape, dtype=dtype, device=self.device), set()]
            entry[1].add(owner)
            return entry[0]
        key = (name, shape[1:], dtype)
        buf = self.growing.get(key)
        if buf is None or buf.shape[0] < shape[0]:
            rows = shape[0] if buf is None else max(shape[0], buf.shape[0] * 3 // 2)
            # the old buffer goes back to the allocator, which hands it out again only behind the work
            # already queued on this stream
            buf = self.growing[key] = make((rows, *shape[1:]), dtype=dtype, device=self.device)
        return buf[:shape[0]]

    def release(self, owner):
        """Forget a program: buffers that no other program uses are freed."""
        for key in [k for k, (_, owners) in self.owned.items() if owner in owners]:
            owners = self.owned[key][1]
            owners.discard(owner)
            if not owners:
                del self.owned[key]

    def bytes(self):
        tensors = [t for t, _ in self.owned.values()] + list(self.growing.values())
        return sum(t.numel() * t.element_size() for t in tensors)

    def clear(self):
        self.owned.clear()
        self.growing.clear()
