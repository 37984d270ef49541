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


def fill_tasks(tasks, counts, rows_per_tile, starts=None):
    """Write (segment, first row, rows, 0) for tiles of at most `rows_per_tile` consecutive
    rows of one segment into the int32 array tasks[n, 4]; returns how many were written.
    With `starts` (the position of each segment's first row) the tiles are ordered by the
    number of keys they attend to, most first: blocks are handed out in this order, and the
    long ones must not be the last to start."""
    n = row = 0
    for seg, count in enumerate(counts):
        tiles = -(-count // rows_per_tile)
        firsts = np.arange(tiles, dtype=np.int64) * rows_per_tile
        tasks[n:n + tiles, 0] = seg
        tasks[n:n + tiles, 1] = row + firsts
        tasks[n:n + tiles, 2] = np.minimum(rows_per_tile, count - firsts)
        tasks[n:n + tiles, 3] = 0
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
        self.kv = []
        self.segments = []        # host: [(request, start, count)]
        self.max_context = 0      # host: largest position + 1 among the rows
        self.decode_only = False  # host: every segment brings exactly one token
        self.span_hint = 0        # host: context length that sizes attention launches (a bucket under capture)
        self.tasks = {}           # rows per tile -> int32 [n, 4] task list on the device
        self.capturing = False    # the step is being recorded into a graph: launches only

    def buffer(self, name, shape, dtype):
        return self.runner.workspace.get(name, shape, dtype)

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
            fill_tasks(host, counts, rows_per_tile, [start for _, start, _ in self.segments])
            tasks = torch.from_numpy(host).to(self.device, non_blocking=False)
            self.tasks[rows_per_tile] = tasks
            if rows_per_tile not in self.runner.task_tilings:
                self.runner.task_tilings.append(rows_per_tile)
        return tasks

    def attend(self, q, q_row_stride, kcache, vcache, view, out, heads, kv_heads, head_dim, window, scale):
        """out[r] = attention of row r's queries over its request's cache."""
        self.runner.attention(self, q, q_row_stride, kcache, vcache, view, out, heads, kv_heads, head_dim, window, scale)


class Workspace:
    """Named device buffers with stable addresses, one per (name, shape, dtype)."""

    def __init__(self, device):
        self.device = device
        self.buffers = {}

    def get(self, name, shape, dtype):
        key = (name, tuple(shape), dtype)
        buf = self.buffers.get(key)
        if buf is None:
            buf = torch.empty(tuple(shape), dtype=dtype, device=self.device)
            self.buffers[key] = buf
        return buf

    def get_zeroed(self, name, shape, dtype):
        """A buffer that is zero when first handed out; its users leave it zero."""
        key = (name, tuple(shape), dtype)
        buf = self.buffers.get(key)
        if buf is None:
            buf = torch.zeros(tuple(shape), dtype=dtype, device=self.device)
            self.buffers[key] = buf
        return buf

    def bytes(self):
        return sum(b.numel() * b.element_size() for b in self.buffers.values())

    def clear(self):
        self.buffers.clear()
