"""What a step hands to the parts: the rows of the batch and where they live.

A step's batch is a list of segments, one per request in the step: `count`
new tokens at positions start..start+count-1.  Flattened, that gives T token
rows.  All per-row and per-segment metadata sits in int32 device tensors; parts
never look at request identities.
"""
from dataclasses import dataclass

import torch

from ..kernels import ops


@dataclass
class GroupView:
    """A cache group as one step sees it."""
    slots: torch.Tensor       # int32 [T]: physical token slot each row's key/value is written to (-1: none)
    tables: torch.Tensor      # int32 [S, W]: block table of each segment's request
    page_size: int
    width: int


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
        self._tasks = {}

    def buffer(self, name, shape, dtype):
        return self.runner.workspace.get(name, shape, dtype)

    def attention_tasks(self, rows_per_tile):
        """int32 [n, 4] on the device: (segment, first row, rows, 0) for tiles of at most
        `rows_per_tile` consecutive rows of one segment."""
        tasks = self._tasks.get(rows_per_tile)
        if tasks is None:
            items, row = [], 0
            for seg, (_, _, count) in enumerate(self.segments):
                for first in range(0, count, rows_per_tile):
                    items.append((seg, row + first, min(rows_per_tile, count - first), 0))
                row += count
            tasks = torch.tensor(items, dtype=torch.int32).to(self.device, non_blocking=False)
            self._tasks[rows_per_tile] = tasks
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
