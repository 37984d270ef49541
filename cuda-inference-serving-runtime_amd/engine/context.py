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
        self.fixed_splits = None  # set when the step runs as a captured program

    def buffer(self, name, shape, dtype):
        return self.runner.workspace.get(name, shape, dtype)

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

    def bytes(self):
        return sum(b.numel() * b.element_size() for b in self.buffers.values())

    def clear(self):
        self.buffers.clear()
