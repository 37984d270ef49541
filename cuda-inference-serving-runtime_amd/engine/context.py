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


class StepArray:
    """The interface of a per-step list that a part wants every step's metadata to carry, beside what every step
    has (tokens, positions, segments, slots, block tables).  The step function lays such arrays out behind its own,
    fills them on the host with the rest of the metadata and uploads everything in one copy; it never looks at what
    they mean.  A part asks for one with `StepContext.step_array` (or names it beforehand in `step_arrays()`); from
    then on every step carries it.  Implementations are small frozen dataclasses (they are dictionary keys):

      words(rows, segments) -> int         int32 words for a step padded to that many rows and segments
      launch_value(batch) -> int | None    what of the batch the part's launches depend on beside the array's
                                           contents (the step function rounds it up and makes it part of the key
                                           of a captured program); None: nothing
      fill(out, batch, value) -> None      write the array (a NumPy int32 view of `words` entries) for `batch`;
                                           `value` is the launch value, rounded up under a captured program
    """


@dataclass
class Batch:
    """A step's batch as the host sees it, for StepArray implementations."""
    counts: list          # new tokens of each segment
    starts: list          # position of each segment's first new token
    first_row: object     # int32 [segments]: row of each segment's first token
    decode_only: bool     # every segment brings exactly one token
    launch_values: dict   # StepArray -> its launch value for this step


class StepContext:
    def __init__(self, runner):
        self.runner = runner
        self.cache = runner.cache
        self.dtype = runner.model.dtype
        self.device = runner.device
        self.scratch = runner.scratch   # the ScratchPool that products of this step use (ops.* take it as `scratch`)
        self.n_rows = self.n_segments = 0
        self.tokens = self.positions = self.seg_of_row = self.logit_rows = None
        self.seg_start = self.seg_first_pos = self.state_slots = None
        self.token_source = None  # int32 [T]: state slot whose device-side picked token a row takes, or -1
        self.kv = []
        self.segments = []        # host: [(request, start, count)]
        self.max_context = 0      # host: largest position + 1 among the rows
        self.decode_only = False  # host: every segment brings exactly one token
        self.span_hint = 0        # host: context length that sizes attention launches (a bucket under capture)
        self.arrays = {}          # StepArray -> (int32 device view, launch value): what parts asked the metadata to carry
        self.batch = None         # host: the Batch that the step arrays were filled from
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

    def step_array(self, array):
        """(int32 device tensor, launch value) of a StepArray.  The step's metadata holds every array asked for
        before; a new one is built and uploaded here once and travels with the metadata from the next step on."""
        got = self.arrays.get(array)
        if got is None:
            if self.capturing:
                raise RuntimeError(f"the step array {array!r} was first asked for under graph capture")
            value = array.launch_value(self.batch)
            self.batch.launch_values[array] = value
            host = np.zeros(array.words(self.n_rows, self.n_segments), dtype=np.int32)
            array.fill(host, self.batch, value)
            got = self.arrays[array] = (torch.from_numpy(host).to(self.device, non_blocking=False), value)
            self.runner.carry(array)
        return got

    def add_product(self, a, w, residual):
        """residual += a . w^T, in place.  Where the product is cut along its inner size and the norm that reads the
        residual next can add the slices itself (`next_norm`), they are left to it: one kernel fewer."""
        if getattr(self.next_norm, "adds_partials", False):
            partials = ops.gemm_unfinished(a, w, residual, scratch=self.scratch)
            if partials is not None:
                self.leave_unfinished(residual, partials)
                return residual
        return ops.gemm(a, w, residual, residual=residual, scratch=self.scratch)

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
