"""The step function.

`ModelRunner.step(entries)` takes a batch of (request, its next tokens, wanted
places), prompt portions beside single decoded tokens, cut anywhere; reserves
cache slots for the new tokens; runs the model on exactly those tokens as one
batch against the cache; and returns the float logits at the wanted places, in
the order of the entries and of their `want` lists.

The reference's step takes exactly one token per request and returns logits for
every row (runtime/model.py:86-120); its order of checks is kept: batch shape,
context limit, token range, page preflight, then execution
(runtime/model.py:93-102).
"""
import gc
from dataclasses import dataclass, field
from typing import List, Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..kernels import ops
from .context import Batch, GroupView, StepContext, Workspace


@dataclass
class StepEntry:
    request: object
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)  # indices into `tokens` whose logits are returned
    pending: bool = False   # its one token is the one last picked for it, still only on the device (ModelRunner.pick)


class PickedTokens:
    """Tokens picked on the device for some requests, on their way to the host."""

    def __init__(self, host, event, requests, slots):
        self.host, self.event, self.requests, self.slots = host, event, requests, slots

    def tokens(self):
        """The token of each request, in the order of the logits they were picked from (waits for the copy)."""
        self.event.synchronize()
        return self.host[self.slots].tolist()


_TORCH_OF = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def _bucket(n):
    """Sizes that captured programs are padded to: powers of two up to 64, then multiples of 64."""
    if n <= 0:
        return 0
    return 1 << (n - 1).bit_length() if n <= 64 else -(-n // 64) * 64


class ModelRunner:
    def __init__(self, model, n_pages, page_size=16, max_requests=64, device="cuda:0", execution="eager", program_capacity=64):
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU: the engine runs on an MI355X only and has no CPU path")
        # fail now if the kernels are missing; a first call builds what this model's parts say they need, all at once
        ops.prepare(model.kernel_units())
        if execution not in ("eager", "graph"):
            raise ValueError(f"execution {execution!r} is not eager or graph")
        self.model = model
        self.execution = execution
        # captured programs, least recently used first.  A serving workload in portions makes a few dozen keys (rows,
        # segments and wanted rows in buckets, contexts in powers of two); an evicted program costs a synchronisation and
        # a capture when its key comes back, so the capacity is well above that and `report()` counts what happened.
        self.programs, self.program_capacity = {}, int(program_capacity)
        self.counters = {"steps": 0, "eager_steps": 0, "captures": 0, "replays": 0, "evictions": 0, "layouts": 0}
        self.device = torch.device(device)
        self.stream = torch.cuda.current_stream(self.device)   # every step and every release is ordered on this stream
        self.page_size = page_size
        self.max_requests = max_requests
        dtype = model.dtype

        def allocate_pages(shape):
            return torch.zeros(shape, dtype=dtype, device=self.device)

        def allocate_state(slots, shape, dt):
            return torch.zeros((slots, *shape), dtype=_TORCH_OF[dt], device=self.device)

        self.cache = CacheManager(model.cache_needs(), n_pages, page_size, max_requests,
                                  state_needs=model.state_needs(), allocate_pages=allocate_pages,
                                  allocate_state=allocate_state, copy_pages=self._copy_pages,
                                  zero_state=lambda t, s: t[s].zero_(),
                                  copy_state=lambda t, a, b: t[b].copy_(t[a]))
        self.workspace = Workspace(self.device)
        self.scratch = ops.ScratchPool()   # what products need beyond their operands (never shared with another runner)
        self.max_context = model.max_positions
        self.table_width = -(-self.max_context // page_size)
        self._staging = []
        self._staging_next = 0
        self._layouts = {}
        # host copies of the block tables by state slot, with the stamp of the table they were made from
        self._table_mirror = [(np.full((max_requests, self.table_width), -1, dtype=np.int32), [None] * max_requests)
                              for _ in self.cache.groups]
        # the step arrays that parts have asked every step's metadata to carry (context.StepArray), in layout order
        self.carried = list(dict.fromkeys(model.step_arrays()))
        self.steps = 0
        # the token last picked on the device for each request, by state slot, and its copies on the way to the host
        self.picked = torch.zeros(max_requests, dtype=torch.int32, device=self.device)
        self._picked_host = [[torch.zeros(max_requests, dtype=torch.int32, pin_memory=True), None] for _ in range(4)]
        self._picked_next = 0
        self._has_picked = set()
        self._last_wanted = None  # (requests, state slots on the host, state slots on the device) of the last step's logits
        self._failed = set()      # requests whose state a failed step may have changed: they can only be released

    # -- requests -------------------------------------------------------------
    def create(self, request):
        return self.cache.create(request)

    def fork(self, source, target):
        return self.cache.fork(source, target)

    def release(self, request):
        # later work that reuses the pages runs on the same stream, after every reader
        self.cache.release(request)
        self._has_picked.discard(request)
        self._failed.discard(request)

    def length(self, request):
        return self.cache.length(request)

    def _copy_pages(self, group, copies):
        src = torch.tensor([c[0] for c in copies], dtype=torch.int32, device=self.device)
        dst = torch.tensor([c[1] for c in copies], dtype=torch.int32, device=self.device)
        ops.page_copy(group.storage, src, dst, group.need.slabs(len(group.sites)), group.pool.n_pages)

    def carry(self, array):
        """From the next step on, every step's metadata holds the step array `array`."""
        if array not in self.carried:
            self.carried.append(array)

    # -- the step -------------------------------------------------------------
    def check(self, entries):
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        vocab, limit, lengths = self.model.vocab_size, self.max_context, self.cache.lengths
        for e in entries:
            if e.request in seen:
                raise ValueError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if e.request not in lengths:
                raise KeyError(f"unknown request {e.request!r}")
            if e.request in self._failed:
                raise RuntimeError(f"request {e.request!r} was in a step that failed after its kernels may have changed its "
                                   f"state: it cannot be stepped again, only released")
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.request!r} brings no tokens")
            if lengths[e.request] + n > limit:
                raise ValueError(f"request {e.request!r} exceeds the context limit of {limit}")
            if e.pending:
                if n != 1 or e.request not in self._has_picked:
                    raise ValueError(f"request {e.request!r} has no one token picked on the device")
            elif n == 1:
                if not 0 <= int(e.tokens[0]) < vocab:
                    raise ValueError(f"request {e.request!r} has a token outside the vocabulary")
            else:
                # a portion: checked as an array, which the metadata then takes as it is (a list is converted once)
                ids = np.asarray(e.tokens)
                if ids.ndim != 1 or ids.dtype.kind not in "iu" or ids.min() < 0 or ids.max() >= vocab:
                    raise ValueError(f"request {e.request!r} has a token outside the vocabulary")
                e.tokens = ids.astype(np.int32, copy=False)
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise ValueError(f"request {e.request!r} wants a place outside its tokens")

    def step(self, entries: List[StepEntry]):
        """Float logits [sum(len(want)), vocab] on the GPU (valid until the next step)."""
        if torch.cuda.current_stream(self.device) != self.stream:
            # pages that a request gave back are used again without a wait, and copies on write are queued before the
            # kernels that need them: both are right only because everything runs on one stream, in order
            raise RuntimeError("a step must be launched on the stream that its runner was made on")
        self.check(entries)
        # slots first, the requests' lengths only once the step is launched (the reference commits after it has
        # submitted the work, runtime/execution.py:125-126): a step that fails on the way (a shape that a kernel
        # refuses, no memory for a buffer) leaves the length and the pages of every request where they stood.  With a
        # cache of keys and values only, that is the whole of a request and the step can be tried again (what its
        # kernels wrote lies beyond the lengths and is written again).  A per-request state is another matter: kernels
        # launched before the failure may have updated it, and nothing keeps the old one, so the requests of such a
        # model are marked failed and can only be released.
        done = self.cache.append_many([(e.request, len(e.tokens)) for e in entries], commit=False)  # OutOfPages changes nothing
        try:
            if self.execution == "graph":
                logits = self._run_program(self._program_key(entries, done), entries, done)
            else:
                ctx = self._context(entries, done)
                logits = self._forward(ctx, any(e.pending for e in entries))
                self.counters["eager_steps"] += 1
        except BaseException:
            self.cache.abandon(done)
            self._last_wanted = None          # the metadata of a step that never ran: nothing to pick from
            if self.cache.state_needs:
                self._failed.update(e.request for e in entries)
            raise
        self.cache.commit(done)
        self.steps += 1
        self.counters["steps"] += 1
        if logits is None:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return logits

    def _forward(self, ctx, take):
        if take:   # rows whose token is still only on the device get it from there
            ops.take_tokens(ctx.tokens, ctx.token_source, self.picked)
        return self.model.forward(ctx)

    def pick(self, sampler, logits, params):
        """Pick a token for each row of the last step's logits and leave it on the device, where a later
        step takes it from (StepEntry.pending); the host does not wait.  Returns PickedTokens, to be read
        before three more calls of this function."""
        if self._last_wanted is None:
            raise ValueError("the logits are not those of the last step (it failed, or none has run)")
        requests, slots, where = self._last_wanted
        if logits.shape[0] != len(requests):
            raise ValueError("the logits are not those of the last step")
        sampler.pick(logits, params, out=self.picked, index=where)
        self._has_picked.update(requests)
        entry = self._picked_host[self._picked_next % 4]
        self._picked_next += 1
        entry[0].copy_(self.picked, non_blocking=True)
        if entry[1] is None:
            entry[1] = torch.cuda.Event()
        entry[1].record()
        return PickedTokens(entry[0].numpy(), entry[1], requests, slots)

    _FIXED = 9   # arrays of the metadata before the cache groups'

    def _width(self, context):
        """Block-table entries a step carries per request: what its longest context needs, in steps of 16 entries,
        not what the context limit would need (at a limit of 128k that would be megabytes a step)."""
        need = -(-int(context) // self.page_size)
        return min(self.table_width, -(-need // 16) * 16)

    def _layout(self, T, S, R, W, carried):
        """Offsets of the packed int32 metadata: tokens, positions, seg_of_row, seg_start, seg_first_pos,
        state_slots, logit_rows, token_source, logit_slots, then per group slots and tables, then the step arrays
        that parts asked for."""
        G = len(self.cache.groups)
        sizes = [T, T, T, S + 1, S, S, R, T, R] + [T, S * W] * G + [int(array.words(T, S)) for array in carried]
        self.counters["layouts"] += 1
        return np.concatenate(([0], np.cumsum(sizes))).astype(np.int64)

    def _table_rows(self, g, done, W):
        """int32 [len(done), W]: the first W entries of the block tables of the step's requests in group g.  A host copy of every
        live request's table is kept by state slot and rewritten only when the table has changed (a new
        page, a page the window has passed, a copy-on-write), so a step costs one gather."""
        group = self.cache.groups[g]
        mirror, stamps = self._table_mirror[g]
        for d in done:
            stamp = group.versions[d.request]
            if stamps[d.state_slot] != stamp:
                table = group.tables[d.request]
                mirror[d.state_slot, :len(table)] = table
                mirror[d.state_slot, len(table):] = -1
                stamps[d.state_slot] = stamp
        return mirror[[d.state_slot for d in done], :W]

    def _launch_values(self, done):
        """What the parts' launches depend on beside rows, segments and contexts: the launch value of every carried
        step array that has one (context.StepArray), for this batch."""
        batch = Batch([d.count for d in done], [d.start for d in done], None, all(d.count == 1 for d in done), {})
        for array in self.carried:
            batch.launch_values[array] = array.launch_value(batch)
        return batch.launch_values

    def _context(self, entries, done, pad=None, device_buffer=None, launch_values=None, context=None):
        """Build the step's metadata on the host, upload it in one copy and wrap it.
        `pad` = (T, S, R) pads the batch with inert rows (for captured programs):
        token 0 at position 0, no segment, no cache slot.  `launch_values`: those of the captured program
        (rounded up), instead of the batch's own."""
        counts = [d.count for d in done]
        starts = [d.start for d in done]
        n_rows, n_seg = sum(counts), len(entries)
        n_want = sum(len(e.want) for e in entries)
        T, S, R = pad if pad is not None else (n_rows, n_seg, n_want)
        # the longest context of the step (a captured program brings the bound of its bucket) sizes the block tables
        longest = max(s + c for s, c in zip(starts, counts))
        W, G, F = self._width(longest if context is None else context), len(self.cache.groups), self._FIXED
        carried = tuple(self.carried)
        layout = (T, S, R, W, carried)
        offsets = self._layouts.get(layout)
        if offsets is None:
            offsets = self._layouts[layout] = [int(x) for x in self._layout(T, S, R, W, carried)]
        total = offsets[-1]
        host = self._stage(total)
        arr = host.numpy()
        tokens, positions, seg_of_row, seg_start, seg_first, state_slots, logit_rows, token_source, logit_slots = (
            arr[offsets[i]:offsets[i + 1]] for i in range(F))
        decode_only = n_rows == n_seg
        slot_of = [d.state_slot for d in done]
        wanted_seg = [s for s, e in enumerate(entries) for _ in e.want]
        if decode_only:
            first_row = np.arange(n_seg, dtype=np.int32)
            tokens[:n_rows] = [e.tokens[0] for e in entries]
            positions[:n_rows] = starts
            seg_of_row[:n_rows] = first_row
            wanted = wanted_seg
        else:
            first_row = np.concatenate(([0], np.cumsum(counts[:-1]))).astype(np.int32)
            tokens[:n_rows] = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
            seg_of_row[:n_rows] = np.repeat(np.arange(n_seg, dtype=np.int32), counts)
            positions[:n_rows] = np.arange(n_rows, dtype=np.int32) + np.repeat(np.asarray(starts, dtype=np.int32) - first_row, counts)
            wanted = [int(first_row[s]) + int(w) for s, e in enumerate(entries) for w in e.want]
        seg_start[:n_seg] = first_row
        seg_start[n_seg:] = n_rows
        seg_first[:n_seg] = starts
        state_slots[:n_seg] = slot_of
        logit_rows[:n_want] = wanted
        wanted_slots = [slot_of[s] for s in wanted_seg]
        logit_slots[:n_want] = wanted_slots
        token_source[:] = -1
        pending = [e.pending for e in entries]
        if decode_only and all(pending):
            token_source[:n_rows] = slot_of
        elif any(pending):
            for s, e in enumerate(entries):
                if e.pending:
                    token_source[first_row[s]] = slot_of[s]
        if pad is not None:      # the inert rest: token 0 at position 0, no segment, no slot, no table
            tokens[n_rows:] = 0
            positions[n_rows:] = 0
            seg_of_row[n_rows:] = -1
            seg_first[n_seg:] = 0
            state_slots[n_seg:] = 0
            logit_rows[n_want:] = 0
            logit_slots[n_want:] = -1
        for g in range(G):
            slots = arr[offsets[F + 2 * g]:offsets[F + 1 + 2 * g]]
            tables = arr[offsets[F + 1 + 2 * g]:offsets[F + 2 + 2 * g]].reshape(S, W)
            if decode_only:
                slots[:n_rows] = [d.slots[g][0] for d in done]
            else:
                slots[:n_rows] = np.concatenate([np.asarray(d.slots[g], dtype=np.int32) for d in done])
            tables[:n_seg] = self._table_rows(g, done, W)
            if pad is not None:
                slots[n_rows:] = -1
                tables[n_seg:] = -1
        # what the parts asked for: first every launch value, then the arrays (one may read another's value)
        batch = Batch(counts, starts, first_row, decode_only, {})
        for array in carried:
            own = array.launch_value(batch)
            batch.launch_values[array] = own if launch_values is None or own is None else launch_values.get(array, 0)
        for i, array in enumerate(carried):
            array.fill(arr[offsets[F + 2 * G + i]:offsets[F + 1 + 2 * G + i]], batch, batch.launch_values[array])
        dev = self._upload(host, total, device_buffer)

        def view(i, shape=None):
            t = dev[offsets[i]:offsets[i + 1]]
            return t if shape is None else t.view(shape)

        ctx = StepContext(self)
        ctx.n_rows, ctx.n_segments = T, S
        ctx.tokens, ctx.positions, ctx.seg_of_row = view(0), view(1), view(2)
        ctx.seg_start, ctx.seg_first_pos, ctx.state_slots, ctx.logit_rows = view(3), view(4), view(5), view(6)
        ctx.token_source = view(7)
        ctx.kv = [GroupView(view(F + 2 * g), view(F + 1 + 2 * g, (S, W)), self.page_size, W) for g in range(G)]
        ctx.batch = batch
        ctx.arrays = {array: (view(F + 2 * G + i), batch.launch_values[array]) for i, array in enumerate(carried)}
        self._last_wanted = ([entries[s].request for s in wanted_seg], wanted_slots, view(8)[:n_want])
        ctx.segments = [(d.request, d.start, d.count) for d in done]
        ctx.max_context = ctx.span_hint = longest
        ctx.decode_only = decode_only
        return ctx

    def _stage(self, n):
        """A pinned host buffer of at least n int32, not in flight."""
        slot = self._staging_next % 4
        self._staging_next += 1
        while len(self._staging) <= slot:
            self._staging.append(None)
        entry = self._staging[slot]
        if entry is None or entry[0].numel() < n:
            cap = max(4096, 1 << (n - 1).bit_length())
            entry = [torch.empty(cap, dtype=torch.int32, pin_memory=True),
                     torch.empty(cap, dtype=torch.int32, device=self.device), None]
            self._staging[slot] = entry
        if entry[2] is not None:
            entry[2].synchronize()  # the copy that last read this buffer is over
        self._current = entry
        return entry[0]

    def _upload(self, host, n, device_buffer=None):
        entry = self._current
        target = entry[1] if device_buffer is None else device_buffer
        target[:n].copy_(host[:n], non_blocking=True)
        entry[2] = torch.cuda.Event()
        entry[2].record()
        return target

    # -- captured programs ------------------------------------------------------------
    def _program_key(self, entries, done):
        """What the launches of a step depend on: the padded numbers of rows, segments and
        wanted rows, whether every segment brings one token, the context length rounded up
        to a power of two (parts size their launches by it), whether tokens are taken from the device, and the
        launch values of the step arrays that parts carry (rounded up; those that are zero are left out, so that
        an array which joins later changes no key of a step it has nothing to say about).  Steps with the same key
        replay one captured graph; only the metadata they read differs."""
        rows = sum(d.count for d in done)
        wanted = sum(len(e.want) for e in entries)
        decode_only = all(d.count == 1 for d in done)
        context = 1 << (max(d.start + d.count for d in done) - 1).bit_length()
        values = tuple((array, _bucket(value)) for array, value in self._launch_values(done).items() if value)
        return (_bucket(rows), _bucket(len(entries)), _bucket(wanted), decode_only, max(context, 256),
                any(e.pending for e in entries), values)

    def _run_program(self, key, entries, done):
        T, S, R, decode_only, context, take, values = key
        program = self.programs.get(key)
        if program is None:
            program = {"meta": None, "graph": None, "runs": 0, "carried": None}
            self.programs[key] = program
            while len(self.programs) > self.program_capacity:
                oldest = next(iter(self.programs))
                torch.cuda.synchronize()
                del self.programs[oldest]
                self.workspace.release(oldest)
                self.counters["evictions"] += 1
        else:
            self.programs[key] = self.programs.pop(key)  # most recently used last
        if program["carried"] != self.carried:
            # a part asked for a step array that the metadata did not hold yet: lay it out again
            torch.cuda.synchronize()
            words = int(self._layout(T, S, R, self._width(context), tuple(self.carried))[-1])
            program.update(meta=torch.zeros(words, dtype=torch.int32, device=self.device),
                           graph=None, runs=0, carried=list(self.carried))
        ctx = self._context(entries, done, pad=(T, S, R), device_buffer=program["meta"], launch_values=dict(values), context=context)
        ctx.owner = key
        ctx.span_hint = context   # launch shapes inside a captured program depend on the key only
        ctx.decode_only = decode_only
        if program["graph"] is None and program["runs"] >= 1 and program["carried"] == self.carried:
            # the first run was eager and allocated every buffer; capture launches nothing
            # nothing but kernel launches may happen while the stream records: keep the garbage
            # collector from freeing device objects (other graphs, events) in the middle of it
            graph = torch.cuda.CUDAGraph()
            collecting = gc.isenabled()
            gc.disable()
            ctx.capturing = True
            try:
                with torch.cuda.graph(graph, capture_error_mode="thread_local"):
                    program["logits"] = self._forward(ctx, take)
            finally:
                if collecting:
                    gc.enable()
            program["graph"] = graph
            self.counters["captures"] += 1
        if program["graph"] is not None:
            program["graph"].replay()
            logits = program["logits"]
            self.counters["replays"] += 1
        else:
            logits = self._forward(ctx, take)
            self.counters["eager_steps"] += 1
        program["runs"] += 1
        wanted = sum(len(e.want) for e in entries)
        if logits is None:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return logits[:wanted]

    # -- what it holds ------------------------------------------------------------------
    def report(self):
        """Counters and bytes of the step function, as the reference's executor reports its own
        (runtime/execution.py:156-165: captures, replays, workspace and staging bytes; runtime/device.py:81-112):
        steps run, how many kernel by kernel, programs captured, replayed and evicted, metadata layouts made;
        bytes of the intermediate buffers, of the products' scratch memory, of the pinned and device staging of the
        metadata, of the captured programs' own metadata; the step arrays that parts asked for; the cache report."""
        staging = sum(e[0].numel() * 4 for e in self._staging if e is not None)
        return {
            **self.counters,
            "execution": self.execution,
            "programs": len(self.programs), "program_capacity": self.program_capacity,
            "workspace_bytes": self.workspace.bytes(), "scratch_bytes": self.scratch.bytes(),
            "staging_host_bytes": staging, "staging_device_bytes": staging,
            "program_metadata_bytes": sum(p["meta"].numel() * 4 for p in self.programs.values() if p["meta"] is not None),
            "step_arrays": [repr(a) for a in self.carried],
            "cache": self.cache.report(),
        }
