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
import os
from dataclasses import dataclass, field
from typing import List, Sequence

import numpy as np
import torch

from ..cache import CacheManager, OutOfPages
from ..kernels import ops
from .context import GroupView, StepContext, Workspace, fill_tasks


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
    def __init__(self, model, n_pages, page_size=16, max_requests=64, device="cuda:0", execution="eager"):
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU: the engine runs on an MI355X only and has no CPU path")
        # fail now if the kernels are missing; a first call builds what this model needs, all at once
        ops.prepare([need.head_dim for need in model.cache_needs().values() if need is not None], model.dtype)
        if execution not in ("eager", "graph"):
            raise ValueError(f"execution {execution!r} is not eager or graph")
        self.model = model
        self.execution = execution
        self.programs, self.program_capacity = {}, 16
        self.block_tiles = None    # long portions through LDS-shared tiles of 64 x this items: None = by the number of blocks
        # long portions of long contexts through 32 x 32 tiles, 64 x this items a block (1, 2, 3, 4): None = by size, 0 = never
        self.square_tiles = int(os.environ["CISR_SQUARE_TILES"]) if os.environ.get("CISR_SQUARE_TILES") else None
        self.square_halves = None  # two halves a block in that form (even and odd steps): None = by the number of blocks, 1, 2
        self.tile_waves = int(os.environ.get("CISR_TILE_WAVES", "4"))   # wavefronts that share one tile's keys
        self.item_tiles = int(os.environ.get("CISR_ITEM_TILES", "2"))   # 16-item tiles a wave of long portions (small heads)
        # In a mixed step a decoded token is a tile whose keys one block walks; from this context on the
        # one-token segments get a launch of their own instead, which splits their keys over blocks
        self.split_single_from = 4096
        self.device = torch.device(device)
        self.page_size = page_size
        self.max_requests = max_requests
        dtype = model.dtype

        def allocate_kv(sites, pages, kv_heads, psize, head_dim):
            return torch.zeros((sites, 2, pages, kv_heads, psize, head_dim), dtype=dtype, device=self.device)

        def allocate_state(slots, shape, dt):
            return torch.zeros((slots, *shape), dtype=_TORCH_OF[dt], device=self.device)

        self.cache = CacheManager(model.cache_needs(), n_pages, page_size, max_requests,
                                  state_needs=model.state_needs(), allocate_kv=allocate_kv,
                                  allocate_state=allocate_state, copy_pages=self._copy_pages,
                                  zero_state=lambda t, s: t[s].zero_(),
                                  copy_state=lambda t, a, b: t[b].copy_(t[a]))
        self.workspace = Workspace(self.device)
        self.max_context = model.max_positions
        self.table_width = -(-self.max_context // page_size)
        self._staging = []
        self._staging_next = 0
        self._layouts = {}
        # host copies of the block tables by state slot, with the stamp of the table they were made from
        self._table_mirror = [(np.full((max_requests, self.table_width), -1, dtype=np.int32), [None] * max_requests)
                              for _ in self.cache.groups]
        self.task_tilings = []   # rows-per-tile values that mixers have asked task lists for
        self.steps = 0
        # the token last picked on the device for each request, by state slot, and its copies on the way to the host
        self.picked = torch.zeros(max_requests, dtype=torch.int32, device=self.device)
        self._picked_host = [[torch.zeros(max_requests, dtype=torch.int32, pin_memory=True), None] for _ in range(4)]
        self._picked_next = 0
        self._has_picked = set()
        self._last_wanted = None  # (requests, state slots on the host, state slots on the device) of the last step's logits

    # -- requests -------------------------------------------------------------
    def create(self, request):
        return self.cache.create(request)

    def fork(self, source, target):
        return self.cache.fork(source, target)

    def release(self, request):
        # later work that reuses the pages runs on the same stream, after every reader
        self.cache.release(request)
        self._has_picked.discard(request)

    def length(self, request):
        return self.cache.length(request)

    def _copy_pages(self, group, copies):
        src = torch.tensor([c[0] for c in copies], dtype=torch.int32, device=self.device)
        dst = torch.tensor([c[1] for c in copies], dtype=torch.int32, device=self.device)
        ops.page_copy(group.storage, src, dst, group.storage.shape[0] * 2, group.pool.n_pages)

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
        self.check(entries)
        # slots first, the requests' lengths only once the step is launched (the reference commits after it has
        # submitted the work, runtime/execution.py:125-126): a step that fails on the way (a shape that a kernel
        # refuses, no memory for a buffer) leaves every request where it stood, and can be tried again
        done = self.cache.append_many([(e.request, len(e.tokens)) for e in entries], commit=False)  # OutOfPages changes nothing
        try:
            if self.execution == "graph":
                logits = self._run_program(self._program_key(entries, done), entries, done)
            else:
                ctx = self._context(entries, done)
                logits = self._forward(ctx, any(e.pending for e in entries))
        except BaseException:
            self.cache.abandon(done)
            raise
        self.cache.commit(done)
        self.steps += 1
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

    _FIXED = 10   # arrays of the metadata before the cache groups'

    def _width(self, context):
        """Block-table entries a step carries per request: what its longest context needs, in steps of 16 entries,
        not what the context limit would need (at a limit of 128k that would be megabytes a step)."""
        need = -(-int(context) // self.page_size)
        return min(self.table_width, -(-need // 16) * 16)

    def _layout(self, T, S, R, W):
        """Offsets of the packed int32 metadata: tokens, positions, seg_of_row, seg_start, seg_first_pos,
        state_slots, logit_rows, token_source, logit_slots, single_rows, then per group slots and tables, then one
        attention task list per known tiling (its length is the most tiles that T rows in S segments can make)."""
        G = len(self.cache.groups)
        sizes = [T, T, T, S + 1, S, S, R, T, R, S] + [T, S * W] * G + [4 * (-(-T // r) + S) for r in self.task_tilings]
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

    def _single_segments(self, done):
        """How many one-token segments of a mixed step get an attention launch of their own: all of them, if
        one of them has a long context; none in a step of one-token segments only, or of short contexts."""
        singles = [d.start + 1 for d in done if d.count == 1]
        if not singles or len(singles) == len(done) or max(singles) < self.split_single_from:
            return 0
        return len(singles)

    def _context(self, entries, done, pad=None, device_buffer=None, n_single=None, context=None):
        """Build the step's metadata on the host, upload it in one copy and wrap it.
        `pad` = (T, S, R) pads the batch with inert rows (for captured programs):
        token 0 at position 0, no segment, no cache slot."""
        counts = [d.count for d in done]
        starts = [d.start for d in done]
        n_rows, n_seg = sum(counts), len(entries)
        n_want = sum(len(e.want) for e in entries)
        T, S, R = pad if pad is not None else (n_rows, n_seg, n_want)
        # the longest context of the step (a captured program brings the bound of its bucket) sizes the block tables
        longest = max(s + c for s, c in zip(starts, counts))
        W, G, F = self._width(longest if context is None else context), len(self.cache.groups), self._FIXED
        layout = (T, S, R, W, tuple(self.task_tilings))
        offsets = self._layouts.get(layout)
        if offsets is None:
            offsets = self._layouts[layout] = [int(x) for x in self._layout(T, S, R, W)]
        total = offsets[-1]
        host = self._stage(total)
        arr = host.numpy()
        tokens, positions, seg_of_row, seg_start, seg_first, state_slots, logit_rows, token_source, logit_slots, single_rows = (
            arr[offsets[i]:offsets[i + 1]] for i in range(10))
        if n_single is None:      # (a captured program brings its padded number)
            n_single = self._single_segments(done)
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
        single_rows[:] = -1
        if n_single:
            own = [int(first_row[s]) for s, c in enumerate(counts) if c == 1]
            single_rows[:len(own)] = own
        tilings = list(self.task_tilings)
        for i, rows_per_tile in enumerate(tilings):
            tasks = arr[offsets[F + 2 * G + i]:offsets[F + 1 + 2 * G + i]].reshape(-1, 4)
            if decode_only:      # one tile of one row a segment
                n = n_seg
                tasks[:n, 0] = tasks[:n, 1] = first_row
                tasks[:n, 2] = 1
                tasks[:n, 3] = 0
            else:
                n = fill_tasks(tasks, counts, rows_per_tile, starts, skip_single=n_single > 0)
            tasks[n:] = (-1, 0, 0, 0)   # tiles of no segment do nothing
        dev = self._upload(host, total, device_buffer)

        def view(i, shape=None):
            t = dev[offsets[i]:offsets[i + 1]]
            return t if shape is None else t.view(shape)

        ctx = StepContext(self)
        ctx.n_rows, ctx.n_segments = T, S
        ctx.tokens, ctx.positions, ctx.seg_of_row = view(0), view(1), view(2)
        ctx.seg_start, ctx.seg_first_pos, ctx.state_slots, ctx.logit_rows = view(3), view(4), view(5), view(6)
        ctx.token_source = view(7)
        ctx.single_rows, ctx.n_single = view(9), n_single
        ctx.kv = [GroupView(view(F + 2 * g), view(F + 1 + 2 * g, (S, W)), self.page_size, W) for g in range(G)]
        ctx.tasks = {r: view(F + 2 * G + i, (-1, 4)) for i, r in enumerate(tilings)}
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
        wanted rows, whether every segment brings one token, and the context length rounded up
        to a power of two (it decides how attention splits the keys).  Steps with the same key
        replay one captured graph; only the metadata they read differs."""
        rows = sum(d.count for d in done)
        wanted = sum(len(e.want) for e in entries)
        decode_only = all(d.count == 1 for d in done)
        context = 1 << (max(d.start + d.count for d in done) - 1).bit_length()
        return (_bucket(rows), _bucket(len(entries)), _bucket(wanted), decode_only, max(context, 256),
                any(e.pending for e in entries), _bucket(self._single_segments(done)))

    def _run_program(self, key, entries, done):
        T, S, R, decode_only, context, take, n_single = key
        program = self.programs.get(key)
        if program is None:
            program = {"meta": None, "graph": None, "runs": 0, "tilings": None}
            self.programs[key] = program
            while len(self.programs) > self.program_capacity:
                oldest = next(iter(self.programs))
                torch.cuda.synchronize()
                del self.programs[oldest]
                self.workspace.release(oldest)
        else:
            self.programs[key] = self.programs.pop(key)  # most recently used last
        if program["tilings"] != self.task_tilings:
            # a mixer asked for a task list that the metadata did not hold yet: lay it out again
            torch.cuda.synchronize()
            program.update(meta=torch.zeros(int(self._layout(T, S, R, self._width(context))[-1]), dtype=torch.int32, device=self.device),
                           graph=None, runs=0, tilings=list(self.task_tilings))
        ctx = self._context(entries, done, pad=(T, S, R), device_buffer=program["meta"], n_single=n_single, context=context)
        ctx.owner = key
        ctx.span_hint = context   # launch shapes inside a captured program depend on the key only
        ctx.decode_only = decode_only
        if program["graph"] is None and program["runs"] >= 1 and program["tilings"] == self.task_tilings:
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
        if program["graph"] is not None:
            program["graph"].replay()
            logits = program["logits"]
        else:
            logits = self._forward(ctx, take)
        program["runs"] += 1
        wanted = sum(len(e.want) for e in entries)
        if logits is None:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return logits[:wanted]

    # -- attention dispatch -------------------------------------------------------
    def attention(self, ctx, q, q_row_stride, kcache, vcache, view, out, heads, kv_heads, head_dim, window, scale,
                  defer_merge=None):
        """bfloat16 with a head size in steps of 8 and pages of a power of two >= 4 run
        on the matrix cores (one block per row for decode steps, tiles of rows from a
        task list otherwise); everything else runs the exact row-wise kernel.

        `defer_merge(splits) -> bool`: the caller's next product can merge the partial results of a decode step whose
        keys are split over `splits` blocks itself (ops.gemm_merged).  Where that is so, no merge kernel runs, `out`
        is left alone and (partial outputs bf16, statistics float, splits) is returned; otherwise None."""
        rows = out.shape[0]
        span = ctx.span_hint if not window else min(ctx.span_hint, window + 31)
        if ops.mfma_attention_supported(out.dtype, head_dim, view.page_size):
            group = heads // kv_heads
            heads_per_chunk = min(group, 16)
            if ctx.decode_only:
                blocks = rows * kv_heads * -(-group // heads_per_chunk)
                waves, splits = self._rows_launch(blocks, span, heads_per_chunk, head_dim)
                if splits > 1 and defer_merge is not None:
                    # the product that follows merges 2, 4 or 8 partial results of a row while it prepares its operand:
                    # one kernel fewer than merging here.  Every block of that product reads them all, so more than 8
                    # rows bring at most 4 each.  (135M sizes, 8 rows at 2k: a step of 0.808 ms with the merge kernel,
                    # 0.808 with 4 splits merged there, whose attention blocks are half as many, 0.784 with 8.)
                    fused = next((n for n in (8, 4, 2) if n <= splits and (n <= 4 or rows <= 8) and defer_merge(n)), None)
                    if fused is not None:
                        workspace = (ctx.buffer("attn.part_o16", (rows * heads * fused * head_dim,), torch.bfloat16),
                                     ctx.buffer("attn.part_ml", (rows * heads * fused * 2,), torch.float32))
                        ops.attention_mfma(q, q_row_stride, kcache, vcache, view.tables, ctx.seg_of_row, ctx.positions, out,
                                           heads, kv_heads, head_dim, view.page_size, window, scale, None, fused, workspace, waves,
                                           merge=False)
                        return workspace[0], workspace[1], fused
                workspace = None
                if splits > 1:
                    workspace = (ctx.buffer("attn.part_o", (rows * heads * splits * head_dim,), torch.float32),
                                 ctx.buffer("attn.part_ml", (rows * heads * splits * 2,), torch.float32))
                ops.attention_mfma(q, q_row_stride, kcache, vcache, view.tables, ctx.seg_of_row, ctx.positions, out,
                                   heads, kv_heads, head_dim, view.page_size, window, scale, None, splits, workspace, waves)
            else:
                if ctx.n_single:
                    # the decoded tokens of this mixed step: a launch of their own that splits their keys
                    n = ctx.n_single
                    waves, splits = self._rows_launch(n * kv_heads * -(-group // heads_per_chunk), span, heads_per_chunk, head_dim)
                    workspace = None
                    if splits > 1:
                        workspace = (ctx.buffer("attn.part_o", (n * heads * splits * head_dim,), torch.float32),
                                     ctx.buffer("attn.part_ml", (n * heads * splits * 2,), torch.float32))
                    ops.attention_mfma(q, q_row_stride, kcache, vcache, view.tables, ctx.seg_of_row, ctx.positions, out,
                                       heads, kv_heads, head_dim, view.page_size, window, scale, None, splits, workspace, waves,
                                       row_ids=ctx.single_rows[:n])
                kind, item_tiles, halves = self.prompt_attention_form(rows, ctx.n_segments, span, heads, kv_heads, head_dim, view.page_size)
                tasks = ctx.attention_tasks((16 if kind == "tiles" else 64) * item_tiles // heads_per_chunk)
                ops.attention_mfma(q, q_row_stride, kcache, vcache, view.tables, ctx.seg_of_row, ctx.positions, out,
                                   heads, kv_heads, head_dim, view.page_size, window, scale, tasks, waves=self.tile_waves,
                                   block_tiles={"tiles": False, "block": True, "square": 32}[kind], item_tiles=item_tiles,
                                   key_groups=halves)
            return
        splits = self._splits(rows * heads, span)
        workspace = None
        if splits > 1:
            workspace = (ctx.buffer("attn.part_o", (rows * heads * splits * head_dim,), torch.float32),
                         ctx.buffer("attn.part_ml", (rows * heads * splits * 2,), torch.float32))
        ops.attention_rowwise(q, q_row_stride, kcache, vcache, view.tables, ctx.seg_of_row, ctx.positions, out,
                              heads, kv_heads, head_dim, view.page_size, window, scale, splits, workspace)

    def prompt_attention_form(self, rows, n_segments, span, heads, kv_heads, head_dim, page_size):
        """Which form of the matrix-core kernel the prompt rows of a step take, (kind, n, halves): ("tiles", n, 1): a block
        is one tile of 16 n items (a token row and a query head) whose waves split its keys; ("block", n, 1): 64 n items,
        four waves that own different rows and share keys and values through LDS; ("square", n, halves): 64 n items on
        the 32 x 32 instruction with waves of their own for the copies, as one half or as two that take the even and the
        odd steps.  `span`: the longest context of the step."""
        group = heads // kv_heads
        heads_per_chunk = min(group, 16)
        long_portions = rows >= 16 * n_segments
        if long_portions and head_dim <= 128:
            # enough long portions to fill the GPU with blocks of 64 items (or more): the waves of a block own different
            # rows and share each step's keys and values through LDS.  Otherwise (few heads, short portions) the waves
            # of a block share one tile of 16 items (32 with small heads) and split its keys, which is what hides
            # the latency of a step when blocks are scarce.
            blocks = -(-rows // (64 // heads_per_chunk)) * kv_heads * -(-group // heads_per_chunk)
            # Long contexts: the 32 x 32 form, with three steps in flight a wave.  It costs about 3 us more to start
            # than the others, so it is for tiles that walk a thousand keys and more; larger blocks share the copies
            # among more waves but need more blocks to fill the GPU (MI355X, 2,048 rows: 1.7B sizes 61 us -> 46,
            # 8B sizes 115 -> 71, 135M sizes 32 -> 30; 4,096 rows at the 1.7B sizes: 147 with 128 items, 125 with 256).
            if page_size >= 8 and self.square_tiles != 0:
                n = 0
                if self.square_tiles is not None:
                    n = self.square_tiles
                elif span >= 1024 and blocks >= 512:
                    # from 2,048 blocks of 64 items on: 192 items, six computing waves beside the two that copy (eight waves:
                    # a compute unit holds two such blocks with small heads, one with large, and no wave slot stays empty).
                    # 32 heads of 64 at 16k rows: 1.42 ms against 1.46 with 256 items and 1.54 with 128; 9 heads over 3 at
                    # 32k: 1.49 against 1.58 and 1.61; 32 heads of 128 over 8 at 8k: 0.60 against 0.63 with 128 items
                    # (heads of more than 64 coordinates, one computing wave a SIMD: already from 1,100 blocks on; 32 heads
                    # of 128 over 8 at 3,072 rows, 1,536 blocks: 106 us against 123; 24 heads of 96 over 8: 72 against 84)
                    n = 3 if blocks >= (2048 if head_dim <= 64 else 1100) else 2
                elif span >= 1024 and blocks >= 128:
                    # (fewer blocks than compute units and a thousand keys: 64-item blocks, in two halves; 1,024 rows of
                    # 12 heads of 128 take 25 us against 35 as LDS block tiles, of 16 heads of 64 over 4: 17 against 18)
                    n = 1
                if n:
                    # about one block a compute unit: the time is the longest tile's chain of steps, which two halves a
                    # block cut in two (2,048 rows at the 135M sizes 31.6 -> 28.4 us, 4,096 rows 64 -> 55; with more
                    # blocks than that the halves only crowd the compute units: 46 -> 68 us at the 1.7B sizes)
                    # (up to 511 blocks of 64 items when the chain is long: 3,072 rows at the 135M sizes, 441 blocks,
                    # 35.6 us against 43.4; 16 heads over 4 at 1,536 rows 22.1 against 25.4; at 1,000 rows the halves lose)
                    # and up to 512 blocks of 128 items from 3,072 keys on: 8 heads of 64 at 6,144 rows 71 against 89,
                    # 9 over 3 at 6,144 rows 76 against 92, 16 over 4 at 3,072 rows 42 against 50
                    few = (-(-blocks // n) <= 320 or (n == 1 and span >= 1536)
                           or (n == 2 and -(-blocks // n) <= 512 and span >= 3072))
                    fits = n == 1 or (n == 2 and head_dim <= 64)
                    halves = 2 if (few and fits if self.square_halves is None else self.square_halves == 2 and fits) else 1
                    return "square", n, halves
            block_tiles = (2 if blocks >= 2048 else 1 if blocks >= 512 else 0) if self.block_tiles is None else self.block_tiles
            if block_tiles:
                return "block", block_tiles, 1
        return "tiles", 2 if self.item_tiles == 2 and long_portions and head_dim <= 64 else 1, 1

    @staticmethod
    def _splits(waves, span):
        """Row-wise kernel: how many ways a row's keys are split among wavefronts: enough to
        fill the GPU when the batch alone does not, never finer than 256 keys a split."""
        if waves >= 2048 or span <= 256:
            return 1
        return int(min(32, -(-span // 256), max(1, 4096 // waves)))

    @staticmethod
    def _rows_launch(blocks, span, heads_per_chunk, head_dim):
        """Matrix-core decode kernel: (wavefronts a block, blocks along the keys).  Few rows:
        eight waves share a row's keys inside one block; when that still leaves the GPU idle
        and the context is long, the keys are also split over blocks (a merge kernel follows).
        Many rows: four waves a block, one block a row and head group, or with small heads eight waves
        when that gives every compute unit at most one block."""
        steps = -(-span // 32)
        few = blocks < 128
        # eight waves a block with few rows and small heads (at 8k and 32k too, now that at most eight splits of few
        # rows are merged by the product that follows: 4 rows at 8k 15.3 us against 16.3 with four waves, 8 rows at
        # 32k 44.4 against 46.5)
        waves = 8 if few and head_dim <= 64 else 4
        if steps <= 2 * waves:
            # two steps a wave: nothing to split (a second block along the keys and the merge cost 2 us of 8 to 10)
            return waves, 1
        if few:
            # Few rows: split the keys until the blocks fill the GPU once: an eight-wave block fills a compute
            # unit (256 blocks; more start a second round: 16 splits of 8 rows at 2k to 4k are 10 % slower than
            # 8), four-wave blocks fit three a unit, of which two are worth having (512 blocks: a thousand are
            # 12 % slower at 30k, where each then lives for three steps a wave only).  A wave keeps at least one
            # 32-key step (with two, 8 rows at 2k have 4 splits and are 5 % slower).
            # At most 32 splits: a single row of 8 key heads at 8k takes 23 us with 32 and 30 with 64.
            room = 256 if waves == 8 else 512
            splits = int(max(1, min(steps // waves, room // blocks, 32)))
        elif head_dim <= 64 and 140 <= blocks <= 256:
            # enough rows to give most compute units one block of eight waves, and no more than one each: the
            # keys are not split and no merge follows (9-11 % faster than four waves and three or four splits at
            # 144 to 256 blocks and 2k keys, 4-5 % at 8k)
            waves, splits = 8, 1
        else:
            # Many rows split until every compute unit has the blocks of four waves that its registers hold (three
            # with small heads, two otherwise: 3-5 % faster at 384 blocks of the 135M sizes than one block a unit;
            # from 512 blocks on a split costs 3-8 %); a wave keeps at least four 32-key steps (with two, 128 rows at
            # 512 keys take 19.4 us against 16.5 unsplit).
            target = 768 if head_dim <= 64 else 512
            per = target // blocks if head_dim <= 64 and blocks > 256 else -(-target // blocks)
            splits = int(max(1, min(steps // (waves * 4), per, 64)))
        return waves, splits
