"""Paged attention as one call: which kernel, in which form and launch shape, and the step metadata it wants.

`paged_attention` is what a mixer calls.  bfloat16 with a head size in steps of 8 and pages of a power of two >= 8
runs on the matrix cores (one block per row for decode steps, tiles of rows from a task list otherwise); everything
else runs the exact row-wise kernel.  The rules that pick a form or a launch shape are plain functions of sizes
(`rows_launch`, `prompt_form`, `rowwise_splits`), each settled by measurements on an MI355X that its comments quote;
what may be tuned sits in `AttentionTuning`.

The kernels read two kinds of per-step lists that only this file knows the meaning of: task lists (tiles of rows
of one segment) and the rows of the one-token segments of a mixed step.  Both are `StepArray`s: a mixer asks the
step's context for them (`ctx.step_array`), and the step function carries them in every step's metadata from then
on without knowing what they hold.  The reference has one attention kernel and no such choice
(kernels/ops.cu:35-80).
"""
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from . import ops


@dataclass
class AttentionTuning:
    """What the rules below may be told instead of deciding by size (None: decide)."""
    block_tiles: Optional[int] = None     # long portions through LDS-shared tiles of 64 x this items
    square_tiles: Optional[int] = None    # long portions of long contexts through 32 x 32 tiles, 64 x this items a block (0: never)
    square_halves: Optional[int] = None   # two halves a block in that form (even and odd steps): 1, 2
    tile_waves: int = 4                   # wavefronts that share one tile's keys
    item_tiles: int = 2                   # 16-item tiles a wave of long portions (small heads)
    # In a mixed step a decoded token is a tile whose keys one block walks; from this context on the one-token
    # segments get a launch of their own instead, which splits their keys over blocks
    split_single_from: int = 4096
    rows_launch: Optional[tuple] = None   # (wavefronts a block, blocks along the keys) of decode rows
    stream_loads: Optional[bool] = None   # decode rows read keys and values with non-temporal loads (None: by the rule)
    # A step of single tokens whose keys are not split runs a block for every (row, key head), the key heads of a row
    # side by side.  From this many blocks on (more than one block a compute unit) the rows are listed longest first,
    # so that the launch does not end with the blocks of a long row alone (64 rows of 228 to 2,304 keys at the 1.7B
    # sizes: 126.6 -> 119.7 us, what 64 rows of their mean length take; 128 rows at the 135M sizes 36.3 -> 34.2)
    order_rows_from: int = 320


DEFAULT_TUNING = AttentionTuning()


# -- step metadata ----------------------------------------------------------------------------------------------

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


@dataclass(frozen=True)
class SingleRows:
    """Step array: the rows of the one-token segments of a mixed step (then -1), when they get an attention launch
    of their own: all of them, if one of them has a context of `split_from` keys or more; none in a step of
    one-token segments only, or of short contexts.  Its launch value is how many entries such a launch covers."""
    split_from: int

    def words(self, rows, segments):
        return segments

    def launch_value(self, batch):
        singles = [start + 1 for start, count in zip(batch.starts, batch.counts) if count == 1]
        if not singles or len(singles) == len(batch.counts) or max(singles) < self.split_from:
            return 0
        return len(singles)

    def fill(self, out, batch, value):
        out[:] = -1
        if value:
            own = [int(batch.first_row[s]) for s, c in enumerate(batch.counts) if c == 1]
            out[:len(own)] = own


@dataclass(frozen=True)
class RowsLongestFirst:
    """Step array: the rows of a step of one-token segments by the number of keys they attend to, most first (rows of
    equal length in their own order), then the padding rows (which have no keys: zeros are written for them).  Blocks
    are handed out in this order."""

    def words(self, rows, segments):
        return rows

    def launch_value(self, batch):
        return None

    def fill(self, out, batch, value):
        out[:] = np.arange(len(out))
        if batch.decode_only:
            order = np.argsort(-np.asarray(batch.starts, dtype=np.int64), kind="stable")
            out[:len(order)] = np.asarray(batch.first_row, dtype=np.int64)[order]


@dataclass(frozen=True)
class TileTasks:
    """Step array: the task list of tiles of at most `rows_per_tile` rows, int32 [n, 4]; tiles of no segment
    (-1, 0, 0, 0) pad it.  `singles`: the SingleRows whose launch takes the one-token segments away from the tiles."""
    rows_per_tile: int
    singles: Optional[SingleRows] = None

    def words(self, rows, segments):
        return 4 * (-(-rows // self.rows_per_tile) + segments)   # the most tiles that `rows` rows in `segments` segments make

    def launch_value(self, batch):
        return None

    def fill(self, out, batch, value):
        tasks = out.reshape(-1, 4)
        if batch.decode_only:      # one tile of one row a segment
            n = len(batch.counts)
            tasks[:n, 0] = tasks[:n, 1] = batch.first_row
            tasks[:n, 2] = 1
            tasks[:n, 3] = 0
        else:
            skip = self.singles is not None and batch.launch_values.get(self.singles, 0) > 0
            n = fill_tasks(tasks, batch.counts, self.rows_per_tile, batch.starts, skip_single=skip)
        tasks[n:] = (-1, 0, 0, 0)


# -- rules ------------------------------------------------------------------------------------------------------

def prompt_form(rows, n_segments, span, heads, kv_heads, head_dim, page_size, tuning=DEFAULT_TUNING):
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
        if page_size >= 8 and tuning.square_tiles != 0:
            n = 0
            if tuning.square_tiles is not None:
                n = tuning.square_tiles
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
                halves = 2 if (few and fits if tuning.square_halves is None else tuning.square_halves == 2 and fits) else 1
                return "square", n, halves
        block_tiles = (2 if blocks >= 2048 else 1 if blocks >= 512 else 0) if tuning.block_tiles is None else tuning.block_tiles
        if block_tiles:
            return "block", block_tiles, 1
    return "tiles", 2 if tuning.item_tiles == 2 and long_portions and head_dim <= 64 else 1, 1


def rows_per_tile_of(form, heads, kv_heads):
    """Rows of one segment that a tile of `form` (prompt_form) holds."""
    kind, n, _ = form
    return (16 if kind == "tiles" else 64) * n // min(heads // kv_heads, 16)


def rowwise_splits(waves, span):
    """Row-wise kernel: how many ways a row's keys are split among wavefronts: enough to
    fill the GPU when the batch alone does not, never finer than 256 keys a split."""
    if waves >= 2048 or span <= 256:
        return 1
    return int(min(32, -(-span // 256), max(1, 4096 // waves)))


def rows_launch(blocks, span, heads_per_chunk, head_dim):
    """Matrix-core decode kernel: (wavefronts a block, blocks along the keys).  Few rows:
    eight waves share a row's keys inside one block; when that still leaves the GPU idle
    and the context is long, the keys are also split over blocks (a merge kernel follows).
    Many rows: four waves a block, one block a row and head group, or with small heads eight waves
    when that gives every compute unit at most one block."""
    steps = -(-span // 32)
    few = blocks < 128
    # eight waves a block with few rows and small heads (at 8k and 32k too: 4 rows at 8k 15.3 us against 16.3 with
    # four waves, 8 rows at 32k 44.4 against 46.5)
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
        if splits > 16 and steps < 2 * waves * splits:
            # more than 16 splits only with two steps a wave and more: their merge costs more than a second step (one
            # and four rows at 8k keys of the 135M sizes: decode steps of 0.829 and 0.901 ms with 31 and 21 splits,
            # 0.796 and 0.877 with 16; at 32k 32 and 21 splits stay, 16 would take 1.33 against 1.02 ms)
            splits = max(16, steps // (2 * waves))
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
    if waves == 8 and blocks >= 48 and span >= (16384 if blocks < 96 else 6144):
        # Eight-wave blocks whose waves walk long runs of keys: four waves and more blocks along the keys instead, about
        # 1,536 in all, which read with non-temporal loads (`rows_stream_loads`).  Decode steps of the 135M sizes: 32
        # rows at 8k keys 1.865 -> 1.779 ms, 64 rows 2.798 -> 2.755; at 32k 16, 32 and 64 rows 2.695 -> 2.625, 4.713 ->
        # 4.455 and 8.539 -> 8.107; 16 rows at 8k gain nothing.
        waves, splits = 4, int(min(max(1, 1536 // blocks), 16, max(1, steps // 16)))
    return waves, splits


def rows_stream_loads(blocks, span, waves, splits, head_dim):
    """Whether the decode kernel launched as `blocks` x `splits` blocks of `waves` wavefronts reads keys and values with
    non-temporal loads (no block reads them again; the caches then do not keep them).  Measured inside decode steps
    of the three sizes at 448 to 32,000 keys and 1 to 64 rows: blocks of four waves never lose by them and gain up to
    11 % of the whole step (64 rows at 8k keys of the 8B sizes 4.64 -> 4.12 ms, 32 rows at 2k of the 1.7B sizes 1.379 ->
    1.275).  Blocks of eight waves (head sizes up to 64) gain 2-3 % of the step where they fill the GPU and a wave has
    little more than two 32-key steps (8 and 16 rows at 2k of the 135M sizes, 4 rows at 8k), and lose 2-11 % where a
    wave walks a longer run of keys (four steps and more: 32 and 64 rows at 2k to 32k) or the blocks are few (+4-6 %
    below 96 blocks)."""
    if head_dim > 64 or waves == 4:               # (larger heads run eight waves as four)
        return True
    steps = -(-span // 32)
    return blocks * splits >= 160 and 2 * steps <= 5 * waves * splits


def fused_merge_splits(splits, rows, accepts):
    """How many of the `splits` blocks along a decode row's keys the product that follows may merge itself
    (`accepts(n)` says whether it takes n), or None: then the merge kernel runs.  That product merges 2, 4 or 8
    partial results of a row while it prepares its operand: one kernel fewer than merging here.  Every block of it
    reads them all, so more than 8 rows bring at most 4 each.  (135M sizes, 8 rows at 2k: a step of 0.808 ms with the
    merge kernel, 0.808 with 4 splits merged there, whose attention blocks are half as many, 0.784 with 8.)  It is
    taken only where it costs at most half of the blocks that `rows_launch` asked for: one row at 8k to 32k keeps its
    24 to 32 splits and the merge kernel."""
    for n in (8, 4, 2):
        if n <= splits and splits <= 2 * n and (n <= 4 or rows <= 8) and accepts(n):
            return n
    return None


# -- the call ---------------------------------------------------------------------------------------------------

def kernel_units(head_dim, dtype):
    """Names of the shared objects that attention with this head size needs beside the core (library.ensure)."""
    from . import library
    if dtype == torch.bfloat16 and head_dim % 8 == 0 and 0 < head_dim <= 256:
        return [library.attention_unit(-(-head_dim // 32) * 32)]
    return []


def _split_workspace(ctx, rows, heads, splits, head_dim, dtype=torch.float32, tag="attn.part_o"):
    return (ctx.buffer(tag, (rows * heads * splits * head_dim,), dtype),
            ctx.buffer("attn.part_ml", (rows * heads * splits * 2,), torch.float32))


def paged_attention(ctx, q, q_row_stride, kcache, vcache, view, out, heads, kv_heads, head_dim, window, scale,
                    defer_merge=None, tuning=DEFAULT_TUNING):
    """out[r] = attention of row r's queries over its request's cached keys up to its own position (or the last
    `window` of them).  `ctx` is the step's context (rows, segments, positions, buffers, step arrays), `view` the
    cache group as the step sees it (block tables, page size).

    `defer_merge(splits) -> bool`: the caller's next product can merge the partial results of a decode step whose
    keys are split over `splits` blocks itself (ops.gemm_merged).  Where that is so, no merge kernel runs, `out`
    is left alone and (partial outputs bf16, statistics float, splits) is returned; otherwise None."""
    rows = out.shape[0]
    span = ctx.span_hint if not window else min(ctx.span_hint, window + 31)
    common = (q, q_row_stride, kcache, vcache, view.tables, ctx.seg_of_row, ctx.positions, out, heads, kv_heads, head_dim,
              view.page_size, window, scale)
    if not ops.mfma_attention_supported(out.dtype, head_dim, view.page_size):
        splits = rowwise_splits(rows * heads, span)
        workspace = _split_workspace(ctx, rows, heads, splits, head_dim) if splits > 1 else None
        ops.attention_rowwise(*common, splits, workspace)
        return None
    group = heads // kv_heads
    heads_per_chunk = min(group, 16)
    chunks = kv_heads * -(-group // heads_per_chunk)

    def stream(blocks, waves, splits):
        if tuning.stream_loads is not None:
            return tuning.stream_loads
        return rows_stream_loads(blocks, span, waves, splits, head_dim)

    if ctx.decode_only:
        waves, splits = tuning.rows_launch or rows_launch(rows * chunks, span, heads_per_chunk, head_dim)
        if splits > 1 and defer_merge is not None:
            fused = fused_merge_splits(splits, rows, defer_merge)
            if fused is not None:
                workspace = _split_workspace(ctx, rows, heads, fused, head_dim, torch.bfloat16, "attn.part_o16")
                ops.attention_mfma(*common, None, fused, workspace, waves, merge=False,
                                   stream_loads=stream(rows * chunks, waves, fused))
                return workspace[0], workspace[1], fused
        workspace = _split_workspace(ctx, rows, heads, splits, head_dim) if splits > 1 else None
        order = None
        if splits == 1 and rows * chunks >= tuning.order_rows_from:
            order = ctx.step_array(RowsLongestFirst())[0][:rows]
        ops.attention_mfma(*common, None, splits, workspace, waves, row_ids=order, stream_loads=stream(rows * chunks, waves, splits))
        return None
    singles = SingleRows(tuning.split_single_from)
    single_rows, n_single = ctx.step_array(singles)
    if n_single:
        # the decoded tokens of this mixed step: a launch of their own that splits their keys
        waves, splits = tuning.rows_launch or rows_launch(n_single * chunks, span, heads_per_chunk, head_dim)
        workspace = _split_workspace(ctx, n_single, heads, splits, head_dim) if splits > 1 else None
        ops.attention_mfma(*common, None, splits, workspace, waves, row_ids=single_rows[:n_single],
                           stream_loads=stream(n_single * chunks, waves, splits))
    form = prompt_form(rows, ctx.n_segments, span, heads, kv_heads, head_dim, view.page_size, tuning)
    kind, item_tiles, halves = form
    tasks, _ = ctx.step_array(TileTasks(rows_per_tile_of(form, heads, kv_heads), singles))
    ops.attention_mfma(*common, tasks.view(-1, 4), waves=tuning.tile_waves,
                       block_tiles={"tiles": False, "block": True, "square": 32}[kind], item_tiles=item_tiles, key_groups=halves)
    return None
