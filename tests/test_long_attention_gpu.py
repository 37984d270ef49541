"""Attention at the shapes that the benchmark times, through the call that the engine makes
(kernels.attention.paged_attention: the rules pick the form and the launch shape, nothing is forced unless a test
says so): decode rows over 8,192 and 32,768 keys, prompt portions of 4,096 rows (also on a cached prefix), and a mixed
step whose decoded tokens have contexts past the point where they get a launch of their own.

The reference is float32 on the GPU with plain torch products and softmax over the gathered pages (a NumPy loop over
rows would take minutes at these sizes); the bfloat16 inputs are widened exactly.  Queries are scaled so that the
scores spread over several units: a few keys carry each row's weight, somewhere in its context, so that a key that is
dropped, doubled or masked wrongly moves the row by far more than rounding does."""
import math

import numpy as np
import pytest
import torch

from runtime.engine.context import Batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
P = 16


class Step:
    """What paged_attention asks of a step's context, without an engine around it."""

    def __init__(self, counts, starts):
        self.counts, self.starts = list(counts), list(starts)
        self.n_segments, self.n_rows = len(counts), sum(counts)
        first = np.concatenate(([0], np.cumsum(counts[:-1]))).astype(np.int32)
        self.decode_only = all(c == 1 for c in counts)
        self.batch = Batch(self.counts, self.starts, first, self.decode_only, {})
        self.span_hint = max(s + c for s, c in zip(starts, counts))
        seg = np.repeat(np.arange(len(counts), dtype=np.int32), counts)
        pos = np.concatenate([np.arange(s, s + c, dtype=np.int32) for s, c in zip(starts, counts)])
        self.seg_of_row, self.positions = torch.from_numpy(seg).to(DEV), torch.from_numpy(pos).to(DEV)
        self.arrays, self.buffers = {}, {}

    def buffer(self, name, shape, dtype):
        key = (name, tuple(shape), dtype)
        if key not in self.buffers:
            self.buffers[key] = torch.empty(shape, dtype=dtype, device=DEV)
        return self.buffers[key]

    def step_array(self, array):
        if array not in self.arrays:
            value = array.launch_value(self.batch)
            self.batch.launch_values[array] = value
            host = np.zeros(array.words(self.n_rows, self.n_segments), dtype=np.int32)
            array.fill(host, self.batch, value)
            self.arrays[array] = (torch.from_numpy(host).to(DEV), value)
        return self.arrays[array]


class View:
    def __init__(self, tables):
        self.tables, self.page_size, self.width = tables, P, tables.shape[1]


def make_cache(step, kv_heads, D, seed):
    """Scattered pages holding random keys and values for every segment's whole context; the queries of the step's rows."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    ends = [s + c for s, c in zip(step.starts, step.counts)]
    per = [-(-e // P) for e in ends]
    n_pages = sum(per) + 3
    order = torch.randperm(n_pages, generator=g, device=DEV).int()
    tables = torch.full((step.n_segments, -(-max(per) // 16) * 16), -1, dtype=torch.int32, device=DEV)
    at = 0
    for s, n in enumerate(per):
        tables[s, :n] = order[at:at + n]
        at += n
    K = torch.randn(n_pages, kv_heads, P, D, generator=g, device=DEV).bfloat16()
    V = torch.randn(n_pages, kv_heads, D, P, generator=g, device=DEV).bfloat16()
    return K, V, tables


def reference(q, K, V, tables, step, heads, kv_heads, D, scale, chunk=256):
    """float32 on the GPU: row r of segment s attends to keys 0..position of its request."""
    out = torch.empty(step.n_rows, heads * D, dtype=torch.float32, device=DEV)
    group = heads // kv_heads
    row = 0
    for s, (start, count) in enumerate(zip(step.starts, step.counts)):
        n = -(-(start + count) // P)
        pages = tables[s, :n].long()
        keys = K[pages].float().permute(1, 0, 2, 3).reshape(kv_heads, n * P, D)            # [kv, ctx, D]
        values = V[pages].float().permute(1, 0, 3, 2).reshape(kv_heads, n * P, D)          # pages hold [D, P]
        index = torch.arange(n * P, device=DEV)
        for a in range(0, count, chunk):
            b = min(count, a + chunk)
            qs = q[row + a:row + b].float().view(b - a, kv_heads, group, D).permute(1, 2, 0, 3)     # [kv, group, rows, D]
            scores = torch.matmul(qs, keys[:, None].transpose(-1, -2)) * scale                       # [kv, group, rows, ctx]
            pos = torch.arange(start + a, start + b, device=DEV)
            scores = scores.masked_fill(index[None, None, None, :] > pos[None, None, :, None], float("-inf"))
            weights = torch.softmax(scores, dim=-1)
            o = torch.matmul(weights, values[:, None])                                               # [kv, group, rows, D]
            out[row + a:row + b] = o.permute(2, 0, 1, 3).reshape(b - a, heads * D)
        row += count
    return out


def attend(step, heads, kv_heads, D, seed, tuning=None, spread=3.0):
    from runtime.kernels import attention
    K, V, tables = make_cache(step, kv_heads, D, seed)
    g = torch.Generator(device=DEV).manual_seed(seed + 1)
    # scores of standard deviation `spread`: q . k has variance D for unit normals
    q = (torch.randn(step.n_rows, heads * D, generator=g, device=DEV) * spread).bfloat16()
    scale = 1.0 / math.sqrt(D)
    out = torch.full((step.n_rows, heads * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    left = attention.paged_attention(step, q, heads * D, K, V, View(tables), out, heads, kv_heads, D, None, scale,
                                     tuning=tuning or attention.DEFAULT_TUNING)
    assert left is None
    want = reference(q, K, V, tables, step, heads, kv_heads, D, scale)
    torch.cuda.synchronize()
    return out.float(), want


def check(got, want, what):
    assert torch.isfinite(got).all(), f"{what}: non-finite outputs"
    scale = want.abs().max().item()
    worst = (got - want).abs().max().item() / scale
    rms = ((got - want).norm() / want.norm()).item()
    print(f"{what}: worst {worst:.2e} of the largest output, relative rms {rms:.2e}")
    # bfloat16 outputs round at 2^-9 = 2.0e-3 of their own size, the weights inside the kernel at as much again; a key
    # lost from a row whose weight sits on a few keys moves that row by a tenth of the largest output and more
    assert worst < 8e-3 and rms < 4e-3, f"{what}: worst {worst:.3e}, rms {rms:.3e}"


SHAPES = [(9, 3, 64), (32, 8, 128)]


@pytest.mark.parametrize("heads, kv_heads, D", SHAPES)
@pytest.mark.parametrize("context", [8192, 32768])
@pytest.mark.parametrize("rows", [1, 8])
def test_decode_rows_over_long_contexts(heads, kv_heads, D, context, rows):
    from runtime.kernels.attention import rows_launch
    starts = [context - 1 - 37 * i for i in range(rows)]       # lengths that are no multiples of anything
    step = Step([1] * rows, starts)
    group = min(heads // kv_heads, 16)
    waves, splits = rows_launch(rows * kv_heads, context, group, D)
    assert splits >= 8, "these points are meant to split the keys over blocks"
    got, want = attend(step, heads, kv_heads, D, seed=context + rows)
    check(got, want, f"{heads}/{kv_heads}x{D}, {rows} rows at {context}: {waves} waves x {splits} splits")


@pytest.mark.parametrize("heads, kv_heads, D", SHAPES)
@pytest.mark.parametrize("launch", [(4, 16), (8, 32), (4, 32)])
def test_decode_rows_with_sixteen_and_thirty_two_splits(heads, kv_heads, D, launch):
    from runtime.kernels.attention import AttentionTuning
    if launch[0] == 8 and D > 64:
        pytest.skip("eight waves a block are for head sizes up to 64")
    step = Step([1] * 3, [8191, 5000, 777])       # the short row leaves most of its splits without a key
    got, want = attend(step, heads, kv_heads, D, seed=sum(launch), tuning=AttentionTuning(rows_launch=launch))
    check(got, want, f"{heads}/{kv_heads}x{D}, {launch[0]} waves x {launch[1]} splits")


@pytest.mark.parametrize("heads, kv_heads, D", SHAPES)
@pytest.mark.parametrize("launch", [(4, 1), (8, 4), (4, 8)])
def test_decode_rows_read_with_non_temporal_loads_give_the_same_bits(heads, kv_heads, D, launch):
    """The two kinds of load differ in what the caches keep, not in what arrives: the outputs are equal bit for bit."""
    from runtime.kernels.attention import AttentionTuning
    step = Step([1] * 5, [4099, 2047, 31, 700, 0])
    plain, want = attend(step, heads, kv_heads, D, seed=sum(launch), tuning=AttentionTuning(rows_launch=launch, stream_loads=False))
    streamed, _ = attend(step, heads, kv_heads, D, seed=sum(launch), tuning=AttentionTuning(rows_launch=launch, stream_loads=True))
    check(streamed, want, f"{heads}/{kv_heads}x{D}, {launch[0]} waves x {launch[1]} splits, non-temporal loads")
    assert torch.equal(plain, streamed)


@pytest.mark.parametrize("heads, kv_heads, D, start, form", [
    (9, 3, 64, 0, ("square", 2, 2)),
    (32, 32, 64, 0, ("square", 3, 1)),
    (32, 8, 128, 0, ("square", 3, 1)),
    (32, 8, 128, 4000, ("square", 3, 1)),        # a portion on a cached prefix: rows 4000..8095
    (9, 3, 64, 28000, ("square", 2, 2)),         # the last portion of a 32k prompt
])
def test_prompt_portions_of_4096_rows(heads, kv_heads, D, start, form):
    from runtime.kernels.attention import prompt_form
    step = Step([4096], [start])
    assert tuple(prompt_form(4096, 1, start + 4096, heads, kv_heads, D, P)) == form
    got, want = attend(step, heads, kv_heads, D, seed=start + heads)
    check(got, want, f"{heads}/{kv_heads}x{D}, 4096 rows from {start}: {form}")


@pytest.mark.parametrize("heads, kv_heads, D", SHAPES)
def test_mixed_step_whose_decoded_tokens_have_long_contexts(heads, kv_heads, D):
    """A portion of 512 rows beside eight decoded tokens with contexts of 4,100 to 6,000 keys: past 4,096 the decoded
    tokens leave the tile list for a launch of their own that splits their keys (nothing forced)."""
    from runtime.kernels.attention import DEFAULT_TUNING, SingleRows
    counts = [1, 1, 512, 1, 1, 1, 1, 1, 1]
    starts = [4100, 5999, 3000, 4500, 4777, 5100, 5555, 4099, 5000]
    step = Step(counts, starts)
    got, want = attend(step, heads, kv_heads, D, seed=7)
    assert step.arrays[SingleRows(DEFAULT_TUNING.split_single_from)][1] == 8, "the decoded tokens had no launch of their own"
    check(got, want, f"{heads}/{kv_heads}x{D}, 512 rows beside 8 decoded tokens")
