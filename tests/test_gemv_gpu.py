"""The matrix-vector kernel (one or two rows against large weights in the engine; here given up to eight rows and weights of any size): every prologue (plain rows, fused RMSNorm with
and without picked rows, the merge of split attention) and every epilogue (store, residual, SwiGLU, rotary embedding
with the cache write) against float64, at the family's sizes and at sizes that fit nothing (inner sizes that leave
lanes without a chunk, or give them several batches; outputs that do not fill the last wave).  A row's result is
bit for bit the same whatever rows stand beside it."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from runtime.kernels import ops as o
    o.lib()
    o.set_gemv(8, 0)          # every product of up to eight rows, whatever the size of the weights
    yield o
    o.set_gemv()


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def f64(t):
    return t.detach().double().cpu().numpy()


def bf(x):
    """float64 array rounded to bfloat16 (as the kernels round their operands)."""
    return torch.from_numpy(np.asarray(x, np.float32)).to(torch.bfloat16).double().numpy()


SHAPES = [(1, 16, 32), (3, 100, 72), (8, 576, 576), (8, 576, 1536), (5, 1003, 200), (2, 300, 4096), (1, 64, 14336), (7, 49, 264),
          (4, 2048, 2048), (8, 40, 2560)]


@pytest.mark.parametrize("M, N, K", SHAPES)
def test_plain_and_residual(ops, M, N, K):
    assert ops.gemv_ok(M, N, K) and not ops.gemv_ok(9, N, K)
    a, w, r = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2, scale=0.1), rnd(M, N, seed=3)
    want = f64(a) @ f64(w).T
    tol = dict(rtol=1e-4, atol=1e-5 * math.sqrt(K))
    np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, device=DEV))), want, **tol)
    np.testing.assert_allclose(f64(ops.gemm(a, w, r.clone(), residual=None)), want, **tol)
    got = r.clone()
    ops.gemm(a, w, got, residual=got)
    np.testing.assert_allclose(f64(got), want + f64(r), **tol)
    out16 = ops.gemm(a, w, torch.empty(M, N, device=DEV, dtype=torch.bfloat16))
    np.testing.assert_allclose(f64(out16), want, rtol=1e-2, atol=1e-2)
    # a row's result does not depend on its company: bit for bit
    full = ops.gemm(a, w, torch.empty(M, N, device=DEV))
    for rows in (1, 2, 4):
        if rows < M:
            part = ops.gemm(a[:rows].contiguous(), w, torch.empty(rows, N, device=DEV))
            assert torch.equal(part, full[:rows]), f"{rows} of {M} rows"


@pytest.mark.parametrize("M, I, K", [(1, 24, 64), (8, 1536, 576), (3, 100, 200), (4, 8192, 2048), (2, 77, 4104)])
def test_swiglu_with_and_without_the_fused_norm(ops, M, I, K):
    x = rnd(M + 2, K, seed=4, scale=2.0)
    nw = 1.0 + rnd(K, seed=5, scale=0.1)
    w = rnd(2 * I, K, dtype=torch.bfloat16, seed=6, scale=1.0 / math.sqrt(K))
    eps = 1e-5
    xs = f64(x)[:M]
    operand = bf(xs * f64(nw))                                   # what the kernel multiplies: bf16(x * w_norm) ...
    scale = 1.0 / np.sqrt((xs * xs).mean(-1, keepdims=True) + eps)   # ... and the row's factor afterwards
    gu = bf(operand @ f64(w).T * scale)
    want = P.swiglu(gu[:, :I], gu[:, I:])
    got = ops.gemm_swiglu(x[:M], w, torch.empty(M, I, dtype=torch.bfloat16, device=DEV), norm=(nw, eps, None))
    np.testing.assert_allclose(f64(got), want, rtol=2e-2, atol=2e-3)
    h = torch.from_numpy(P.rmsnorm(xs, f64(nw), eps)).to(torch.bfloat16).to(DEV)
    gu = bf(f64(h) @ f64(w).T)
    got = ops.gemm_swiglu(h, w, torch.empty(M, I, dtype=torch.bfloat16, device=DEV))
    np.testing.assert_allclose(f64(got), P.swiglu(gu[:, :I], gu[:, I:]), rtol=2e-2, atol=2e-3)


@pytest.mark.parametrize("R, V, K", [(1, 3001, 576), (5, 1003, 200), (8, 49152, 576)])
def test_fused_norm_on_picked_rows(ops, R, V, K):
    """The output head: RMSNorm of the rows that `rows` picks, then the product with the vocabulary."""
    x = rnd(40, K, seed=7, scale=3.0)
    nw = 1.0 + rnd(K, seed=8, scale=0.1)
    w = rnd(V, K, dtype=torch.bfloat16, seed=9, scale=0.05)
    rows = torch.tensor([39, 0, 17, 17, 3, 8, 21, 30][:R], dtype=torch.int32, device=DEV)
    got = ops.gemm_normed(x, (nw, 1e-6, rows), w, torch.empty(R, V, device=DEV))
    xs = f64(x)[rows.cpu().numpy()]
    want = bf(xs * f64(nw)) @ f64(w).T / np.sqrt((xs * xs).mean(-1, keepdims=True) + 1e-6)
    np.testing.assert_allclose(f64(got), want, rtol=1e-4, atol=1e-5 * math.sqrt(K))
    if R >= 3:
        assert torch.equal(got[2], got[3]), "the same row picked twice"


@pytest.mark.parametrize("heads, kv_heads, dim, theta", [(4, 2, 16, 1e4), (9, 3, 64, 1e5), (6, 6, 32, 5e5), (32, 8, 128, 5e5)])
@pytest.mark.parametrize("normed", [True, False])
@pytest.mark.parametrize("M", [1, 3, 8])
def test_fused_projection_rotary_scatter(ops, heads, kv_heads, dim, theta, normed, M):
    from runtime.parts.position import RotaryEmbedding
    K, Pg, pages = (heads * dim if heads * dim <= 1024 else 1024), 8, 12
    rope = RotaryEmbedding(dim, theta, 200); rope.prepare(torch.device(DEV), torch.bfloat16)
    cos, sin = rope.tables()
    W = rnd((heads + 2 * kv_heads) * dim, K, dtype=torch.bfloat16, seed=10, scale=1.0 / math.sqrt(K))
    x = rnd(M, K, seed=11, scale=2.0)
    nw = 1.0 + rnd(K, seed=12, scale=0.1)
    positions = torch.tensor([0, 199, 5, 77, 8, 130, 64, 1][:M], dtype=torch.int32, device=DEV)
    slots = torch.tensor([3, 95, 40, 8, 17, 66, 7, 50][:M], dtype=torch.int32, device=DEV)
    kc = torch.zeros(pages, kv_heads, Pg, dim, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(pages, kv_heads, dim, Pg, dtype=torch.bfloat16, device=DEV)
    q = torch.zeros(M, heads * dim, dtype=torch.bfloat16, device=DEV)
    xs = f64(x)
    if normed:
        a = x
        qkv = bf(xs * f64(nw)) @ f64(W).T / np.sqrt((xs * xs).mean(-1, keepdims=True) + 1e-5)
        ops.qkv_rope(a, W, q, positions, slots, cos, sin, kc, vc, heads, kv_heads, dim, Pg, norm=(nw, 1e-5))
    else:
        a = x.to(torch.bfloat16)
        qkv = f64(a) @ f64(W).T
        ops.qkv_rope(a, W, q, positions, slots, cos, sin, kc, vc, heads, kv_heads, dim, Pg)
    pos = positions.cpu().numpy()
    want_q = P.rope(qkv[:, :heads * dim].reshape(M, heads, dim), pos, theta)
    want_k = P.rope(qkv[:, heads * dim:(heads + kv_heads) * dim].reshape(M, kv_heads, dim), pos, theta)
    want_v = qkv[:, (heads + kv_heads) * dim:].reshape(M, kv_heads, dim)
    np.testing.assert_allclose(f64(q).reshape(M, heads, dim), want_q, rtol=2e-2, atol=2e-2)
    for m, slot in enumerate(slots.cpu().tolist()):
        np.testing.assert_allclose(f64(kc[slot // Pg, :, slot % Pg, :]), want_k[m], rtol=2e-2, atol=2e-2)
        np.testing.assert_allclose(f64(vc[slot // Pg, :, :, slot % Pg]), want_v[m], rtol=2e-2, atol=2e-2)
    written = torch.zeros(pages * Pg, dtype=torch.bool)
    written[slots.cpu().long()] = True
    assert (kc.permute(0, 2, 1, 3).reshape(pages * Pg, -1)[~written] == 0).all(), "a key was written to a slot of no row"
    assert (vc.permute(0, 3, 1, 2).reshape(pages * Pg, -1)[~written] == 0).all(), "a value was written to a slot of no row"


@pytest.mark.parametrize("M, heads, dim, splits, N", [(1, 9, 64, 8, 576), (8, 9, 64, 8, 576), (3, 4, 16, 2, 72), (1, 32, 128, 8, 4096), (5, 32, 64, 4, 2048)])
def test_output_projection_merges_split_attention_itself(ops, M, heads, dim, splits, N):
    K = heads * dim
    assert ops.gemm_merged_ok(M, rnd(N, K, dtype=torch.bfloat16), heads, dim, splits)
    g = torch.Generator().manual_seed(M + splits)
    part_o = (torch.randn(M, heads, splits, dim, generator=g)).to(torch.bfloat16).to(DEV)
    stats = torch.stack([torch.randn(M, heads, splits, generator=g) * 3, torch.rand(M, heads, splits, generator=g) + 0.1], dim=-1).to(DEV)
    stats[0, 0, 1:, 1] = 0.0                     # splits that saw no key
    if M > 1:
        stats[1, :, :, 1] = 0.0                  # a row without any key: zeros
    w = rnd(N, K, dtype=torch.bfloat16, seed=4, scale=1.0 / math.sqrt(K))
    r = rnd(M, N, seed=5)
    m, l = f64(stats[..., 0]), f64(stats[..., 1])
    wts = np.where(l > 0, np.exp2(m - m.max(-1, keepdims=True)) * l, 0.0)
    den = wts.sum(-1)
    merged = (wts[..., None] * f64(part_o)).sum(2) / np.where(den > 0, den, 1.0)[..., None] * (den > 0)[..., None]
    want = f64(r) + bf(merged.reshape(M, K)) @ f64(w).T
    got = ops.gemm_merged((part_o, stats.contiguous(), splits), heads, dim, w, torch.empty(M, N, device=DEV), r)
    np.testing.assert_allclose(f64(got), want, rtol=1e-3, atol=2e-3)


def test_which_products_take_this_kernel(ops):
    w = rnd(64, 128, dtype=torch.bfloat16)
    assert ops.gemv_ok(8, 64, 128) and not ops.gemv_ok(9, 64, 128) and not ops.gemv_ok(4, 64, 100)      # (an inner size that is no multiple of 8)
    assert not ops.gemv_ok(8, 64, 16384)                                                            # eight rows of it do not fit LDS
    assert ops.gemv_ok(4, 64, 16384)
    assert not ops.wide_ok(8, w)
    ops.set_gemv()              # the engine's rule: up to four rows, weights of 4 MB and more
    try:
        assert ops.gemv_ok(1, 2048, 2048) and ops.gemv_ok(2, 6144, 4096) and ops.gemv_ok(1, 49152, 2048)
        assert not ops.gemv_ok(1, 49152, 576)          # rows of W too short to fill a wave's lanes twice
        assert ops.gemv_ok(3, 6144, 4096) and ops.gemv_ok(4, 6144, 4096) and not ops.gemv_ok(5, 6144, 4096) and not ops.gemv_ok(1, 3072, 576)
        ops.set_gemv(0)
        assert not ops.gemv_ok(1, 6144, 4096)
    finally:
        ops.set_gemv(8, 0)
