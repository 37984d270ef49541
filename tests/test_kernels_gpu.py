"""Each HIP kernel alone against a plain float64 reference, at sizes other than
the engine's tiny configurations (tails, non powers of two, every head size)."""
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
    return o


@pytest.fixture(autouse=True)
def other_kernels_take_few_rows(no_gemv):
    """This module is about the kernels that take products of 9 rows and more, which its tests also run with fewer
    rows; the matrix-vector kernel, which would take those, has a module of its own (test_gemv_gpu.py)."""


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def f64(t):
    return t.detach().double().cpu().numpy()


def test_library_is_loaded_from_the_tree(ops):
    from runtime.kernels import library
    assert library.loaded_path() and "libcisr_kernels_" in library.loaded_path()


def test_bf16_rounding_vector(ops):
    # reference tests/test_precision.py:65-70: specials kept, -0 keeps its sign, ties to even
    values = torch.tensor([0., -0., math.inf, -math.inf, math.nan, 1., 1.00390625, 1.01171875], device=DEV)
    out = ops.f32_to_bf16(values, torch.empty(8, dtype=torch.bfloat16, device=DEV)).float().cpu().numpy()
    assert np.isnan(out[4])
    np.testing.assert_array_equal(out[:4], values.cpu().numpy()[:4])
    assert np.signbit(out[1]) and out[5] == 1.0 and out[6] == 1.0   # 1 + 2^-8 is a tie: rounds to even (1.0)
    assert out[7] == 1.015625                                        # 1 + 3*2^-8 ties up to the even 1 + 2^-6
    x = rnd(1000, seed=3)
    np.testing.assert_array_equal(ops.f32_to_bf16(x, torch.empty(1000, dtype=torch.bfloat16, device=DEV)).float().cpu().numpy(),
                                  x.bfloat16().float().cpu().numpy())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding(ops, dtype):
    table = rnd(37, 70, dtype=dtype)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = ops.embedding(ids, table, torch.empty(5, 70, device=DEV))
    np.testing.assert_array_equal(f64(out), f64(table)[ids.cpu().numpy()])


@pytest.mark.parametrize("dim", [10, 64, 130, 576, 2048, 4100, 8200])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(ops, dim, out_dtype):
    # reference tests/test_cuda.py:28-36 (dims 10/64/130/512)
    x, w = rnd(7, dim, seed=1, scale=3.0), rnd(dim, seed=2)
    for eps in (1e-5, 1e-2):
        out = ops.rmsnorm(x, w, torch.empty(7, dim, dtype=out_dtype, device=DEV), eps)
        np.testing.assert_allclose(f64(out), P.rmsnorm(f64(x), f64(w), eps), **tol(out_dtype))
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    out = ops.rmsnorm(x, w, torch.empty(3, dim, dtype=out_dtype, device=DEV), 1e-6, rows)
    np.testing.assert_allclose(f64(out), P.rmsnorm(f64(x)[[6, 0, 3]], f64(w), 1e-6), **tol(out_dtype))
    assert (ops.rmsnorm(torch.zeros(2, dim, device=DEV), w, torch.empty(2, dim, dtype=out_dtype, device=DEV), 1e-5) == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm_and_residual_add(ops, dtype):
    x, d, w = rnd(5, 130, seed=1), rnd(5, 130, dtype=dtype, seed=2), rnd(130, seed=3)
    want_sum = f64(x) + f64(d)
    x1 = x.clone()
    out = ops.add_rmsnorm(x1, d, w, torch.empty(5, 130, dtype=dtype, device=DEV), 1e-5)
    np.testing.assert_allclose(f64(x1), want_sum, rtol=1e-6, atol=1e-6)       # the sum stays float
    np.testing.assert_allclose(f64(out), P.rmsnorm(want_sum, f64(w), 1e-5), **tol(dtype))
    x2 = x.clone()
    ops.residual_add(x2, d)
    np.testing.assert_allclose(f64(x2), want_sum, rtol=1e-6, atol=1e-6)
    # widths of whole 16-byte runs take the form with eight elements a thread (bf16 delta)
    x, d = rnd(7, 136, seed=4), rnd(7, 136, dtype=dtype, seed=5)
    x3 = x.clone()
    ops.residual_add(x3, d)
    np.testing.assert_allclose(f64(x3), f64(x) + f64(d), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu(ops, dtype):
    gu = rnd(6, 2 * 173, dtype=dtype, scale=4.0)
    gu[0, 0], gu[0, 1], gu[0, 2] = 0.0, 60.0, -60.0
    out = ops.swiglu(gu, torch.empty(6, 173, dtype=dtype, device=DEV))
    np.testing.assert_allclose(f64(out), P.swiglu(f64(gu)[:, :173], f64(gu)[:, 173:]), **tol(dtype))
    assert torch.isfinite(out.float()).all() and out[0, 0] == 0
    # a width of whole 16-byte runs takes the form with eight elements a thread (bf16)
    gu = rnd(5, 2 * 176, dtype=dtype, scale=4.0, seed=9)
    gu[1, 7], gu[1, 8], gu[1, 175] = 0.0, 60.0, -60.0
    out = ops.swiglu(gu, torch.empty(5, 176, dtype=dtype, device=DEV))
    np.testing.assert_allclose(f64(out), P.swiglu(f64(gu)[:, :176], f64(gu)[:, 176:]), **tol(dtype))
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv_heads, dim, theta", [(4, 2, 10, 1e4), (6, 6, 24, 5e5), (9, 3, 64, 1e5), (2, 1, 256, 1e4)])
def test_rope_scatter(ops, dtype, heads, kv_heads, dim, theta):
    # reference tests/test_cuda.py:37-39 (D=10, positions 0/17/500)
    from runtime.parts import RotaryEmbedding
    rope = RotaryEmbedding(dim, theta, 600)
    rope.prepare(DEV, dtype)
    cos, sin = rope.tables()
    T, P_, pages = 5, 4, 6
    qkv = rnd(T, (heads + 2 * kv_heads) * dim, dtype=dtype, seed=4)
    ref = f64(qkv)
    pos = [0, 17, 500, 599, 3]
    slots = [5, 0, 22, -1, 9]
    kc = torch.full((pages, kv_heads, P_, dim), 7.0, dtype=dtype, device=DEV)
    vc = torch.full((pages, kv_heads, dim, P_), 7.0, dtype=dtype, device=DEV)   # values: transposed inside a page
    ops.rope_scatter(qkv, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                     cos, sin, kc, vc, heads, kv_heads, dim, P_)
    q_ref = P.rope(ref[:, :heads * dim].reshape(T, heads, dim), pos, theta)
    k_ref = P.rope(ref[:, heads * dim:(heads + kv_heads) * dim].reshape(T, kv_heads, dim), pos, theta)
    v_ref = ref[:, (heads + kv_heads) * dim:].reshape(T, kv_heads, dim)
    np.testing.assert_allclose(f64(qkv)[:, :heads * dim].reshape(T, heads, dim), q_ref, **tol(dtype))
    kc64, vc64 = f64(kc), f64(vc)
    written = set()
    for t, s in enumerate(slots):
        if s < 0:
            continue
        np.testing.assert_allclose(kc64[s // P_, :, s % P_], k_ref[t], **tol(dtype))
        np.testing.assert_array_equal(vc64[s // P_, :, :, s % P_], v_ref[t])
        written.add(s)
    for s in range(pages * P_):
        if s not in written:   # nothing else is touched, a negative slot writes nothing
            assert (kc64[s // P_, :, s % P_] == 7).all() and (vc64[s // P_, :, :, s % P_] == 7).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv_heads, dim, rot", [(4, 2, 10, 10), (9, 3, 64, 64), (5, 1, 24, 16)])
def test_rope_scatter_with_interleaved_pairs(ops, dtype, heads, kv_heads, dim, rot):
    """The pairing rule is a parameter of the rotary kernel: pair i is coordinates (2i, 2i + 1) instead of
    (i, i + rot/2); with rot < dim the coordinates from rot on pass through.  Checked against complex
    multiplication of (x[2i] + j x[2i+1]) by exp(j angle); the split-half rule on the same rows must differ."""
    from runtime.parts import RotaryEmbedding
    theta = 1e4
    rope = RotaryEmbedding(dim, theta, 600, rotary_dim=rot, pairing="interleaved")
    rope.prepare(DEV, dtype)
    cos, sin = rope.tables()
    T, P_, pages = 4, 4, 5
    qkv = rnd(T, (heads + 2 * kv_heads) * dim, dtype=dtype, seed=12)
    ref = f64(qkv)
    pos, slots = [0, 17, 500, 3], [6, 1, 19, 8]
    kc = torch.zeros((pages, kv_heads, P_, dim), dtype=dtype, device=DEV)
    vc = torch.zeros((pages, kv_heads, dim, P_), dtype=dtype, device=DEV)
    split = qkv.clone()
    ops.rope_scatter(qkv, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                     cos, sin, kc, vc, heads, kv_heads, dim, P_, interleaved=True)

    def turn(x):          # [T, heads, dim]
        angle = np.asarray(pos, np.float64)[:, None] * (theta ** (-np.arange(rot // 2) * 2.0 / rot))[None, :]
        z = (x[..., 0:rot:2] + 1j * x[..., 1:rot:2]) * np.exp(1j * angle)[:, None, :]
        out = x.copy()
        out[..., 0:rot:2], out[..., 1:rot:2] = z.real, z.imag
        return out

    q_ref = turn(ref[:, :heads * dim].reshape(T, heads, dim))
    k_ref = turn(ref[:, heads * dim:(heads + kv_heads) * dim].reshape(T, kv_heads, dim))
    np.testing.assert_allclose(f64(qkv)[:, :heads * dim].reshape(T, heads, dim), q_ref, **tol(dtype))
    for t, s in enumerate(slots):
        np.testing.assert_allclose(f64(kc)[s // P_, :, s % P_], k_ref[t], **tol(dtype))
        np.testing.assert_array_equal(f64(vc)[s // P_, :, :, s % P_], ref[t, (heads + kv_heads) * dim:].reshape(kv_heads, dim))
    ops.rope_scatter(split, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                     cos, sin, torch.zeros_like(kc), torch.zeros_like(vc), heads, kv_heads, dim, P_)
    assert np.abs(f64(split)[1:, :heads * dim] - f64(qkv)[1:, :heads * dim]).max() > 1e-2      # the other rule gives other rows


@pytest.mark.parametrize("heads, kv_heads, dim, page_size, T, start", [
    (9, 3, 64, 16, 100, None), (4, 4, 16, 4, 37, None), (3, 1, 128, 16, 33, None), (34, 34, 32, 8, 50, None),
    (9, 3, 64, 16, 100, 0), (34, 34, 32, 16, 70, 16), (3, 1, 128, 32, 64, 8), (4, 2, 64, 16, 48, 5), (32, 32, 64, 16, 64, 0)])
def test_rope_scatter_of_portions(ops, heads, kv_heads, dim, page_size, T, start):
    """Portions of 32 rows and more (bf16, whole heads turn) write their values through LDS, 16 rows a block: runs of
    consecutive slots, slots that jump between pages and requests, rows without a slot, more value columns than one
    pass holds, a last block that is not full; nothing but the slots given is written.  With `start` the rows are one
    request's positions from there on, page after page (tiles that are one run inside a page are written 32 bytes a
    coordinate), with a few rows without a slot among them."""
    from runtime.parts import RotaryEmbedding
    theta = 1e4
    rope = RotaryEmbedding(dim, theta, 700)
    rope.prepare(DEV, torch.bfloat16)
    cos, sin = rope.tables()
    rng = np.random.default_rng(T)
    pages = T + 5             # a run takes a page of its own
    free = rng.permutation(pages).tolist()
    slots, pos = [], []
    if start is not None:
        own = [free.pop() for _ in range(-(-(start + T) // page_size))]
        slots = [own[(start + i) // page_size] * page_size + (start + i) % page_size for i in range(T)]
        pos = [start + i for i in range(T)]
    while len(slots) < T:      # runs of consecutive slots of random length, each from the start of a free page or inside it
        run = int(rng.integers(1, 2 * page_size))
        page, off, p0 = free.pop(), int(rng.integers(0, page_size)), int(rng.integers(0, 600))
        for i in range(min(run, page_size - off, T - len(slots))):
            slots.append(page * page_size + off + i); pos.append(p0 + i)
    for i in rng.choice(T, 3, replace=False):
        slots[i] = -1
    qkv = rnd(T, (heads + 2 * kv_heads) * dim, dtype=torch.bfloat16, seed=5)
    ref = f64(qkv)
    kc = torch.full((pages, kv_heads, page_size, dim), 7.0, dtype=torch.bfloat16, device=DEV)
    vc = torch.full((pages, kv_heads, dim, page_size), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.rope_scatter(qkv, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                     cos, sin, kc, vc, heads, kv_heads, dim, page_size)
    q_ref = P.rope(ref[:, :heads * dim].reshape(T, heads, dim), pos, theta)
    k_ref = P.rope(ref[:, heads * dim:(heads + kv_heads) * dim].reshape(T, kv_heads, dim), pos, theta)
    v_ref = ref[:, (heads + kv_heads) * dim:].reshape(T, kv_heads, dim)
    np.testing.assert_allclose(f64(qkv)[:, :heads * dim].reshape(T, heads, dim), q_ref, **tol(torch.bfloat16))
    kc64, vc64 = f64(kc), f64(vc)
    want_k, want_v = np.full(kc64.shape, 7.0), np.full(vc64.shape, 7.0)
    for t, s in enumerate(slots):
        if s >= 0:
            want_k[s // page_size, :, s % page_size] = k_ref[t]
            want_v[s // page_size, :, :, s % page_size] = v_ref[t]
    np.testing.assert_array_equal(vc64, want_v)
    np.testing.assert_allclose(kc64, want_k, **tol(torch.bfloat16))


def test_rope_partial_rotation_and_identity(ops):
    from runtime.parts import RotaryEmbedding, NoPosition
    dim, rot = 16, 8
    rope = RotaryEmbedding(dim, 1e4, 50, rotary_dim=rot); rope.prepare(DEV, torch.float32)
    qkv = rnd(3, 3 * dim, seed=9); ref = f64(qkv)
    kc = torch.zeros(1, 1, 4, dim, device=DEV); vc = torch.zeros(1, 1, dim, 4, device=DEV)
    pos = [3, 40, 7]
    ops.rope_scatter(qkv, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV),
                     *rope.tables(), kc, vc, 1, 1, dim, 4)
    q = ref[:, :dim].reshape(3, 1, dim)
    want = np.concatenate([P.rope(q[..., :rot], pos, 1e4), q[..., rot:]], -1)
    np.testing.assert_allclose(f64(qkv)[:, :dim].reshape(3, 1, dim), want, rtol=2e-5, atol=2e-6)
    k = ref[:, dim:2 * dim].reshape(3, 1, dim)
    want_k = np.concatenate([P.rope(k[..., :rot], pos, 1e4), k[..., rot:]], -1)
    np.testing.assert_allclose(f64(kc)[0, :, :3].transpose(1, 0, 2), want_k, rtol=2e-5, atol=2e-6)
    none = NoPosition(dim, 50); none.prepare(DEV, torch.float32)
    qkv2 = rnd(3, 3 * dim, seed=9)
    ops.rope_scatter(qkv2, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV),
                     *none.tables(), kc, vc, 1, 1, dim, 4)
    np.testing.assert_array_equal(f64(qkv2), ref)


def paged_case(heads, kv_heads, dim, page_size, lengths, dtype, seed=0, pages=None, sharpen=None):
    """A cache with scattered pages holding `lengths[i]` keys for request i, one
    query row per request at its last position plus extra rows at earlier positions."""
    rng = np.random.default_rng(seed)
    per = [-(-n // page_size) for n in lengths]
    pages = pages or sum(per) + 3
    order = rng.permutation(pages).tolist()
    width = max(per) + 2
    tables = np.full((len(lengths), width), -1, np.int32)
    K = rng.standard_normal((pages, kv_heads, page_size, dim)).astype(np.float32)
    V = rng.standard_normal((pages, kv_heads, page_size, dim)).astype(np.float32)
    for i, n in enumerate(lengths):
        for j in range(per[i]):
            tables[i, j] = order.pop()
    rows = []  # (segment, position)
    for i, n in enumerate(lengths):
        rows.append((i, n - 1))
        if n > 3:
            rows.append((i, n // 2))
            rows.append((i, 0))
    q = rng.standard_normal((len(rows), heads, dim)).astype(np.float32)
    if sharpen is not None:   # one far key gets a score that stands out
        seg, key_pos = sharpen
        page, off = tables[seg, key_pos // page_size], key_pos % page_size
        r = next(i for i, (s, p) in enumerate(rows) if s == seg and p == lengths[seg] - 1)
        group = heads // kv_heads
        for h in range(heads):   # heads of one group ask the same question, the key answers it
            q[r, h] = q[r, (h // group) * group]
            K[page, h // group, off] = q[r, h] * 4.0
    kt = torch.from_numpy(K).to(dtype).to(DEV)
    vt = torch.from_numpy(np.ascontiguousarray(V.transpose(0, 1, 3, 2))).to(dtype).to(DEV)   # [pages, kv, D, P]
    qt = torch.from_numpy(q).to(dtype).to(DEV)
    return qt, kt, vt, torch.from_numpy(tables).to(DEV), rows


def reference_attention(qt, kt, vt, tables, rows, page_size, window=None, scale=None):
    q, K, V, tab = f64(qt), f64(kt), f64(vt).transpose(0, 1, 3, 2), tables.cpu().numpy()
    out = []
    for r, (seg, pos) in enumerate(rows):
        lo = 0 if not window else max(0, pos + 1 - window)
        ks = np.stack([K[tab[seg, t // page_size], :, t % page_size] for t in range(lo, pos + 1)])
        vs = np.stack([V[tab[seg, t // page_size], :, t % page_size] for t in range(lo, pos + 1)])
        qq = q[r] if scale is None else q[r] * scale * math.sqrt(q.shape[-1])
        out.append(P.attention_one_query(qq, ks, vs))
    return np.stack(out)


def run_rowwise(ops, qt, kt, vt, tables, rows, page_size, splits=1, window=None, scale=None):
    T, heads, dim = qt.shape
    kv_heads = kt.shape[1]
    seg = torch.tensor([r[0] for r in rows], dtype=torch.int32, device=DEV)
    pos = torch.tensor([r[1] for r in rows], dtype=torch.int32, device=DEV)
    out = torch.empty(T, heads * dim, dtype=qt.dtype, device=DEV)
    ws = (torch.empty(T * heads * splits * dim, device=DEV), torch.empty(T * heads * splits * 2, device=DEV))
    ops.attention_rowwise(qt.reshape(T, heads * dim), heads * dim, kt, vt, tables, seg, pos, out, heads, kv_heads, dim,
                          page_size, window, scale if scale is not None else 1 / math.sqrt(dim), splits, ws)
    return f64(out).reshape(T, heads, dim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv_heads, dim, page_size", [
    (4, 2, 10, 4), (6, 6, 24, 8), (9, 3, 64, 16), (8, 1, 128, 64), (2, 2, 256, 1), (5, 5, 16, 3)])
def test_attention_rowwise(ops, dtype, heads, kv_heads, dim, page_size):
    # reference tests/test_cuda.py:41-63: head sizes 10..256, interleaved pages, grouped heads,
    # split counts 1/3/16 where 16 exceeds the shorter request's tokens
    qt, kt, vt, tables, rows = paged_case(heads, kv_heads, dim, page_size, [17, 7, 1, 130], dtype, seed=dim)
    want = reference_attention(qt, kt, vt, tables, rows, page_size)
    for splits in (1, 3, 16, 33):
        got = run_rowwise(ops, qt, kt, vt, tables, rows, page_size, splits)
        np.testing.assert_allclose(got, want, **tol(dtype), err_msg=f"splits={splits}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_window_scale_and_padding_rows(ops, dtype):
    qt, kt, vt, tables, rows = paged_case(4, 2, 32, 8, [70, 9], dtype, seed=11)
    for window in (1, 8, 9, 33):   # the edge: exactly `window` keys lo..pos
        want = reference_attention(qt, kt, vt, tables, rows, 8, window=window)
        for splits in (1, 4):
            np.testing.assert_allclose(run_rowwise(ops, qt, kt, vt, tables, rows, 8, splits, window=window), want, **tol(dtype))
    want = reference_attention(qt, kt, vt, tables, rows, 8, scale=0.3)
    np.testing.assert_allclose(run_rowwise(ops, qt, kt, vt, tables, rows, 8, 1, scale=0.3), want, **tol(dtype))
    # a row without a segment (padding) gives zeros and touches nothing else
    rows2 = list(rows); rows2[1] = (-1, 0)
    got = run_rowwise(ops, qt, kt, vt, tables, rows2, 8, 2)
    assert (got[1] == 0).all()
    np.testing.assert_allclose(got[0], reference_attention(qt, kt, vt, tables, rows, 8)[0], **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_one_far_key_among_hundreds(ops, dtype):
    # key 3 of 700 carries a score far above the rest: the output must be its value row
    qt, kt, vt, tables, rows = paged_case(4, 2, 64, 16, [700, 40], dtype, seed=5, sharpen=(0, 3))
    want = reference_attention(qt, kt, vt, tables, rows, 16)
    page, off = tables[0, 0].item(), 3
    np.testing.assert_allclose(want[0, 0], f64(vt)[page, 0, :, off], atol=1e-6)   # the case is what it claims to be
    for splits in (1, 8):
        np.testing.assert_allclose(run_rowwise(ops, qt, kt, vt, tables, rows, 16, splits), want, **tol(dtype))


def test_attention_equal_large_scores_give_the_mean(ops):
    # reference tests/test_reference.py:7-13 on the kernel
    heads, kv, dim, n = 4, 2, 8, 3
    q = torch.full((1, heads * dim), 1e3, device=DEV)
    kc = torch.full((1, kv, 4, dim), 1e3, device=DEV)
    vc = torch.arange(kv * 4 * dim, dtype=torch.float32, device=DEV).reshape(1, kv, dim, 4)
    out = torch.empty(1, heads * dim, device=DEV)
    ops.attention_rowwise(q, heads * dim, kc, vc, torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                          torch.zeros(1, dtype=torch.int32, device=DEV), torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                          out, heads, kv, dim, 4, None, 1 / math.sqrt(dim))
    assert torch.isfinite(out).all()
    np.testing.assert_allclose(f64(out).reshape(heads, dim)[0], f64(vc)[0, 0, :, :n].mean(-1), rtol=1e-6)
    np.testing.assert_allclose(f64(out).reshape(heads, dim)[3], f64(vc)[0, 1, :, :n].mean(-1), rtol=1e-6)


def run_mfma(ops, qt, kt, vt, tables, rows, page_size, mode, splits=1, window=None, scale=None, rows_per_tile=None, waves=4,
             row_ids=None, positions_given=False):
    """mode "tiles": rows are grouped into tiles of consecutive rows of one segment;
    mode "rows": one block per row with `splits` blocks along the keys."""
    T, heads, dim = qt.shape
    kv_heads = kt.shape[1]
    seg = torch.tensor([r[0] for r in rows], dtype=torch.int32, device=DEV)
    pos = torch.tensor([r[1] for r in rows], dtype=torch.int32, device=DEV)
    out = torch.full((T, heads * dim), 9.0, dtype=qt.dtype, device=DEV)
    tasks = None
    ws = (torch.empty(T * heads * splits * dim, device=DEV), torch.empty(T * heads * splits * 2, device=DEV))
    # ("square...": blocks on the 32 x 32 instruction; "...halves": two halves a block for the even and the odd steps)
    items_of = {"tiles": 16, "tiles2": 32, "block": 64, "block2": 128, "square": 64, "square2": 128, "square3": 192, "square4": 256,
                "square_halves": 64, "square2_halves": 128}
    if mode in items_of:
        group = heads // kv_heads
        rpt = rows_per_tile or items_of[mode] // min(group, 16)
        items, i = [], 0
        while i < T:   # consecutive rows of one segment with consecutive positions form a tile
            n = 1
            while i + n < T and n < rpt and rows[i + n][0] == rows[i][0] and rows[i + n][1] == rows[i + n - 1][1] + 1:
                n += 1
            # (the fourth entry: the position of the tile's first row plus one, or 0 for "read the positions array")
            items.append((rows[i][0], i, n, rows[i][1] + 1 if positions_given else 0)); i += n
        tasks = torch.tensor(items, dtype=torch.int32, device=DEV)
    ops.attention_mfma(qt.reshape(T, heads * dim), heads * dim, kt, vt, tables, seg, pos, out, heads, kv_heads, dim,
                       page_size, window, scale if scale is not None else 1 / math.sqrt(dim), tasks, splits, ws, waves,
                       block_tiles=32 if mode.startswith("square") else mode.startswith("block"),
                       item_tiles=(4 if mode == "square4" else 3 if mode == "square3" else 2 if mode in ("tiles2", "block2", "square2", "square2_halves") else 1),
                       key_groups=2 if mode.endswith("_halves") else 1,
                       row_ids=None if row_ids is None else torch.tensor(row_ids, dtype=torch.int32, device=DEV))
    return f64(out).reshape(T, heads, dim)


MFMA_WORST, MFMA_RMS = 8e-3, 4e-3
_mfma_seen = {"worst": 0.0, "rms": 0.0}


def close_mfma(got, want, err_msg=""):
    """Matrix-core attention against the float64 reference: the largest difference as a part of the largest output,
    and the relative root-mean-square difference.  bfloat16 rounds the weights inside the kernel and the outputs
    at 2^-9 each; what the kernels come to is printed at the end of the module (worst 3.5e-3, rms 2.2e-3 when the bounds were set).
    One key dropped, doubled or taken from a wrong page among the tens to hundreds of a row moves that row by
    several hundredths of the largest output."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape and np.isfinite(got).all(), err_msg
    worst = np.abs(got - want).max() / np.abs(want).max()
    rms = np.linalg.norm(got - want) / np.linalg.norm(want)
    _mfma_seen["worst"], _mfma_seen["rms"] = max(_mfma_seen["worst"], worst), max(_mfma_seen["rms"], rms)
    assert worst < MFMA_WORST and rms < MFMA_RMS, f"{err_msg}: worst {worst:.2e} (bound {MFMA_WORST}), rms {rms:.2e} (bound {MFMA_RMS})"


def teardown_module(module):
    print(f"\nmatrix-core attention against its reference: worst {_mfma_seen['worst']:.2e} of the largest output, rms {_mfma_seen['rms']:.2e}")


def square_modes(dim):
    """The forms of the 32 x 32 kernel that take this head size (blocks of more than eight waves: up to 64)."""
    return ("square", "square2", "square3", "square_halves") + (("square4", "square2_halves") if dim <= 64 else ())


@pytest.mark.parametrize("heads, kv_heads, dim, page_size", [
    (4, 2, 16, 8), (6, 6, 24, 8), (9, 3, 64, 16), (8, 1, 128, 64), (2, 2, 256, 8), (5, 5, 40, 16), (32, 1, 64, 16), (20, 1, 32, 8)])
def test_attention_mfma_rows(ops, heads, kv_heads, dim, page_size):
    """Decode form: single rows at scattered positions, every split count, including more splits than 32-key steps."""
    qt, kt, vt, tables, rows = paged_case(heads, kv_heads, dim, page_size, [17, 7, 1, 130, 333], torch.bfloat16, seed=dim + heads)
    want = reference_attention(qt, kt, vt, tables, rows, page_size)
    for splits in (1, 2, 3, 16, 40):
        for waves in (4, 8):
            got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "rows", splits, waves=waves)
            close_mfma(got, want, f"splits={splits} waves={waves}")
    rows2 = list(rows); rows2[0] = (-1, 0)            # a padding row gives zeros
    got = run_mfma(ops, qt, kt, vt, tables, rows2, page_size, "rows", 2)
    assert (got[0] == 0).all()
    close_mfma(got[1:], want[1:])
    again = [run_mfma(ops, qt, kt, vt, tables, rows, page_size, "rows", 16) for _ in range(3)]
    assert all((a == again[0]).all() for a in again)  # the merge order is fixed: repeated runs agree bit for bit
    # a list of rows (the decode rows of a mixed step): only those are computed and written, a negative entry is none
    for splits in (1, 5, 20):
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "rows", splits, waves=8, row_ids=[3, -1, 0, -1])
        close_mfma(got[[3, 0]], want[[3, 0]], f"listed rows, splits={splits}")
        assert (got[[1, 2, 4]] == 9.0).all()


@pytest.mark.parametrize("heads, kv_heads, dim, page_size", [(9, 3, 64, 16), (4, 2, 32, 8), (8, 2, 128, 32), (6, 6, 24, 8)])
def test_attention_mfma_rows_over_many_steps(ops, heads, kv_heads, dim, page_size):
    """Decode form with many 32-key steps a wave (long contexts, few or no splits): the loop that keeps several steps'
    loads in flight, with wave counts and splits that give a wave 1 to 35 steps, a far key that stands out, and a
    window whose passed pages are gone from the table."""
    lengths = [1100, 97, 705, 2]
    qt, kt, vt, tables, rows = paged_case(heads, kv_heads, dim, page_size, lengths, torch.bfloat16, seed=3 * dim + heads, sharpen=(0, 5))
    want = reference_attention(qt, kt, vt, tables, rows, page_size)
    for splits in (1, 2, 5):
        for waves in (4, 8):
            got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "rows", splits, waves=waves)
            close_mfma(got, want, f"splits={splits} waves={waves}")
    window = 300
    want_w = reference_attention(qt, kt, vt, tables, rows, page_size, window=window)
    t2 = tables.clone()
    first_needed = min(p + 1 - window for s, p in rows if s == 0 and p + 1 > window)      # request 0: rows at 1099 and 550
    t2[0, :first_needed // page_size] = -1
    only = [i for i, (s, p) in enumerate(rows) if not (s == 0 and p + 1 <= window)]       # (its row at 0 needs page 0)
    for splits, waves in ((1, 8), (1, 4), (3, 8)):
        got = run_mfma(ops, qt[only].contiguous(), kt, vt, t2, [rows[i] for i in only], page_size, "rows", splits, waves=waves, window=window)
        close_mfma(got, want_w[only], f"window, splits={splits} waves={waves}")


def portion_case(heads, kv_heads, dim, page_size, plan, seed):
    """plan: [(cached keys before the portion, portion length)] per request: every row of every portion is a query."""
    rng = np.random.default_rng(seed)
    lengths = [a + b for a, b in plan]
    qt, kt, vt, tables, _ = paged_case(heads, kv_heads, dim, page_size, lengths, torch.bfloat16, seed=seed)
    rows = [(s, p) for s, (a, b) in enumerate(plan) for p in range(a, a + b)]
    q = rng.standard_normal((len(rows), heads, dim)).astype(np.float32)
    return torch.from_numpy(q).to(torch.bfloat16).to(DEV), kt, vt, tables, rows


@pytest.mark.parametrize("heads, kv_heads, dim, page_size", [
    (4, 2, 16, 8), (6, 6, 24, 8), (9, 3, 64, 16), (8, 2, 128, 16), (3, 3, 256, 64), (32, 1, 64, 16), (7, 7, 48, 16)])
def test_attention_mfma_tiles(ops, heads, kv_heads, dim, page_size):
    """Prompt portions: rows of a portion attend to the cached prefix and causally to
    the portion itself; portions of 1, 2 and many rows, starting at and off page edges."""
    plan = [(0, 70), (33, 2), (64, 1), (5, 37), (100, 45)]
    qt, kt, vt, tables, rows = portion_case(heads, kv_heads, dim, page_size, plan, seed=dim * 3 + heads)
    want = reference_attention(qt, kt, vt, tables, rows, page_size)
    got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "tiles")
    close_mfma(got, want)
    got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "tiles", waves=8)
    close_mfma(got, want)
    got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "tiles", rows_per_tile=1)   # tiles need not be full
    close_mfma(got, want)
    if dim <= 64:
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "tiles2")               # two item tiles a wave
        close_mfma(got, want)
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "tiles2", rows_per_tile=2)
        close_mfma(got, want)
    if dim > 128:                                                                        # block tiles: head sizes up to 128
        with pytest.raises(ops.KernelError):
            run_mfma(ops, qt, kt, vt, tables, rows, page_size, "block")
        return
    for mode in ("block", "block2"):                                                     # 64 / 128-item tiles through LDS
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, mode)
        close_mfma(got, want, mode)
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, mode, rows_per_tile=3)
        close_mfma(got, want, mode)
    if page_size < 8:                                                                    # 32 x 32 tiles: pages of at least 8 keys
        with pytest.raises(ops.KernelError):
            run_mfma(ops, qt, kt, vt, tables, rows, page_size, "square")
        return
    if dim > 64:
        with pytest.raises(ops.KernelError):
            run_mfma(ops, qt, kt, vt, tables, rows, page_size, "square4")
    for mode in square_modes(dim):                                                       # 64 / 128 / 192 / 256 items on the 32 x 32 instruction
        for given in (False, True):
            got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, mode, positions_given=given)
            close_mfma(got, want, f"{mode} positions given: {given}")
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, mode, rows_per_tile=3, positions_given=True)
        close_mfma(got, want, mode)


@pytest.mark.parametrize("heads, kv_heads, dim, page_size", [(4, 4, 64, 16), (6, 2, 128, 16), (5, 1, 96, 8), (2, 2, 32, 32)])
def test_attention_square_tiles_over_long_contexts(ops, heads, kv_heads, dim, page_size):
    """The 32 x 32 form keeps three steps of a tile in flight and moves the reference point of the exponentials only
    when the maximum has grown a lot: long prefixes (many plain steps before the diagonal), portions that start in the
    middle of a 32-key step, one key far above the rest late in the context (the reference point jumps, the outputs
    are rescaled), and tiles of every height."""
    plan = [(0, 300), (517, 130), (64, 33), (1000, 40)]
    qt, kt, vt, tables, rows = portion_case(heads, kv_heads, dim, page_size, plan, seed=dim + 7 * heads)
    # request 1: key 490 of its 647 carries a score far above the rest for every query of head 0
    page, off = tables[1, 490 // page_size].item(), 490 % page_size
    first = sum(b for _, b in plan[:1])
    direction = torch.nn.functional.normalize(qt[first:first + 130, 0].float().mean(0), dim=0)
    kt[page, 0, off, :] = (direction * 40).to(kt.dtype)
    qt[first:first + 130, 0] = (qt[first:first + 130, 0].float() + direction * 6).to(qt.dtype)
    want = reference_attention(qt, kt, vt, tables, rows, page_size)
    for mode in square_modes(dim):
        for rpt in (None, 5):
            got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, mode, rows_per_tile=rpt, positions_given=True)
            close_mfma(got, want, f"{mode} rows a tile: {rpt}")
    for window in (40, 257):
        want_w = reference_attention(qt, kt, vt, tables, rows, page_size, window=window)
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "square2", window=window, positions_given=True)
        close_mfma(got, want_w, f"window {window}")


@pytest.mark.parametrize("dim, page_size", [(64, 16), (128, 16), (32, 8)])
def test_attention_survives_scores_beyond_the_exponent_range(ops, dim, page_size):
    """One key whose score lies a thousand powers of two above every score before it (the weights computed with the
    old reference point overflow to infinity, which must be noticed and redone), and a prefix whose scores all lie far
    below the first key's (weights that underflow to zero must stay harmless): every form of the kernel against the
    plain softmax in float64."""
    heads, kv_heads = 4, 2
    plan = [(0, 200), (300, 70)]
    qt, kt, vt, tables, rows = portion_case(heads, kv_heads, dim, page_size, plan, seed=5 * dim)
    first = plan[0][1]
    direction = torch.nn.functional.normalize(qt[first:, 0].float().mean(0), dim=0)
    # request 1: key 330 (inside its portion) answers head 0 and 1 of every later row with a huge score
    page, off = tables[1, 330 // page_size].item(), 330 % page_size
    kt[page, 0, off, :] = (direction * 200).to(kt.dtype)
    qt[first:, 0] = (qt[first:, 0].float() + direction * 30).to(qt.dtype)
    qt[first:, 1] = qt[first:, 0]
    # request 0: key 0 towers over all that follow for head 2 (kv head 1): their weights underflow
    d0 = torch.nn.functional.normalize(qt[:first, 2].float().mean(0), dim=0)
    page0 = tables[0, 0].item()
    kt[page0, 1, 0, :] = (d0 * 200).to(kt.dtype)
    qt[:first, 2] = (qt[:first, 2].float() + d0 * 30).to(qt.dtype)
    want = reference_attention(qt, kt, vt, tables, rows, page_size)
    assert np.isfinite(want).all()
    modes = ["tiles", "block", "block2"] + list(square_modes(dim)) + (["tiles2"] if dim <= 64 else [])
    for mode in modes:
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, mode, positions_given=mode.startswith("square"))
        assert np.isfinite(got).all(), mode
        close_mfma(got, want, mode)
    for splits in (1, 3):
        got = run_mfma(ops, qt, kt, vt, tables, rows, page_size, "rows", splits)
        assert np.isfinite(got).all()
        close_mfma(got, want, f"rows, splits={splits}")


def test_attention_mfma_window_and_far_key(ops):
    qt, kt, vt, tables, rows = portion_case(4, 2, 32, 8, [(40, 30), (0, 9)], seed=21)
    for window in (1, 8, 9, 33, 64):
        want = reference_attention(qt, kt, vt, tables, rows, 8, window=window)
        close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 8, "tiles", window=window), want)
        close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 8, "block", window=window), want)
        close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 8, "block2", window=window), want)
        close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 8, "tiles2", window=window), want)
        for mode in square_modes(32):
            close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 8, mode, window=window), want, mode)
        close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 8, "rows", 2, window=window), want)
    want = reference_attention(qt, kt, vt, tables, rows, 8, scale=0.3)
    close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 8, "tiles", scale=0.3), want)
    # pages the window has passed are marked -1 in the table and must never be needed
    tables2 = tables.clone(); tables2[0, :4] = -1          # keys 0..31 of request 0; window 8 from position 40 starts at 33
    want = reference_attention(qt, kt, vt, tables, rows, 8, window=8)
    close_mfma(run_mfma(ops, qt, kt, vt, tables2, rows, 8, "tiles", window=8), want)
    close_mfma(run_mfma(ops, qt, kt, vt, tables2, rows, 8, "block", window=8), want)
    close_mfma(run_mfma(ops, qt, kt, vt, tables2, rows, 8, "block2", window=8), want)
    close_mfma(run_mfma(ops, qt, kt, vt, tables2, rows, 8, "square", window=8), want)
    close_mfma(run_mfma(ops, qt, kt, vt, tables2, rows, 8, "square2", window=8, positions_given=True), want)
    close_mfma(run_mfma(ops, qt, kt, vt, tables2, rows, 8, "rows", 3, window=8), want)
    # one far key among hundreds stands out
    qt, kt, vt, tables, rows = paged_case(4, 2, 64, 16, [700, 40], torch.bfloat16, seed=5, sharpen=(0, 3))
    want = reference_attention(qt, kt, vt, tables, rows, 16)
    for mode, splits in (("rows", 1), ("rows", 8), ("tiles", 1), ("block", 1), ("block2", 1), ("square", 1), ("square2", 1)):
        close_mfma(run_mfma(ops, qt, kt, vt, tables, rows, 16, mode, splits), want)


def test_attention_mfma_ignores_what_unseen_slots_hold(ops):
    """Pages are not cleared when they change owners: the slots of a request's last page behind its last key, and
    page 0 (read in place of a page that a window has passed), may hold anything, Inf and NaN included.  Keys there
    have weight zero, and their values must not reach the output (0 x Inf is NaN)."""
    heads, kv_heads, dim, P_ = 6, 2, 64, 16
    plan = [(21, 14), (0, 5), (70, 1)]                       # last keys at 34, 4 and 70: none at a page's end
    qt, kt, vt, tables, rows = portion_case(heads, kv_heads, dim, P_, plan, seed=77)
    tab = tables.cpu().numpy()
    poison = [float("inf"), float("-inf"), float("nan")]
    want = {}
    for window in (None, 16):
        want[window] = reference_attention(qt, kt, vt, tables, rows, P_, window=window)
    for s, (a, b) in enumerate(plan):
        last = a + b - 1
        page = tab[s, last // P_]
        for off in range(last % P_ + 1, P_):                 # the rest of the last page
            kt[page, :, off, :] = poison[off % 3]
            vt[page, :, :, off] = poison[(off + 1) % 3]
    used = {int(p) for p in tab.flatten() if p >= 0}
    spare = next(p for p in range(kt.shape[0]) if p not in used)
    kt[spare], vt[spare] = float("nan"), float("inf")        # a page of nobody's, standing in for page 0 below
    for window in (None, 16):
        t2 = tables.clone()
        if window:                                           # request 2 (position 70, window 16 from 55): pages 0..2 passed
            t2[2, :3] = -1
        for mode, splits in (("tiles", 1), ("tiles2", 1), ("block", 1), ("block2", 1), ("square", 1), ("square2", 1), ("square4", 1),
                             ("square_halves", 1), ("square2_halves", 1), ("rows", 1), ("rows", 3)):
            got = run_mfma(ops, qt, kt, vt, t2, rows, P_, mode, splits, window=window)
            assert np.isfinite(got).all(), f"{mode} window={window}: poison reached the output"
            close_mfma(got, want[window], f"{mode} window={window}")
    # page 0 itself poisoned, with a table whose passed pages read it
    if 0 not in {int(tab[2, j]) for j in range(3, 5)}:
        k0, v0 = kt[0].clone(), vt[0].clone()
        kt[0], vt[0] = float("nan"), float("nan")
        t2 = tables.clone(); t2[2, :3] = -1
        only = [i for i, (s, _) in enumerate(rows) if s == 2]
        sub_rows = [rows[i] for i in only]
        got = run_mfma(ops, qt[only].contiguous(), kt, vt, t2, sub_rows, P_, "rows", 2, window=16)
        assert np.isfinite(got).all()
        close_mfma(got, want[16][only])
        kt[0], vt[0] = k0, v0


def test_stream_read_reads_and_writes_nothing(ops):
    """The read-bandwidth probe of the benchmark: any size that is a multiple of 16 bytes, any number of blocks; it
    leaves its sink alone (the folded word never has the value that would be written)."""
    from runtime import measure
    sink = torch.zeros(4, dtype=torch.int32, device=DEV)
    for nbytes, blocks in ((16, 1), (4096, 3), (1 << 20, 512), (16 * 100003, 7), (48, 256)):
        buf = torch.arange(nbytes, dtype=torch.int64, device=DEV).to(torch.uint8)
        measure.stream_read(buf, sink, blocks)
    torch.cuda.synchronize()
    assert (sink == 0).all()
    with pytest.raises(ops.KernelError):
        measure.stream_read(torch.zeros(24, dtype=torch.uint8, device=DEV), sink)


def test_gemm_skinny_and_fused_swiglu(ops):
    """Few rows of bf16 run the weight-streaming kernel: every row count up to 64, output widths off
    the 16-column tile, float/bf16 outputs, residual, and the fused SwiGLU against the two-kernel path."""
    for M, N, K in [(1, 16, 32), (3, 100, 72), (8, 1728, 576), (16, 576, 1536), (17, 49, 264), (33, 130, 200), (64, 96, 4096), (50, 1003, 200)]:
        a, w, r = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2), rnd(M, N, seed=3)
        want = f64(a) @ f64(w).T
        np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, device=DEV))), want, rtol=1e-4, atol=1e-4 * math.sqrt(K))
        np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, dtype=torch.bfloat16, device=DEV))), want, rtol=1e-2, atol=1e-2 * math.sqrt(K))
        out = r.clone(); ops.gemm(a, w, out, residual=out)
        np.testing.assert_allclose(f64(out), want + f64(r), rtol=1e-4, atol=1e-4 * math.sqrt(K))
    for M, I, K in [(1, 16, 32), (8, 1536, 576), (40, 172, 64), (64, 264, 200)]:
        a = rnd(M, K, dtype=torch.bfloat16, seed=4, scale=0.5)
        w = rnd(2 * I, K, dtype=torch.bfloat16, seed=5, scale=0.2)
        gu = f64(a) @ f64(w).T
        gq = torch.from_numpy(gu).to(torch.bfloat16).double().numpy()   # the two-kernel path rounds the product first
        want = P.swiglu(gq[:, :I], gq[:, I:])
        got = ops.gemm_swiglu(a, w, torch.empty(M, I, dtype=torch.bfloat16, device=DEV))
        np.testing.assert_allclose(f64(got), want, rtol=2e-2, atol=2e-2)
        for rows in (70, 300, 1200):   # more rows: the tiled product with the activation as its epilogue
            big = rnd(rows, K, dtype=torch.bfloat16, seed=4, scale=0.5)
            gq = torch.from_numpy(f64(big) @ f64(w).T).to(torch.bfloat16).double().numpy()
            tiled = ops.gemm_swiglu(big, w, torch.empty(rows, I, dtype=torch.bfloat16, device=DEV))
            np.testing.assert_allclose(f64(tiled), P.swiglu(gq[:, :I], gq[:, I:]), rtol=2e-2, atol=2e-2)
    # rows that are not 16-byte aligned: product into a scratch buffer, then the activation kernel
    a, w = rnd(70, 100, dtype=torch.bfloat16, seed=8, scale=0.5), rnd(2 * 90, 100, dtype=torch.bfloat16, seed=9, scale=0.2)
    assert not ops.swiglu_fused_ok(a, w)
    with pytest.raises(ops.KernelError):
        ops.gemm_swiglu(a, w, torch.empty(70, 90, dtype=torch.bfloat16, device=DEV))
    gq = torch.from_numpy(f64(a) @ f64(w).T).to(torch.bfloat16).double().numpy()
    two = ops.gemm_swiglu(a, w, torch.empty(70, 90, dtype=torch.bfloat16, device=DEV), gate_up=torch.empty(70, 180, dtype=torch.bfloat16, device=DEV))
    np.testing.assert_allclose(f64(two), P.swiglu(gq[:, :90], gq[:, 90:]), rtol=2e-2, atol=2e-2)
    # a row's result does not depend on how many rows are beside it: bit for bit among the batches that one kernel
    # takes (up to 16 rows of a narrow output: four columns a block; more: sixteen), to rounding between the two
    a, w = rnd(64, 576, dtype=torch.bfloat16, seed=6), rnd(300, 576, dtype=torch.bfloat16, seed=7)
    full = ops.gemm(a, w, torch.empty(64, 300, device=DEV))
    few = ops.gemm(a[:16].contiguous(), w, torch.empty(16, 300, device=DEV))
    for m in (1, 4, 5, 8, 9, 16):
        assert torch.equal(ops.gemm(a[:m].contiguous(), w, torch.empty(m, 300, device=DEV)), few[:m])
    for m in (17, 48):
        assert torch.equal(ops.gemm(a[:m].contiguous(), w, torch.empty(m, 300, device=DEV)), full[:m])
    torch.testing.assert_close(few, full[:16], rtol=1e-5, atol=1e-4)
    # a wide output with more than 32 rows runs with eight waves a block instead of sixteen, which changes the
    # order of the sum over K: bit for bit among such batches, and to rounding against the smaller ones
    a, w = rnd(64, 200, dtype=torch.bfloat16, seed=8), rnd(6400, 200, dtype=torch.bfloat16, seed=9)
    small = ops.gemm(a[:32].contiguous(), w, torch.empty(32, 6400, device=DEV))
    large = ops.gemm(a, w, torch.empty(64, 6400, device=DEV))
    assert torch.equal(ops.gemm(a[:7].contiguous(), w, torch.empty(7, 6400, device=DEV)), small[:7])
    assert torch.equal(ops.gemm(a[:40].contiguous(), w, torch.empty(40, 6400, device=DEV)), large[:40])
    torch.testing.assert_close(small, large[:32], rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(f64(large), f64(a) @ f64(w).T, rtol=1e-4, atol=1e-4 * math.sqrt(200))


@pytest.mark.parametrize("M", [1, 3, 4, 5, 8, 9, 13, 16])
def test_gemm_narrow_outputs_of_few_rows(ops, M):
    """At most 16 rows against small weights with a narrow output run four output columns a block (four chunks of
    the inner size side by side in one matrix instruction): every epilogue and the fused norm, widths that are no
    multiple of 4, inner sizes that are no multiple of the 128-wide step or shorter than one."""
    for N, K in [(4, 8), (6, 40), (50, 128), (576, 576), (576, 1536), (1003, 136), (37, 4096), (100, 72)]:
        a, w, r = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2), rnd(M, N, seed=3)
        want = f64(a) @ f64(w).T
        tol_f = dict(rtol=1e-4, atol=1e-4 * math.sqrt(K))
        np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, device=DEV))), want, **tol_f)
        np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, dtype=torch.bfloat16, device=DEV))), want, rtol=1e-2, atol=1e-2 * math.sqrt(K))
        out = r.clone(); ops.gemm(a, w, out, residual=out)
        np.testing.assert_allclose(f64(out), want + f64(r), **tol_f)
        # rows of a larger buffer (a stride that is not the width)
        big = rnd(M, K + 24, dtype=torch.bfloat16, seed=4)
        np.testing.assert_allclose(f64(ops.gemm(big[:, :K], w, torch.empty(M, N, device=DEV))), f64(big[:, :K]) @ f64(w).T, **tol_f)
    for I, K, eps in [(6, 40, 1e-5), (172, 64, 1e-6), (1536, 576, 1e-5), (90, 200, 1e-2)]:
        x, nw = rnd(M + 2, K, seed=5, scale=2.0), 1 + 0.1 * rnd(K, seed=6)
        w = rnd(2 * I, K, dtype=torch.bfloat16, seed=7, scale=0.2)
        h = P.rmsnorm(f64(x), f64(nw), eps)
        gu = h @ f64(w).T
        want = P.swiglu(gu[:, :I], gu[:, I:])
        got = ops.gemm_swiglu(x[:M], w, torch.empty(M, I, dtype=torch.bfloat16, device=DEV), norm=(nw, eps, None))
        assert np.abs(f64(got) - want[:M]).max() < 2e-2 * max(np.abs(want).max(), 1e-3)
        hb = torch.from_numpy(h[:M]).to(torch.bfloat16).to(DEV)
        gq = torch.from_numpy(f64(hb) @ f64(w).T).to(torch.bfloat16).double().numpy()
        got = ops.gemm_swiglu(hb, w, torch.empty(M, I, dtype=torch.bfloat16, device=DEV))
        np.testing.assert_allclose(f64(got), P.swiglu(gq[:, :I], gq[:, I:]), rtol=2e-2, atol=2e-2)
        # the fused norm with gathered rows, float output
        rows = torch.tensor([(M + 1 - i) % (M + 2) for i in range(M)], dtype=torch.int32, device=DEV)
        wn_ = w[:I].contiguous()
        got = ops.gemm_normed(x, (nw, eps, rows), wn_, torch.empty(M, I, device=DEV))
        ref = h[rows.cpu().numpy()] @ f64(wn_).T
        assert np.abs(f64(got) - ref).max() < 6e-3 * np.abs(ref).max()


@pytest.mark.parametrize("M, heads, kv_heads, dim, splits", [(1, 9, 3, 64, 8), (3, 4, 2, 16, 2), (8, 9, 3, 64, 4), (5, 6, 6, 24, 4),
                                                             (16, 4, 1, 32, 2), (4, 9, 3, 64, 8), (13, 2, 2, 128, 4)])
def test_output_projection_merges_split_attention_itself(ops, M, heads, kv_heads, dim, splits):
    """Decode attention with its keys split over blocks may leave the partial results unmerged (bf16 normalised
    outputs, float statistics); the output projection then merges them while it prepares its operand.  Against the
    merge kernel followed by the plain product, and against a float64 merge of made-up partial results in which
    one split of a row has no keys and one row has none at all."""
    K, N = heads * dim, 4 * ((heads * dim // 2) // 4) + 2
    w = rnd(N, K, dtype=torch.bfloat16, seed=2, scale=0.1)
    assert ops.gemm_merged_ok(M, w, heads, dim, splits)
    # made-up partial results
    rng = np.random.default_rng(M + splits)
    po = torch.from_numpy(rng.standard_normal((M, heads, splits, dim)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    ms = rng.standard_normal((M, heads, splits)) * 3
    ls = rng.uniform(0.5, 40.0, (M, heads, splits))
    ms[0, :, splits - 1], ls[0, :, splits - 1] = -np.inf, 0.0        # a split that saw no key
    if M > 2:
        ms[2], ls[2] = -np.inf, 0.0                                  # a row without keys (padding): zeros
    pm = torch.from_numpy(np.stack([ms, ls], -1).astype(np.float32)).to(DEV).contiguous()
    weights = np.where(ls > 0, np.exp2(ms - np.max(ms, -1, keepdims=True, initial=-1e30)) * ls, 0.0)
    den = weights.sum(-1, keepdims=True)
    merged = np.where(den > 0, (weights[..., None] * f64(po)).sum(2) / np.where(den > 0, den, 1.0), 0.0).reshape(M, K)
    r = rnd(M, N, seed=5)
    out = r.clone()
    ops.gemm_merged((po, pm, splits), heads, dim, w, out, out)
    want = f64(r) + merged @ f64(w).T
    np.testing.assert_allclose(f64(out), want, rtol=2e-2, atol=2e-2 * np.abs(want).max())
    assert np.isfinite(f64(out)).all()
    # the real thing: split decode attention left unmerged, against the merge kernel and the plain product
    lengths = [333, 40, 130, 17, 700][:max(1, min(M, 5))]
    qt, kt, vt, tables, rows = paged_case(heads, kv_heads, dim, 16, lengths, torch.bfloat16, seed=dim + M)
    rows = (rows * 4)[:M]
    qt = qt[[i % qt.shape[0] for i in range(M)]].contiguous()
    T = len(rows)
    seg = torch.tensor([x[0] for x in rows], dtype=torch.int32, device=DEV)
    pos = torch.tensor([x[1] for x in rows], dtype=torch.int32, device=DEV)
    plain_out = torch.empty(T, K, dtype=torch.bfloat16, device=DEV)
    ws32 = (torch.empty(T * heads * splits * dim, device=DEV), torch.empty(T * heads * splits * 2, device=DEV))
    ops.attention_mfma(qt.reshape(T, K), K, kt, vt, tables, seg, pos, plain_out, heads, kv_heads, dim, 16, None, 1 / math.sqrt(dim),
                       None, splits, ws32, 8)
    two = r.clone(); ops.gemm(plain_out, w, two, residual=two)
    ws16 = (torch.empty(T * heads * splits * dim, dtype=torch.bfloat16, device=DEV), torch.empty(T * heads * splits * 2, device=DEV))
    untouched = torch.full((T, K), 3.0, dtype=torch.bfloat16, device=DEV)
    ops.attention_mfma(qt.reshape(T, K), K, kt, vt, tables, seg, pos, untouched, heads, kv_heads, dim, 16, None, 1 / math.sqrt(dim),
                       None, splits, ws16, 8, merge=False)
    assert (untouched == 3.0).all()
    one = r.clone(); ops.gemm_merged((ws16[0], ws16[1], splits), heads, dim, w, one, one)
    scale = np.abs(f64(two) - f64(r)).max()
    assert np.abs(f64(one) - f64(two)).max() < 2e-2 * scale       # the partial outputs are rounded to bf16 before they are merged
    # what it refuses: more rows, other split counts
    assert not ops.gemm_merged_ok(17, w, heads, dim, splits) and not ops.gemm_merged_ok(M, w, heads, dim, 3)


def test_fused_norm_products(ops):
    """RMSNorm inside the product's kernel (plain, row-gathered, SwiGLU) against norm then product."""
    for M, N, K, eps in [(1, 48, 64, 1e-5), (8, 1728, 576, 1e-5), (33, 130, 200, 1e-6), (64, 100, 144, 1e-2)]:
        x = rnd(M + 3, K, seed=1, scale=2.0)
        nw = 1 + 0.1 * rnd(K, seed=2)
        w = rnd(N, K, dtype=torch.bfloat16, seed=3, scale=0.1)
        h = P.rmsnorm(f64(x), f64(nw), eps)
        want = h @ f64(w).T
        scale = np.abs(want).max()
        got = ops.gemm_normed(x[:M], (nw, eps, None), w, torch.empty(M, N, device=DEV))
        assert np.abs(f64(got) - want[:M]).max() < 6e-3 * scale      # operands rounded to bf16 as in the two-kernel path
        rows = torch.tensor([M + 2, 0, M // 2], dtype=torch.int32, device=DEV)
        got = ops.gemm_normed(x, (nw, eps, rows), w, torch.empty(3, N, dtype=torch.bfloat16, device=DEV))
        assert np.abs(f64(got) - want[[M + 2, 0, M // 2]]).max() < 1.2e-2 * scale
        # against the engine's own two-kernel path: same roundings up to the place of the row factor
        hb = ops.rmsnorm(x[:M].contiguous(), nw, torch.empty(M, K, dtype=torch.bfloat16, device=DEV), eps)
        two = ops.gemm(hb, w, torch.empty(M, N, device=DEV))
        one = ops.gemm_normed(x[:M], (nw, eps, None), w, torch.empty(M, N, device=DEV))
        assert np.abs(f64(one) - f64(two)).max() < 6e-3 * scale
    M, I, K = 8, 172, 64
    x, nw = rnd(M, K, seed=4), 1 + 0.1 * rnd(K, seed=5)
    w = rnd(2 * I, K, dtype=torch.bfloat16, seed=6, scale=0.3)
    gu = P.rmsnorm(f64(x), f64(nw), 1e-5) @ f64(w).T
    want = P.swiglu(gu[:, :I], gu[:, I:])
    got = ops.gemm_swiglu(x, w, torch.empty(M, I, dtype=torch.bfloat16, device=DEV), norm=(nw, 1e-5, None))
    assert np.abs(f64(got) - want).max() < 2e-2 * np.abs(want).max()


@pytest.mark.parametrize("heads, kv_heads, dim, theta, normed", [(4, 2, 16, 1e4, True), (9, 3, 64, 1e5, True), (2, 1, 128, 5e5, False), (3, 3, 48, 1e4, True),
                                                                 (9, 3, 64, 1e5, False), (5, 1, 32, 1e4, True)])
def test_fused_projection_rotary_scatter(ops, heads, kv_heads, dim, theta, normed):
    from runtime.parts import RotaryEmbedding
    rope = RotaryEmbedding(dim, theta, 700); rope.prepare(DEV, torch.bfloat16)
    cos, sin = rope.tables()
    K, P_, pages = 72, 4, 16
    for M in (1, 5, 12, 40):     # one, two and four tiles of the narrow kernels, and the sixteen-column kernel
        pos = ([0, 17, 500, 699, 3] + [(53 * i) % 700 for i in range(5, M)])[:M]
        slots = ([5, 0, 22, -1, 9] + [63 - i for i in range(5, M)])[:M]
        x = rnd(M, K, seed=1, scale=1.5)
        nw = 1 + 0.1 * rnd(K, seed=2)
        w = rnd((heads + 2 * kv_heads) * dim, K, dtype=torch.bfloat16, seed=3, scale=0.2)
        h = P.rmsnorm(f64(x), f64(nw), 1e-5) if normed else f64(x.bfloat16())
        ref = h @ f64(w).T
        q_ref = P.rope(ref[:, :heads * dim].reshape(M, heads, dim), pos, theta)
        k_ref = P.rope(ref[:, heads * dim:(heads + kv_heads) * dim].reshape(M, kv_heads, dim), pos, theta)
        v_ref = ref[:, (heads + kv_heads) * dim:].reshape(M, kv_heads, dim)
        kc = torch.full((pages, kv_heads, P_, dim), 7.0, dtype=torch.bfloat16, device=DEV)
        vc = torch.full((pages, kv_heads, dim, P_), 7.0, dtype=torch.bfloat16, device=DEV)
        q = torch.empty(M, heads * dim, dtype=torch.bfloat16, device=DEV)
        a = x if normed else x.bfloat16()
        ops.qkv_rope(a, w, q, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                     cos, sin, kc, vc, heads, kv_heads, dim, P_, norm=(nw, 1e-5) if normed else None)
        tol = dict(rtol=2e-2, atol=2e-2 * np.abs(ref).max())
        np.testing.assert_allclose(f64(q).reshape(M, heads, dim), q_ref, **tol, err_msg=f"M={M}")
        kc64, vc64 = f64(kc), f64(vc)
        for t, s_ in enumerate(slots):
            if s_ < 0:
                continue
            np.testing.assert_allclose(kc64[s_ // P_, :, s_ % P_], k_ref[t], **tol, err_msg=f"M={M}")
            np.testing.assert_allclose(vc64[s_ // P_, :, :, s_ % P_], v_ref[t], **tol, err_msg=f"M={M}")
        untouched = [s_ for s_ in range(pages * P_) if s_ not in slots]
        assert all((kc64[s_ // P_, :, s_ % P_] == 7).all() and (vc64[s_ // P_, :, :, s_ % P_] == 7).all() for s_ in untouched)
        # q only (a layer that reads another layer's cache)
        wq = w[:heads * dim].contiguous()
        q2 = torch.empty_like(q)
        ops.qkv_rope(a, wq, q2, torch.tensor(pos, dtype=torch.int32, device=DEV), None, cos, sin, None, None, heads, kv_heads, dim, P_,
                     norm=(nw, 1e-5) if normed else None)
        assert torch.equal(q, q2), f"M={M}"


@pytest.mark.parametrize("heads, kv_heads, dim, M, K", [(4, 2, 16, 5, 72), (9, 3, 64, 8, 4104), (2, 1, 128, 20, 2056), (3, 3, 48, 40, 520),
                                                       (5, 1, 32, 64, 9000)])
def test_fused_projection_rotary_scatter_through_the_wide_product(ops, monkeypatch, heads, kv_heads, dim, M, K):
    """The same projection with large weights (forced here): normed bf16 rows in, the wide product with the rotary
    embedding and the cache write as its finishing step, in one slice of K and in several, one to four row tiles."""
    from runtime.parts import RotaryEmbedding
    for limit in ("WIDE_MIN_BYTES", "WIDE_MIN_BYTES_FEW_ROWS", "WIDE_MIN_BYTES_MANY_ROWS"):
        monkeypatch.setattr(ops, limit, 0)
    theta = 1e4
    rope = RotaryEmbedding(dim, theta, 700); rope.prepare(DEV, torch.bfloat16)
    cos, sin = rope.tables()
    P_, pages = 4, 2 * M
    rng = np.random.default_rng(M)
    pos = rng.integers(0, 700, size=M).tolist()
    slots = rng.permutation(pages * P_)[:M].tolist()
    slots[M // 2] = -1
    a = rnd(M, K, dtype=torch.bfloat16, seed=1, scale=1.5)
    w = rnd((heads + 2 * kv_heads) * dim, K, dtype=torch.bfloat16, seed=3, scale=0.2 / math.sqrt(K / 72))
    assert ops.wide_ok(M, w) and ops.qkv_rope_fused_ok(a, w, dim, cos, False)
    assert not ops.qkv_rope_fused_ok(a.float(), w, dim, cos, True)    # the norm is then a kernel of its own
    ref = f64(a) @ f64(w).T
    q_ref = P.rope(ref[:, :heads * dim].reshape(M, heads, dim), pos, theta)
    k_ref = P.rope(ref[:, heads * dim:(heads + kv_heads) * dim].reshape(M, kv_heads, dim), pos, theta)
    v_ref = ref[:, (heads + kv_heads) * dim:].reshape(M, kv_heads, dim)
    kc = torch.full((pages, kv_heads, P_, dim), 7.0, dtype=torch.bfloat16, device=DEV)
    vc = torch.full((pages, kv_heads, dim, P_), 7.0, dtype=torch.bfloat16, device=DEV)
    q = torch.empty(M, heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.qkv_rope(a, w, q, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                 cos, sin, kc, vc, heads, kv_heads, dim, P_)
    tol = dict(rtol=2e-2, atol=2e-2 * np.abs(ref).max())
    np.testing.assert_allclose(f64(q).reshape(M, heads, dim), q_ref, **tol)
    kc64, vc64 = f64(kc), f64(vc)
    for t, s_ in enumerate(slots):
        if s_ < 0:
            continue
        np.testing.assert_allclose(kc64[s_ // P_, :, s_ % P_], k_ref[t], **tol)
        np.testing.assert_allclose(vc64[s_ // P_, :, :, s_ % P_], v_ref[t], **tol)
    untouched = [s_ for s_ in range(pages * P_) if s_ not in slots]
    assert all((kc64[s_ // P_, :, s_ % P_] == 7).all() and (vc64[s_ // P_, :, :, s_ % P_] == 7).all() for s_ in untouched)
    # the same numbers as the product followed by the rotary kernel, but for the rounding of the product to bf16 between them
    qkv = ops.gemm(a, w, torch.empty(M, w.shape[0], dtype=torch.bfloat16, device=DEV))
    kc2, vc2 = torch.full_like(kc, 7.0), torch.full_like(vc, 7.0)
    ops.rope_scatter(qkv, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                     cos, sin, kc2, vc2, heads, kv_heads, dim, P_)
    np.testing.assert_allclose(f64(q), f64(qkv[:, :heads * dim]), **tol)
    np.testing.assert_allclose(f64(kc), f64(kc2), **tol)
    # q only (a layer that reads another layer's cache)
    q2 = torch.empty_like(q)
    ops.qkv_rope(a, w[:heads * dim].contiguous(), q2, torch.tensor(pos, dtype=torch.int32, device=DEV), None, cos, sin, None, None,
                 heads, kv_heads, dim, P_)
    assert torch.equal(q, q2)


GEMM_SHAPES = [(1, 1, 1), (5, 7, 9), (64, 64, 32), (130, 200, 172), (33, 513, 144), (17, 130, 1000), (300, 129, 72), (8, 1536, 576), (512, 576, 200), (1024, 1100, 64)]


def test_gemm_wide_for_large_weights(ops, monkeypatch):
    """Few rows against weights of many megabytes run the kernel that keeps the activations in registers and cuts
    K into slices: forced here for small shapes: every number of row tiles, widths off the 16-column unit,
    inner sizes of one step, of a partial pair, of several slices with an uneven cut, residual, bf16 output, SwiGLU."""
    monkeypatch.setattr(ops, "WIDE_MIN_BYTES", 0)
    monkeypatch.setattr(ops, "WIDE_MIN_BYTES_FEW_ROWS", 0)
    monkeypatch.setattr(ops, "WIDE_MIN_BYTES_MANY_ROWS", 0)
    shapes = [(1, 16, 8), (3, 100, 72), (8, 1728, 576), (16, 576, 1536), (17, 49, 264), (33, 130, 200), (48, 40, 2056),
              (64, 96, 4096), (50, 1003, 200), (8, 64, 14336), (64, 48, 9000), (20, 33, 4104)]
    for M, N, K in shapes:
        a, w, r = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2), rnd(M, N, seed=3)
        assert ops.wide_ok(M, w)
        want = f64(a) @ f64(w).T
        np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, device=DEV))), want, rtol=1e-4, atol=1e-4 * math.sqrt(K))
        np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, dtype=torch.bfloat16, device=DEV))), want, rtol=1e-2, atol=1e-2 * math.sqrt(K))
        out = r.clone(); ops.gemm(a, w, out, residual=out)
        np.testing.assert_allclose(f64(out), want + f64(r), rtol=1e-4, atol=1e-4 * math.sqrt(K))
    for M, I, K in [(1, 16, 32), (8, 1536, 576), (24, 100, 4096), (40, 172, 64), (64, 264, 2200)]:
        a = rnd(M, K, dtype=torch.bfloat16, seed=4, scale=0.5)
        w = rnd(2 * I, K, dtype=torch.bfloat16, seed=5, scale=0.2 if K < 1000 else 0.05)
        assert ops.wide_ok(M, w, True)
        gu = f64(a) @ f64(w).T
        gq = torch.from_numpy(gu).to(torch.bfloat16).double().numpy()
        got = ops.gemm_swiglu(a, w, torch.empty(M, I, dtype=torch.bfloat16, device=DEV))
        np.testing.assert_allclose(f64(got), P.swiglu(gq[:, :I], gq[:, I:]), rtol=2e-2, atol=2e-2)
    # a row's result does not depend on the rows beside it (same number of row tiles: the same launch)
    a, w = rnd(16, 4104, dtype=torch.bfloat16, seed=6), rnd(80, 4104, dtype=torch.bfloat16, seed=7)
    whole = ops.gemm(a, w, torch.empty(16, 80, device=DEV)).clone()
    for rows in (1, 5, 9):
        part = ops.gemm(a[:rows].contiguous(), w, torch.empty(rows, 80, device=DEV))
        assert torch.equal(part, whole[:rows])
    # with large weights the fused forms step aside for it
    assert not ops.fused_norm_ok(rnd(8, 576), rnd(1728, 576, dtype=torch.bfloat16), 8)
    monkeypatch.setattr(ops, "WIDE_MIN_BYTES_FEW_ROWS", 1 << 40)
    assert ops.fused_norm_ok(rnd(8, 576), rnd(1728, 576, dtype=torch.bfloat16), 8) and not ops.wide_ok(8, w)


@pytest.mark.parametrize("M", [1, 8, 24, 64])
def test_gemm_wide_at_the_sizes_that_choose_it(ops, M):
    """The wide product at sizes where it is the kernel of choice (Llama-3-8B's feed-forward and a 1.7B-size
    down projection), against float products of the same bf16 operands."""
    torch.manual_seed(M)
    H, I = 4096, 14336
    a = (torch.randn(M, H, device=DEV) * 0.5).bfloat16()
    w_gu = (torch.randn(2 * I, H, device=DEV) * 0.02).bfloat16()
    assert ops.wide_ok(M, w_gu, True)
    gu = a.float() @ w_gu.float().T
    gq = gu.bfloat16().float()
    want = torch.nn.functional.silu(gq[:, :I]) * gq[:, I:]
    got = ops.gemm_swiglu(a, w_gu, torch.empty(M, I, dtype=torch.bfloat16, device=DEV))
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-3)
    act = want.bfloat16()
    w_d = (torch.randn(H, I, device=DEV) * 0.02).bfloat16()
    r = torch.randn(M, H, device=DEV)
    assert ops.wide_ok(M, w_d)
    out = r.clone()
    ops.gemm(act, w_d, out, residual=out)
    torch.testing.assert_close(out, r + act.float() @ w_d.float().T, rtol=1e-4, atol=1e-4)
    # a narrow output with a long inner size (several slices of K, one unit or two a block)
    w_n = (torch.randn(2048, 8192, device=DEV) * 0.02).bfloat16()
    x = (torch.randn(M, 8192, device=DEV) * 0.5).bfloat16()
    assert ops.wide_ok(M, w_n)
    y = ops.gemm(x, w_n, torch.empty(M, 2048, device=DEV))
    torch.testing.assert_close(y, x.float() @ w_n.float().T, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("M", [4, 8, 40, 64, 100, 300])
def test_product_left_unfinished_is_added_by_the_norm_that_follows(ops, M, monkeypatch):
    """A product that the wide kernel cuts along its inner size may leave its slices' partial sums to the kernel that
    reads the rows next: sum + residual + norm in one kernel, or the sum alone; the rows are bit for bit what the
    product's own second kernel gives, the norm differs by the order of its sum of squares only.  Products that are
    not cut (or not wide) are not taken.  With more than 64 rows the product is the library's and what is left to
    the next kernel is its bf16 result (slices 0): the same rows and the same norm, bit for bit."""
    torch.manual_seed(M)
    N, K = 2048, 8192                       # the down projection of the 1.7B sizes
    w = (torch.randn(N, K, device=DEV) * 0.02).bfloat16()
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    r = torch.randn(M, N, device=DEV)
    nw = 1 + 0.1 * torch.randn(N, device=DEV)
    assert ops.wide_ok(M, w) if M <= 64 else ops.library_ok(M, w)
    want_x = r.clone()
    ops.gemm(a, w, want_x, residual=want_x)
    for out_dtype in (torch.bfloat16, torch.float32):
        want_y = ops.rmsnorm(want_x, nw, torch.empty(M, N, dtype=out_dtype, device=DEV), 1e-5)
        x = r.clone()
        partials = ops.gemm_unfinished(a, w, x)
        assert partials is not None and (partials[1] > 1 if M <= 64 else partials[1] == 0)
        assert torch.equal(x, r)            # nothing added yet
        y = ops.rmsnorm_partials(x, partials, nw, torch.empty(M, N, dtype=out_dtype, device=DEV), 1e-5)
        assert torch.equal(x, want_x)
        if M > 64:
            assert torch.equal(y, want_y)
        torch.testing.assert_close(y.float(), want_y.float(), rtol=1e-2 if out_dtype == torch.bfloat16 else 1e-5, atol=1e-5)
    x = r.clone()
    ops.add_partials(x, ops.gemm_unfinished(a, w, x))
    assert torch.equal(x, want_x)
    torch.testing.assert_close(x, r + a.float() @ w.float().T, rtol=1e-4 if M <= 64 else 2e-2, atol=1e-4 if M <= 64 else 2e-2)
    if M > 64:
        return
    # not taken: small weights (another kernel), a product of one slice, rows that are no contiguous floats
    small = (torch.randn(64, 128, device=DEV) * 0.02).bfloat16()
    assert ops.gemm_unfinished(a[:, :128].contiguous(), small, torch.zeros(M, 64, device=DEV)) is None
    for limit in ("WIDE_MIN_BYTES", "WIDE_MIN_BYTES_FEW_ROWS", "WIDE_MIN_BYTES_MANY_ROWS"):
        monkeypatch.setattr(ops, limit, 0)
    assert ops.wide_ok(M, small) and ops.gemm_unfinished(a[:, :128].contiguous(), small, torch.zeros(M, 64, device=DEV)) is None
    assert ops.gemm_unfinished(a, w, torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)) is None
    assert ops.gemm_unfinished(a, w, torch.zeros(M, 2 * N, device=DEV)[:, :N]) is None


def test_library_products_of_many_rows_also_in_captured_graphs(ops, monkeypatch):
    """Large bf16 products of many rows may go to the vendor's library, with the residual sum and the activation
    as kernels after it.  Checked against float products, eagerly and in a captured graph that is replayed with
    new inputs, eager work and synchronisations between the replays (a library call may record nodes that go
    wrong on later replays: every replay is checked)."""
    monkeypatch.setattr(ops, "LIBRARY_MIN_ROWS", 256)
    monkeypatch.setattr(ops, "LIBRARY_MIN_BYTES", 16 << 20)
    torch.manual_seed(0)
    M, N, K, I = 512, 4096, 4096, 5000
    w = (torch.randn(N, K, device=DEV) * 0.02).bfloat16()
    w_gu = (torch.randn(2 * I, K, device=DEV) * 0.02).bfloat16()
    assert ops.library_ok(M, w) and ops.library_ok(M, w_gu) and not ops.library_ok(255, w) and not ops.library_ok(M, w[:1000])
    assert not ops.library_ok(M, w.float())     # the 32-bit path never leaves the kernels of this repository
    a = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    res = torch.empty(M, N, device=DEV)
    act = torch.empty(M, I, dtype=torch.bfloat16, device=DEV)

    def step():
        ops.gemm(a, w, out)
        ops.gemm(a, w, res, residual=res)
        ops.gemm_swiglu(a, w_gu, act)

    def check(tag):
        ref = a.float() @ w.float().T
        torch.testing.assert_close(out.float(), ref, rtol=2e-2, atol=2e-2, msg=tag)
        torch.testing.assert_close(res - r0, ref, rtol=2e-2, atol=2e-2, msg=tag)   # the product is rounded to bf16 before the sum
        gq = (a.float() @ w_gu.float().T).bfloat16().float()
        torch.testing.assert_close(act.float(), torch.nn.functional.silu(gq[:, :I]) * gq[:, I:], rtol=2e-2, atol=2e-3, msg=tag)

    r0 = torch.randn(M, N, device=DEV)
    a.copy_(torch.randn(M, K, device=DEV) * 0.5); res.copy_(r0)
    step(); check("eager")
    res.copy_(r0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(5):
        a.copy_(torch.randn(M, K, device=DEV) * 0.5); res.copy_(r0)
        out.fill_(7); act.fill_(7)
        junk = (torch.randn(300, 300, device=DEV) @ torch.randn(300, 300, device=DEV)).sum().item()   # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        check(f"replay {i}")


@pytest.mark.parametrize("M, N, K", GEMM_SHAPES)
def test_gemm_f32(ops, M, N, K):
    a, w, r = rnd(M, K, seed=1), rnd(N, K, seed=2), rnd(M, N, seed=3)
    want = f64(a) @ f64(w).T
    # unit-variance operands summed in ascending k: partial sums grow like sqrt(k), each
    # addition rounds at 6e-8 of it, so the error of a length-K sum is a few 1e-7 * K
    atol = 3e-7 * K + 2e-6
    np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, device=DEV))), want, rtol=2e-5, atol=atol)
    out = r.clone()
    ops.gemm(a, w, out, residual=out)   # in place on the residual
    np.testing.assert_allclose(f64(out), want + f64(r), rtol=2e-5, atol=atol)


@pytest.mark.parametrize("M, N, K", GEMM_SHAPES)
def test_gemm_bf16(ops, M, N, K):
    a, w, r = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2), rnd(M, N, seed=3)
    want = f64(a) @ f64(w).T   # products of bf16 values are exact in float: only the sum order differs
    np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(M, N, device=DEV))), want, rtol=1e-4, atol=1e-4 * math.sqrt(K))
    got = ops.gemm(a, w, torch.empty(M, N, dtype=torch.bfloat16, device=DEV))
    np.testing.assert_allclose(f64(got), want, rtol=1e-2, atol=1e-2 * math.sqrt(K))
    out = r.clone()
    ops.gemm(a, w, out, residual=out)
    np.testing.assert_allclose(f64(out), want + f64(r), rtol=1e-4, atol=1e-4 * math.sqrt(K))


@pytest.mark.parametrize("tile", [112, 122, 222, 422, 442])
def test_gemm_bf16_every_block_tile_alone(ops, tile):
    """The rule picks a block tile by the shape; here each built tile (rows / 16 a wave x 100, columns / 16 a wave x 10,
    waves along the rows) multiplies shapes that no tile divides, with and without the residual, and the activation
    where the tile pairs column tiles."""
    stream = torch.cuda.current_stream().cuda_stream
    for M, N, K in ((150, 200, 136), (70, 1000, 72), (333, 96, 520)):
        a, w, r = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2), rnd(M, N, seed=3)
        want = f64(a) @ f64(w).T
        out = r.clone()
        assert ops.lib().cisr_gemm_bf16_tile(a.data_ptr(), K, w.data_ptr(), K, out.data_ptr(), N, out.data_ptr(), N, M, N, K,
                                             0, tile, stream) == 0
        np.testing.assert_allclose(f64(out), want + f64(r), rtol=1e-4, atol=1e-4 * math.sqrt(K))
        half = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        assert ops.lib().cisr_gemm_bf16_tile(a.data_ptr(), K, w.data_ptr(), K, half.data_ptr(), N, None, 0, M, N, K, 1, tile, stream) == 0
        np.testing.assert_allclose(f64(half), want, rtol=1e-2, atol=1e-2 * math.sqrt(K))
        if tile in (122, 222, 422, 442) and N % 2 == 0:
            H = N // 2
            act = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
            assert ops.lib().cisr_gemm_bf16_swiglu_tile(a.data_ptr(), K, w.data_ptr(), K, act.data_ptr(), H, M, H, K, H, tile, stream) == 0
            g, u = f64(torch.from_numpy(want[:, :H]).bfloat16()), f64(torch.from_numpy(want[:, H:]).bfloat16())
            np.testing.assert_allclose(f64(act), g / (1 + np.exp(-g)) * u, rtol=2e-2, atol=2e-2)
    a, w = rnd(40, 64, dtype=torch.bfloat16), rnd(48, 64, dtype=torch.bfloat16)
    out = torch.empty(40, 48, device=DEV)
    assert ops.lib().cisr_gemm_bf16_tile(a.data_ptr(), 64, w.data_ptr(), 64, out.data_ptr(), 48, None, 0, 40, 48, 64, 0, 999, stream) != 0


def test_gemm_strided_rows_and_bad_operands(ops):
    from runtime.kernels.ops import KernelError
    big = rnd(9, 50, dtype=torch.bfloat16)
    a = big[:, 10:31]   # 21 columns of a wider buffer: rows are strided and unaligned
    w = rnd(13, 21, dtype=torch.bfloat16, seed=2)
    np.testing.assert_allclose(f64(ops.gemm(a, w, torch.empty(9, 13, device=DEV))), f64(a) @ f64(w).T, rtol=1e-4, atol=1e-3)
    with pytest.raises(KernelError):
        ops.gemm(rnd(4, 8), rnd(5, 9), torch.empty(4, 5, device=DEV))
    with pytest.raises(KernelError):
        ops.gemm(rnd(4, 8), rnd(5, 8, dtype=torch.bfloat16), torch.empty(4, 5, device=DEV))
    with pytest.raises(KernelError):
        ops.gemm(rnd(4, 8), rnd(5, 8), torch.empty(4, 5, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError):
        ops.gemm(torch.zeros(4, 8), torch.zeros(5, 8), torch.empty(4, 5))  # CPU tensors: no fallback


def test_argmax_lowest_index_wins(ops):
    logits = rnd(6, 1003, seed=8)
    logits[1, 500] = logits[1, 17] = 50.0
    logits[2, :] = 1.0
    logits[3, 1002] = 99.0
    out = ops.argmax(logits, torch.empty(6, dtype=torch.int32, device=DEV)).cpu().numpy()
    want = f64(logits).argmax(-1)
    np.testing.assert_array_equal(out, want)
    assert out[1] == 17 and out[2] == 0 and out[3] == 1002


def test_token_choices_scattered_by_index_and_taken_back(ops):
    """A token choice that leaves row r's token at out[index[r]] (nowhere for an index outside out), and the
    rows of a step that take their token from there."""
    z = rnd(7, 517, seed=12)
    greedy = f64(z).argmax(-1)
    index = torch.tensor([4, 0, -1, 9, 2, 40, 7], dtype=torch.int32, device=DEV)
    for how in ("argmax", "sample"):
        out = torch.full((10,), -5, dtype=torch.int32, device=DEV)
        if how == "argmax":
            ops.argmax(z, out, index)
        else:
            ops.sample(z, torch.zeros(7, device=DEV), torch.zeros(7, dtype=torch.int64, device=DEV),
                       torch.zeros(7, dtype=torch.int64, device=DEV), out, index)
        want = np.full(10, -5)
        for r, i in enumerate(index.tolist()):
            if 0 <= i < 10:
                want[i] = greedy[r]
        np.testing.assert_array_equal(out.cpu().numpy(), want)
    # sampled rows land at their index too, with the same draw as without an index
    temp, seeds = torch.full((7,), 0.9, device=DEV), torch.arange(7, dtype=torch.int64, device=DEV)
    counters = torch.full((7,), 3, dtype=torch.int64, device=DEV)
    direct = ops.sample(z, temp, seeds, counters, torch.empty(7, dtype=torch.int32, device=DEV)).cpu().numpy()
    out = torch.full((10,), -5, dtype=torch.int32, device=DEV)
    ops.sample(z, temp, seeds, counters, out, index)
    for r, i in enumerate(index.tolist()):
        if 0 <= i < 10:
            assert out[i].item() == direct[r]
    tokens = torch.arange(100, 106, dtype=torch.int32, device=DEV)
    source = torch.tensor([-1, 9, 4, -1, 0, 77], dtype=torch.int32, device=DEV)
    ops.take_tokens(tokens, source, out)
    picked = out.cpu().numpy()
    np.testing.assert_array_equal(tokens.cpu().numpy(), [100, picked[9], picked[4], 103, picked[0], 105])
    with pytest.raises(Exception):
        ops.argmax(z, out, index[:3].contiguous())


def test_sampling_kernel(ops):
    from runtime.sampling import uniform01
    V = 11
    logits = torch.tensor(np.log(np.arange(1, V + 1, dtype=np.float64)), dtype=torch.float32, device=DEV)[None].repeat(4000, 1).contiguous()
    temp = torch.full((4000,), 1.0, device=DEV)
    seeds = torch.full((4000,), 1234, dtype=torch.int64, device=DEV)
    counters = torch.arange(4000, dtype=torch.int64, device=DEV)
    out = ops.sample(logits, temp, seeds, counters, torch.empty(4000, dtype=torch.int32, device=DEV)).cpu().numpy()
    freq = np.bincount(out, minlength=V) / 4000
    p = np.arange(1, V + 1) / np.arange(1, V + 1).sum()
    assert np.abs(freq - p).max() < 0.03
    # the draw is the inverse CDF at the documented random number
    cdf = np.cumsum(p)
    want = [int(np.searchsorted(cdf, uniform01(1234, c), side="right")) for c in range(50)]
    assert (out[:50] == np.minimum(want, V - 1)).mean() > 0.95   # equal but for rounding at a CDF edge
    # temperature 0 is greedy; a tiny temperature too; rows do not influence each other
    z = rnd(5, 777, seed=3)
    greedy = ops.argmax(z, torch.empty(5, dtype=torch.int32, device=DEV)).cpu().numpy()
    for t in (0.0, 1e-4):
        got = ops.sample(z, torch.full((5,), t, device=DEV), torch.zeros(5, dtype=torch.int64, device=DEV),
                         torch.zeros(5, dtype=torch.int64, device=DEV), torch.empty(5, dtype=torch.int32, device=DEV))
        np.testing.assert_array_equal(got.cpu().numpy(), greedy)
    one = ops.sample(z[2:3].contiguous(), torch.full((1,), 0.8, device=DEV), torch.full((1,), 5, dtype=torch.int64, device=DEV),
                     torch.full((1,), 9, dtype=torch.int64, device=DEV), torch.empty(1, dtype=torch.int32, device=DEV))
    five = ops.sample(z, torch.full((5,), 0.8, device=DEV), torch.full((5,), 5, dtype=torch.int64, device=DEV),
                      torch.full((5,), 9, dtype=torch.int64, device=DEV), torch.empty(5, dtype=torch.int32, device=DEV))
    assert one[0] == five[2]


def test_page_copy(ops):
    pool = rnd(3, 2, 5, 2, 4, 8, dtype=torch.bfloat16)   # [sites, k/v, pages, kv_heads, page, dim]
    before = pool.clone()
    ops.page_copy(pool, torch.tensor([1, 4], dtype=torch.int32, device=DEV), torch.tensor([3, 0], dtype=torch.int32, device=DEV), 6, 5)
    assert torch.equal(pool[:, :, 3], before[:, :, 1]) and torch.equal(pool[:, :, 0], before[:, :, 4])
    assert torch.equal(pool[:, :, [1, 2, 4]], before[:, :, [1, 2, 4]])


def test_kernels_refuse_what_they_cannot_take(ops):
    from runtime.kernels.ops import KernelError
    with pytest.raises(KernelError, match="head size"):
        run_rowwise(ops, rnd(1, 2, 258), rnd(1, 2, 4, 258), rnd(1, 2, 258, 4), torch.zeros(1, 1, dtype=torch.int32, device=DEV), [(0, 0)], 4)
    with pytest.raises(KernelError, match="divide"):
        run_rowwise(ops, rnd(1, 3, 16), rnd(1, 2, 4, 16), rnd(1, 2, 16, 4), torch.zeros(1, 1, dtype=torch.int32, device=DEV), [(0, 0)], 4)
    with pytest.raises(KernelError, match="not supported"):   # the matrix-core kernel takes bf16, head sizes in steps of 8, pages of 8, 16, ... keys
        ops.attention_mfma(rnd(1, 2 * 12, dtype=torch.bfloat16), 24, rnd(1, 2, 4, 12, dtype=torch.bfloat16), rnd(1, 2, 12, 4, dtype=torch.bfloat16),
                           torch.zeros(1, 1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                           torch.zeros(1, dtype=torch.int32, device=DEV), torch.empty(1, 24, dtype=torch.bfloat16, device=DEV), 2, 2, 12, 4, None, 1.0)
    assert not ops.mfma_attention_supported(torch.bfloat16, 64, 3) and not ops.mfma_attention_supported(torch.float32, 64, 16)
    assert not ops.mfma_attention_supported(torch.bfloat16, 64, 4) and ops.mfma_attention_supported(torch.bfloat16, 64, 8)   # (a lane takes 8 keys of a value page at once)
    with pytest.raises(KernelError):
        ops.rmsnorm(rnd(2, 8), rnd(9), torch.empty(2, 8, device=DEV), 1e-5)
    with pytest.raises(KernelError):
        ops.embedding(torch.zeros(2, dtype=torch.int64, device=DEV), rnd(4, 8), torch.empty(2, 8, device=DEV))


@pytest.mark.gpu
@pytest.mark.parametrize("blocks,exchange", [(32, 0), (256, 0), (96, 500)])
def test_grid_meet_counts_every_group_every_round(ops, blocks, exchange):
    from runtime import measure
    from runtime.kernels.ops import KernelError
    rounds = 50
    words = measure.grid_meet(blocks, rounds, exchange)
    torch.cuda.synchronize()
    assert int(words[-1]) == 0                              # no block gave up waiting
    assert int(words[0]) == rounds * (blocks // 32)         # every group arrived in every round
    groups = blocks // 32
    for g in range(groups):
        assert int(words[16 * (1 + g)]) == rounds * 32
    with pytest.raises(KernelError, match="multiple of 32"):
        measure.grid_meet(48, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias_dtype", [torch.float32, torch.bfloat16])
def test_bias_add(ops, x_dtype, bias_dtype):
    for rows, cols in ((1, 7), (37, 576), (300, 1000)):
        g = torch.Generator(device="cpu").manual_seed(rows + cols)
        x = torch.randn(rows, cols, generator=g).to(x_dtype).to(DEV)
        bias = torch.randn(cols, generator=g).to(bias_dtype).to(DEV)
        want = (x.double() + bias.double()[None, :]).to(x_dtype)          # one rounding, to x's type
        got = ops.bias_add(x.clone(), bias)
        assert torch.equal(got, want), (rows, cols)
    from runtime.kernels.ops import KernelError
    with pytest.raises(KernelError, match="shape"):
        ops.bias_add(torch.zeros(3, 5, device=DEV), torch.zeros(4, device=DEV))
