"""Checked Python entry points of the HIP kernels.

Every function validates device, dtype, contiguity and shapes on the host
before the launch, because a kernel that reads out of bounds can take the GPU
down.  Tensors are torch tensors on the GPU; launches go to torch's current
stream, so they are ordered with torch's own work and can be captured into a
graph.  Nothing here computes on the CPU.  One kind of call leaves the kernels of this repository: large bf16
products of more than 64 rows, which go to the vendor's library through torch.mm (see library_ok).
"""
import ctypes as C

import torch

from . import library

F32, BF16 = 0, 1
MFMA_HEAD_PADS = library.ATTENTION_PADS
SKINNY_ROWS = 64   # products with at most this many rows run the weight-streaming kernel
_DT = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_configured = False


def lib():
    global _configured
    handle = library.load()
    if not _configured:
        _declare(handle)
        _configured = True
    return handle


def _declare(h):
    p, i, f, ll = C.c_void_p, C.c_int, C.c_float, C.c_longlong
    sig = {
        "cisr_embedding": [p, p, p, i, i, i, i, p],
        "cisr_rmsnorm": [p, p, p, p, i, i, f, i, p],
        "cisr_add_rmsnorm": [p, p, p, p, i, i, f, i, p],
        "cisr_residual_add": [p, p, ll, i, p],
        "cisr_swiglu": [p, p, i, i, i, p],
        "cisr_rope_scatter": [p, p, p, p, p, p, p, i, i, i, i, i, i, i, i, i, i, p],
        "cisr_page_copy": [p, p, p, i, i, ll, ll, p],
        "cisr_f32_to_bf16": [p, p, ll, p],
        "cisr_bias_add": [p, p, ll, i, i, i, p],
        "cisr_attn_rowwise": [p, i, p, p, p, p, p, p, p, p, i, i, i, i, i, i, i, f, i, i, p],
        "cisr_gemm_f32": [p, i, p, i, p, i, p, i, i, i, i, p],
        "cisr_gemm_bf16": [p, i, p, i, p, i, p, i, i, i, i, i, p],
        "cisr_gemm_bf16_swiglu": [p, i, p, i, p, i, i, i, i, i, p],
        "cisr_gemm_bf16_tile": [p, i, p, i, p, i, p, i, i, i, i, i, i, p],
        "cisr_gemm_bf16_swiglu_tile": [p, i, p, i, p, i, i, i, i, i, i, p],
        "cisr_gemm_skinny_bf16": [p, i, p, i, p, i, p, i, i, i, i, i, i, p, f, p, p],
        "cisr_qkv_rope_skinny": [p, i, p, i, p, i, i, i, p, f, p, p, p, p, p, p, i, i, i, i, i, p],
        "cisr_attn_merge": [p, p, p, i, i, i, i, p, p],
        "cisr_argmax": [p, p, p, i, p, p, i, i, p],
        "cisr_sample": [p, p, p, p, p, p, i, i, i, p],
        "cisr_take_tokens": [p, p, p, i, i, p],
        "cisr_gemm_wide_bf16": [p, i, p, i, p, i, p, i, i, i, i, i, i, p, C.c_longlong, p],
        "cisr_gemm_wide_partials_bf16": [p, i, p, i, i, i, i, p, C.c_longlong, p],
        "cisr_rmsnorm_partials": [p, p, i, p, p, i, i, f, i, p],
        "cisr_add_rmsnorm_bf16": [p, p, p, p, i, i, f, i, p],
        "cisr_qkv_rope_wide": [p, i, p, i, p, i, i, i, p, p, p, p, p, p, i, i, i, i, i, p, C.c_longlong, p],
        "cisr_gemm_merged_bf16": [p, p, i, i, i, p, i, p, i, p, i, i, i, p],
        "cisr_gemm_merged_ok": [i, i, i, i, i],
    }
    for name, args in sig.items():
        fn = getattr(h, name)
        fn.argtypes = args
        fn.restype = C.c_int
    h.cisr_gemm_wide_workspace.argtypes = [i, i, i, i]
    h.cisr_gemm_wide_workspace.restype = C.c_longlong
    h.cisr_gemv_ok.argtypes = [i, i, i]
    h.cisr_gemv_ok.restype = C.c_int
    h.cisr_gemv_set.argtypes = [i, ll]
    h.cisr_gemv_set.restype = None


_attention_entries = {}


def _attention_entry(dpad):
    """The matrix-core attention entry point for a padded head size (its shared object is built and loaded
    at the first use of that size)."""
    fn = _attention_entries.get(dpad)
    if fn is None:
        p, i, f = C.c_void_p, C.c_int, C.c_float
        fn = getattr(library.load_attention(dpad), f"cisr_attn_mfma_d{dpad}")
        fn.argtypes = [p, i, p, p, p, i, p, i, p, p, p, p, p, i, i, i, i, i, f, i, i, i, i, p]
        fn.restype = C.c_int
        _attention_entries[dpad] = fn
    return fn


def prepare(units=()):
    """Build, side by side, the core and the further shared objects `units` (names of library.units(): what the
    parts of a model say they need, `kernel_units`), and load the core."""
    library.ensure([library.CORE] + [u for u in dict.fromkeys(units) if u != library.CORE])
    lib()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The handle of the current stream of the current device.  Every launch asks for it: torch's short way where it has
    one (a prompt step run kernel by kernel asks 240 times; `torch.cuda.current_stream()` takes 9 us a call, 2 ms a step)."""
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(code, what):
    if code != 0:
        raise KernelError(f"{what}: HIP error {code}")


def _dev(t, name, dtype=None, shape=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: expected a GPU tensor")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor must be contiguous")
    if dtype is not None:
        allowed = dtype if isinstance(dtype, (tuple, list)) else (dtype,)
        if t.dtype not in allowed:
            raise KernelError(f"{name}: dtype {t.dtype}, expected {allowed}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
    return t.data_ptr()


def _storage(t, name):
    if t.dtype not in _DT:
        raise KernelError(f"{name}: storage dtype {t.dtype} is not float32 or bfloat16")
    return _DT[t.dtype]


def embedding(tokens, table, out):
    """out[r] = table[tokens[r]] widened to float.  tokens int32 [T], table [V, H], out float [T, H]."""
    rows = tokens.shape[0]
    vocab, dim = table.shape
    _check(lib().cisr_embedding(_dev(tokens, "tokens", torch.int32, (rows,)), _dev(table, "table"),
                                _dev(out, "out", torch.float32, (rows, dim)), rows, dim, vocab,
                                _storage(table, "table"), _stream()), "embedding")
    return out


def rmsnorm(x, weight, out, eps, rows=None):
    """out = rmsnorm(x[rows]) * weight.  x float [T, H]; weight float [H]; out [R, H] float or bf16."""
    dim = x.shape[1]
    n_out = out.shape[0]
    if rows is None and n_out != x.shape[0]:
        raise KernelError("rmsnorm: out rows differ from input rows")
    rp = None if rows is None else _dev(rows, "rows", torch.int32, (n_out,))
    _check(lib().cisr_rmsnorm(_dev(x, "x", torch.float32), _dev(weight, "weight", torch.float32, (dim,)),
                              _dev(out, "out", None, (n_out, dim)), rp, n_out, dim, float(eps),
                              _storage(out, "out"), _stream()), "rmsnorm")
    return out


def partials_ok(x):
    """Whether add_partials / rmsnorm_partials take the float rows x."""
    return (x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] % 4 == 0 and x.shape[1] <= 8192
            and x.data_ptr() % 16 == 0)


def add_partials(x, partials):
    """x += what gemm_unfinished left (float rows, in place): the partial sums in slice order, or (slices 0) the
    bf16 product."""
    parts, slices = partials
    rows, dim = x.shape
    if slices == 0:
        return residual_add(x, parts)
    if not partials_ok(x) or parts.numel() < slices * rows * dim:
        raise KernelError("add_partials: contiguous float rows of a multiple of 4 (at most 8192) and their partial sums")
    _check(lib().cisr_rmsnorm_partials(x.data_ptr(), _dev(parts, "partials", torch.float32), int(slices), None, None, rows, dim,
                                       0.0, _DT[torch.float32], _stream()), "add_partials")
    return x


def rmsnorm_partials(x, partials, weight, out, eps):
    """x += what gemm_unfinished left (in place), out = rmsnorm(x) * weight: one kernel."""
    parts, slices = partials
    rows, dim = x.shape
    if not partials_ok(x) or out.data_ptr() % 16:
        raise KernelError("rmsnorm_partials: contiguous float rows of a multiple of 4 (at most 8192)")
    wp, op = _dev(weight, "weight", torch.float32, (dim,)), _dev(out, "out", None, (rows, dim))
    if slices == 0:
        _check(lib().cisr_add_rmsnorm_bf16(x.data_ptr(), _dev(parts, "product", torch.bfloat16, (rows, dim)), wp, op, rows, dim,
                                           float(eps), _storage(out, "out"), _stream()), "rmsnorm_partials")
        return out
    if parts.numel() < slices * rows * dim:
        raise KernelError("rmsnorm_partials: too few partial sums")
    _check(lib().cisr_rmsnorm_partials(x.data_ptr(), _dev(parts, "partials", torch.float32), int(slices), wp, op,
                                       rows, dim, float(eps), _storage(out, "out"), _stream()), "rmsnorm_partials")
    return out


def add_rmsnorm(x, delta, weight, out, eps):
    """x += delta (float residual, in place), out = rmsnorm(x) * weight."""
    rows, dim = x.shape
    dt = _storage(delta, "delta")
    if out.dtype != delta.dtype:
        raise KernelError("add_rmsnorm: out and delta must share a dtype")
    _check(lib().cisr_add_rmsnorm(_dev(x, "x", torch.float32), _dev(delta, "delta", None, (rows, dim)),
                                  _dev(weight, "weight", torch.float32, (dim,)), _dev(out, "out", None, (rows, dim)),
                                  rows, dim, float(eps), dt, _stream()), "add_rmsnorm")
    return out


def residual_add(x, delta):
    """x += delta, x float, delta float or bf16 of the same shape."""
    if x.shape != delta.shape:
        raise KernelError("residual_add: shapes differ")
    _check(lib().cisr_residual_add(_dev(x, "x", torch.float32), _dev(delta, "delta"), x.numel(),
                                   _storage(delta, "delta"), _stream()), "residual_add")
    return x


def swiglu(gate_up, out):
    """out[r, i] = silu(gate_up[r, i]) * gate_up[r, I + i]."""
    rows, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("swiglu: input width must be even")
    inter = two_i // 2
    _check(lib().cisr_swiglu(_dev(gate_up, "gate_up"), _dev(out, "out", gate_up.dtype, (rows, inter)), rows, inter,
                             _storage(gate_up, "gate_up"), _stream()), "swiglu")
    return out


def bias_add(x, bias):
    """x[r, c] += bias[c], in place (added in float).  x [T, N] float or bf16, contiguous; bias [N] float or bf16."""
    rows, cols = x.shape
    _check(lib().cisr_bias_add(_dev(x, "x"), _dev(bias, "bias", None, (cols,)), rows, cols, _storage(x, "x"), _storage(bias, "bias"),
                               _stream()), "bias_add")
    return x


def rope_scatter(qkv, positions, slots, cos, sin, kcache, vcache, heads, kv_heads, dim, page_size, interleaved=False):
    """Rotate q (in place) and k of the fused projection rows, write k and v into
    the cache at `slots`.  kcache/vcache None: q only (a layer reading another's cache).
    Pair i of a head is coordinates (i, i + rot/2), or with `interleaved` (2i, 2i + 1).
    qkv [T, (heads + 2 kv_heads) * dim] (or [T, heads * dim] without a cache);
    cos/sin float [max_pos, rot/2]; keys [pages, kv_heads, page_size, dim],
    values transposed in a page: [pages, kv_heads, dim, page_size]."""
    rows = qkv.shape[0]
    has_kv = kcache is not None
    width = (heads + (2 * kv_heads if has_kv else 0)) * dim
    dt = _storage(qkv, "qkv")
    max_pos, half = cos.shape
    rot = 2 * half
    if rot > dim or rot <= 0:
        raise KernelError(f"rope_scatter: rotary size {rot} does not fit head size {dim}")
    kp = vp = sp = None
    if has_kv:
        pages = kcache.shape[0]
        kp = _dev(kcache, "kcache", qkv.dtype, (pages, kv_heads, page_size, dim))
        vp = _dev(vcache, "vcache", qkv.dtype, (pages, kv_heads, dim, page_size))
        sp = _dev(slots, "slots", torch.int32, (rows,))
    _check(lib().cisr_rope_scatter(_dev(qkv, "qkv", None, (rows, width)), _dev(positions, "positions", torch.int32, (rows,)),
                                   sp, _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, half)),
                                   kp, vp, rows, heads, kv_heads, dim, rot, page_size, max_pos, int(has_kv),
                                   int(bool(interleaved)), dt, _stream()), "rope_scatter")


def page_copy(pool, src, dst, slabs, pages_per_slab):
    """pool viewed as [slabs, pages_per_slab, page]: page dst[i] := page src[i] in every slab."""
    n = src.shape[0]
    total = pool.numel() * pool.element_size()
    if total % (slabs * pages_per_slab):
        raise KernelError("page_copy: pool does not divide into slabs and pages")
    slab_bytes = total // slabs
    page_bytes = slab_bytes // pages_per_slab
    _check(lib().cisr_page_copy(_dev(pool, "pool"), _dev(src, "src", torch.int32, (n,)), _dev(dst, "dst", torch.int32, (n,)),
                                n, slabs, page_bytes, slab_bytes, _stream()), "page_copy")


def f32_to_bf16(x, out):
    _check(lib().cisr_f32_to_bf16(_dev(x, "x", torch.float32), _dev(out, "out", torch.bfloat16, x.shape), x.numel(),
                                  _stream()), "f32_to_bf16")
    return out


def attention_rowwise(q, q_row_stride, kcache, vcache, tables, seg_of_row, positions, out, heads, kv_heads, dim,
                      page_size, window, scale, splits=1, workspace=None):
    """Each row attends to its request's cached keys lo..position.  q is a view
    into a row-major buffer with `q_row_stride` elements per row; out [T, heads*dim]."""
    rows = out.shape[0]
    dt = _storage(out, "out")
    if dim % 2 or dim > 256:
        raise KernelError(f"attention: head size {dim} must be even and at most 256")
    if heads % kv_heads:
        raise KernelError(f"attention: {heads} query heads do not divide into {kv_heads} key heads")
    pages = kcache.shape[0]
    width = tables.shape[1]
    if q.dtype != out.dtype or kcache.dtype != out.dtype:
        raise KernelError("attention: q, cache and out must share a dtype")
    if q.numel() < (rows - 1) * q_row_stride + heads * dim:
        raise KernelError("attention: q buffer too small for its stride")
    po = pm = None
    if splits > 1:
        if workspace is None:
            raise KernelError("attention: split runs need a workspace")
        part_o, part_ml = workspace
        po = _dev(part_o, "part_o", torch.float32)
        pm = _dev(part_ml, "part_ml", torch.float32)
        if part_o.numel() < rows * heads * splits * dim or part_ml.numel() < rows * heads * splits * 2:
            raise KernelError("attention: split workspace too small")
    _check(lib().cisr_attn_rowwise(q.data_ptr(), q_row_stride, _dev(kcache, "kcache", None, (pages, kv_heads, page_size, dim)),
                                   _dev(vcache, "vcache", None, (pages, kv_heads, dim, page_size)),
                                   _dev(tables, "tables", torch.int32), _dev(seg_of_row, "seg_of_row", torch.int32, (rows,)),
                                   _dev(positions, "positions", torch.int32, (rows,)), _dev(out, "out", None, (rows, heads * dim)),
                                   po, pm, rows, heads, kv_heads, dim, page_size, width, int(window or 0), float(scale),
                                   int(splits), dt, _stream()), "attention_rowwise")
    return out


# Large bf16 products of many rows go to the vendor's library through torch.mm (the reference's linears are
# library calls too: cuBLAS through runtime/blas.py:44-56, or CuPy's matmul, runtime/model.py:108): from this many rows on, with weights of at least LIBRARY_MIN_BYTES;
# the residual sum or the activation is then a kernel after the product.  Measured on an MI355X at 2048 rows:
# 1,270-1,480 TFLOP/s against 830-920 of the tiled kernel here on the 8B shapes (a prompt step of 30.6 against
# 39.9 ms); at 65-255 rows with weights streamed from HBM it is up to 2.5 times as fast on narrow outputs with
# a long inner size, which leave the tiled kernel few tiles (it does not cut K).  With at most 64 rows the
# weight-streaming kernels here are as fast or faster (8 rows: 50 against 67 us for gate and up of the 8B
# sizes), as are all products of small weights, and both save the kernel after the product.  The least weights are
# those of the 1.7B sizes' output projection (8 MB: 10.7 against 13.9 us at 128 rows, 29 against 33 at 2,048, the
# residual sum included; the products of the 135M sizes, 0.7 to 3.5 MB, are as fast or faster here).  0 rows: never.
LIBRARY_MIN_ROWS = 65
LIBRARY_MIN_BYTES = 8 << 20
LIBRARY_GATED_MIN_ROWS, LIBRARY_GATED_MIN_BYTES = 33, 64 << 20


class ScratchPool:
    """Device memory that some products need beyond their inputs and outputs: the library's bf16 product before its
    sum into the residual, the wide kernel's partial sums, the slice winners of the argmax.  A buffer is handed out
    again to every later call that it is large enough for, and none is freed before `clear`: captured programs keep
    the addresses.  A step function owns one pool (calls on its stream are ordered, so they can share buffers);
    calls that name no pool share DEFAULT_SCRATCH."""

    def __init__(self):
        self.buffers = {}   # (kind, device, dtype) -> [tensors]

    def get(self, kind, elements, dtype, device):
        pool = self.buffers.setdefault((kind, device, dtype), [])
        for buf in pool:
            if buf.numel() >= elements:
                return buf
        pool.append(torch.empty(1 << max(int(elements) - 1, 0).bit_length(), dtype=dtype, device=device))
        return pool[-1]

    def bytes(self):
        return sum(t.numel() * t.element_size() for pool in self.buffers.values() for t in pool)

    def clear(self):
        self.buffers.clear()


DEFAULT_SCRATCH = ScratchPool()


def library_ok(m, w, gated=False):
    """`gated`: the product of gate and up, whose activation is a kernel of its own after the library's product.  With
    weights of 64 MB and more it goes there from 33 rows on: 64 rows against the 8B sizes' 235 MB take 60.7 us there and
    69.7 in the wide kernel here (58.4 against 63.0 at 33 rows; 23.0 against 26.5 at the 1.7B sizes), the activation
    included; the other products of 33 to 64 rows are as fast here."""
    least = LIBRARY_MIN_ROWS
    if gated and w.numel() * 2 >= LIBRARY_GATED_MIN_BYTES:
        least = min(least, LIBRARY_GATED_MIN_ROWS)
    return (LIBRARY_MIN_ROWS > 0 and m >= least and w.dtype == torch.bfloat16 and w.is_contiguous()
            and w.numel() * 2 >= LIBRARY_MIN_BYTES)


def _scratch_bf16(scratch, device, rows, cols):
    return (scratch or DEFAULT_SCRATCH).get("library", rows * cols, torch.bfloat16, device)[:rows * cols].view(rows, cols)


def gemm(a, w, out, residual=None, after_norm=False, scratch=None):
    """out[M, N] = a[M, K] . w[N, K]^T (+ residual).  float operands run the true
    32-bit kernel; bf16 operands run on the matrix cores with float accumulation.
    out may be float or (bf16 operands only) bf16; residual is float and may be `out`.
    `after_norm`: a hint for the choice of kernel, see wide_ok.  `scratch`: the ScratchPool of the caller's steps."""
    m, k = a.shape
    n, k2 = w.shape
    if k != k2:
        raise KernelError(f"gemm: inner sizes differ ({k} vs {k2})")
    if a.dtype != w.dtype:
        raise KernelError(f"gemm: operand dtypes differ ({a.dtype} vs {w.dtype})")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows must be contiguous")
    if tuple(out.shape) != (m, n) or not out.is_cuda or not a.is_cuda or not w.is_cuda:
        raise KernelError("gemm: bad output shape or device")
    rp, ldr = None, 0
    if residual is not None:
        if residual.dtype != torch.float32 or out.dtype != torch.float32 or tuple(residual.shape) != (m, n) or residual.stride(1) != 1:
            raise KernelError("gemm: residual needs float [M, N] and a float output")
        rp, ldr = residual.data_ptr(), residual.stride(0)
    if a.dtype == torch.float32:
        if out.dtype != torch.float32:
            raise KernelError("gemm: float operands need a float output")
        code = lib().cisr_gemm_f32(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                   rp, ldr, m, n, k, _stream())
    elif (a.dtype == torch.bfloat16 and library_ok(m, w) and a.is_contiguous() and out.is_contiguous()
          and (out.dtype == torch.bfloat16 and residual is None or residual is out)):
        if residual is None:
            torch.mm(a, w.t(), out=out)
            return out
        product = _scratch_bf16(scratch, a.device, m, n)
        torch.mm(a, w.t(), out=product)
        return residual_add(out, product)
    elif a.dtype == torch.bfloat16 and m <= SKINNY_ROWS and _skinny_ok(a, w) and wide_ok(m, w, after_norm=after_norm):
        return _gemm_wide(a, w, out, residual, False, "gemm", scratch)
    elif a.dtype == torch.bfloat16 and m <= SKINNY_ROWS and _skinny_ok(a, w):
        code = lib().cisr_gemm_skinny_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(),
                                           out.stride(0), rp, ldr, m, n, k, _storage(out, "out"), 0, None, 0.0, None,
                                           _stream())
    elif a.dtype == torch.bfloat16:
        code = lib().cisr_gemm_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                    rp, ldr, m, n, k, _storage(out, "out"), _stream())
    else:
        raise KernelError(f"gemm: unsupported dtype {a.dtype}")
    _check(code, "gemm")
    return out


# Weights of at least this many bytes are streamed by the kernel that keeps the activations in registers
# (norm, rotary embedding and cache write are then kernels of their own); smaller ones by the kernels that
# fuse them, which cost fewer launches.  Measured on an MI355X against the other kernel in captured graphs:
# with at most 16 rows the activations are a small part of the traffic and the fused kernels hold out up to
# about 64 MB; with 17 to 32 rows the wide kernel wins from about 12 MB on, with more from about 30 MB on
# (a block then holds so much of the activations that it needs many rows of W to spread their cost over).
WIDE_MIN_BYTES_FEW_ROWS = 64 << 20
WIDE_MIN_BYTES = 12 << 20
WIDE_MIN_BYTES_MANY_ROWS = 30 << 20
_wide_plans = {}


def wide_ok(m, w, swiglu=False, after_norm=False):
    """Whether a product of m rows with the bf16 weights w runs the wide weight-streaming kernel.
    `after_norm`: the rows are the output of an RMSNorm, which the other kernel would fuse (it then reads the
    float residual and the norm's weights for every 16 rows of W, which costs it more than bf16 rows do)."""
    n, k = w.shape
    if gemv_ok(m, n, k):   # up to four rows against large weights: the matrix-vector kernel takes them
        return False
    least = WIDE_MIN_BYTES_FEW_ROWS if m <= 16 else WIDE_MIN_BYTES if m <= 32 else WIDE_MIN_BYTES_MANY_ROWS
    if m <= 16 and n < 16 * _compute_units(w.device) and k >= 4096:
        # a narrow output with a long inner size: the fused kernels have a block for every 16 columns and
        # cannot fill the GPU; this one cuts K as well
        least = min(least, max(WIDE_MIN_BYTES, 16 << 20))
    if m >= 4 and after_norm and k >= 2048:     # (one or two rows of the residual cost the fused kernel next to nothing)
        least = min(least, max(WIDE_MIN_BYTES, 24 << 20))
    if (w.dtype != torch.bfloat16 or not 0 < m <= SKINNY_ROWS or w.numel() * 2 < least or k % 8 or w.stride(0) % 8
            or w.data_ptr() % 16 or w.stride(1) != 1):
        return False
    return _wide_plan(m, n // 2 if swiglu else n, k, swiglu) >= 0


GEMV_ROWS, GEMV_MIN_BYTES = 4, 4 << 20


def gemv_ok(m, n, k):
    """Whether a product of m rows with weights [n, k] runs the matrix-vector kernel (up to four rows against weights
    of 4 MB and more with an inner size of at least 1024: a wave owns whole rows of the weights; see csrc/gemv.hip
    and the measurements in csrc/gemm_skinny.hip).  The weight-streaming entry points choose it themselves; callers ask only to know that
    the wide kernel and its separate norm are not wanted."""
    return bool(lib().cisr_gemv_ok(int(m), int(n), int(k)))


def set_gemv(rows=GEMV_ROWS, least_bytes=GEMV_MIN_BYTES):
    """The most rows (0 to 8; 0 switches it off) and the least bytes of weights that the matrix-vector kernel is given
    (least_bytes 0 also lifts the rule's least inner size): for measurements and tests.  Without arguments: the rule
    as it is."""
    lib().cisr_gemv_set(int(rows), int(least_bytes))


_units = {}


def _compute_units(device):
    if device not in _units:
        _units[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return _units[device]


def _wide_plan(m, n, k, swiglu):
    key = ((m + 15) // 16, m, n, k, swiglu)
    need = _wide_plans.get(key)
    if need is None:
        need = _wide_plans[key] = int(lib().cisr_gemm_wide_workspace(m, n, k, n if swiglu else 0))
    return need


def _wide_workspace(scratch, device, floats):
    if floats <= 0:
        return None
    return (scratch or DEFAULT_SCRATCH).get("wide", floats, torch.float32, device)


def _gemm_wide(a, w, out, residual, swiglu, what, scratch=None):
    m, k = a.shape
    n = w.shape[0] // 2 if swiglu else w.shape[0]
    need = _wide_plan(m, n, k, swiglu)
    if need < 0 or a.stride(0) % 8 or a.data_ptr() % 16:
        raise KernelError(f"{what}: shape not supported by the wide kernel")
    work = _wide_workspace(scratch, a.device, need)
    rp, ldr = (residual.data_ptr(), residual.stride(0)) if residual is not None else (None, 0)
    _check(lib().cisr_gemm_wide_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                     rp, ldr, m, n, k, _storage(out, "out"), n if swiglu else 0,
                                     None if work is None else work.data_ptr(), 0 if work is None else work.numel(),
                                     _stream()), what)
    return out


def gemm_unfinished(a, w, residual, scratch=None):
    """The product a . w^T that is to be added to the float rows `residual`, left unfinished where adding it takes a
    kernel of its own: the wide kernel's partial sums of a product cut into slices, (partial sums [slices, M, N],
    slices), or the library's bf16 product, (product [M, N], 0); rmsnorm_partials or add_partials then are that
    kernel.  None (nothing done) for every other product: call gemm."""
    m, k = a.shape
    n = w.shape[0]
    if (a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k or tuple(residual.shape) != (m, n)
            or not partials_ok(residual)):
        return None
    if library_ok(m, w):
        if not a.is_contiguous():
            return None
        product = _scratch_bf16(scratch, a.device, m, n)
        torch.mm(a, w.t(), out=product)
        return product, 0
    if not 0 < m <= SKINNY_ROWS or not _skinny_ok(a, w) or not wide_ok(m, w):
        return None
    need = _wide_plan(m, n, k, False)
    if need <= 0:
        return None
    work = _wide_workspace(scratch, a.device, need)
    _check(lib().cisr_gemm_wide_partials_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), m, n, k,
                                              work.data_ptr(), work.numel(), _stream()), "gemm_unfinished")
    return work, need // (m * n)


def _skinny_ok(a, w):
    k = a.shape[1]
    return (k % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def _norm_args(x, norm, k):
    """(weight pointer, eps, rows pointer, number of output rows) for a fused RMSNorm prologue."""
    weight, eps, rows = norm
    _dev(x, "x", torch.float32)
    if x.shape[1] != k or x.stride(0) % 8 or x.data_ptr() % 16:
        raise KernelError("fused norm: the residual rows must be 32-byte aligned floats of the product's inner size")
    wp = _dev(weight, "norm weight", torch.float32, (k,))
    rp = None if rows is None else _dev(rows, "rows", torch.int32)
    return wp, float(eps), rp, (x.shape[0] if rows is None else rows.shape[0])


def fused_norm_ok(x, w, rows_out):
    """Whether the weight-streaming kernel can take RMSNorm(x) . w^T with the norm fused (and large weights
    do not make the norm as a kernel of its own and the wide kernel the better choice)."""
    return (not wide_ok(rows_out, w, after_norm=True) and w.dtype == torch.bfloat16 and rows_out <= SKINNY_ROWS and x.dtype == torch.float32 and x.shape[1] % 8 == 0
            and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def swiglu_fused_ok(a, w_gate_up):
    """Whether gemm_swiglu runs as one kernel for these operands (no scratch buffer needed): bf16 with
    16-byte aligned rows; few rows take the weight-streaming kernel, more the tiled one."""
    return a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and a.is_cuda and _skinny_ok(a, w_gate_up)


def gemm_normed(x, norm, w, out):
    """out[R, N] = RMSNorm(x[rows]) . w^T with the norm applied inside the product's kernel.
    x float [T, K]; norm = (weight float [K], eps, rows int32 [R] or None); w bf16 [N, K]; out float or bf16."""
    n, k = w.shape
    wp, eps, rp, m = _norm_args(x, norm, k)
    if not fused_norm_ok(x, w, m) or tuple(out.shape) != (m, n) or out.stride(1) != 1:
        raise KernelError("gemm_normed: shape not supported by the fused kernel")
    _check(lib().cisr_gemm_skinny_bf16(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                       None, 0, m, n, k, _storage(out, "out"), 0, wp, eps, rp, _stream()), "gemm_normed")
    return out


def gemm_swiglu(a, w_gate_up, out, gate_up=None, norm=None, scratch=None):
    """out[M, I] = silu(a . Wg^T) * (a . Wu^T) with w_gate_up = [Wg; Wu] ([2I, K]).
    Few rows of bf16 run one fused weight-streaming kernel (with `norm` = (weight, eps, None), `a` is the float
    residual and RMSNorm is fused too); otherwise the product goes to `gate_up` [M, 2I] and the activation is
    a second kernel.  `scratch`: the ScratchPool of the caller's steps."""
    m, k = a.shape
    two_i, k2 = w_gate_up.shape
    inter = two_i // 2
    if k != k2 or two_i % 2 or tuple(out.shape) != (m, inter) or not out.is_contiguous():
        raise KernelError("gemm_swiglu: shapes do not fit")
    if norm is not None:
        wp, eps, rp, _ = _norm_args(a, norm, k)
        if not fused_norm_ok(a, w_gate_up, m) or out.dtype != torch.bfloat16:
            raise KernelError("gemm_swiglu: shape not supported by the fused kernel")
        _check(lib().cisr_gemm_skinny_bf16(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
                                           out.data_ptr(), out.stride(0), None, 0, m, inter, k, BF16, inter, wp, eps, rp,
                                           _stream()), "gemm_swiglu")
        return out
    if out.dtype != a.dtype or a.dtype != w_gate_up.dtype:
        raise KernelError("gemm_swiglu: dtypes differ")
    if a.dtype == torch.bfloat16 and library_ok(m, w_gate_up, gated=True) and a.is_contiguous():
        product = _scratch_bf16(scratch, a.device, m, two_i)
        torch.mm(a, w_gate_up.t(), out=product)
        return swiglu(product, out)
    if swiglu_fused_ok(a, w_gate_up):
        if m <= SKINNY_ROWS and wide_ok(m, w_gate_up, True, after_norm=True):
            return _gemm_wide(a, w_gate_up, out, None, True, "gemm_swiglu", scratch)
        if m <= SKINNY_ROWS:
            _check(lib().cisr_gemm_skinny_bf16(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
                                               out.data_ptr(), out.stride(0), None, 0, m, inter, k, BF16, inter, None, 0.0,
                                               None, _stream()), "gemm_swiglu")
        else:   # many rows: the tiled product with the activation as its epilogue
            _check(lib().cisr_gemm_bf16_swiglu(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
                                               out.data_ptr(), out.stride(0), m, inter, k, inter, _stream()), "gemm_swiglu")
        return out
    if gate_up is None:
        raise KernelError("gemm_swiglu: this shape needs a buffer [M, 2I] for the product of gate and up")
    gemm(a, w_gate_up, gate_up, scratch=scratch)
    return swiglu(gate_up, out)


def qkv_rope_fused_ok(a, w, head_dim, cos, normed):
    """Whether the fused projection + rotary + scatter kernel takes this shape."""
    m, k = a.shape
    if normed and wide_ok(m, w, after_norm=True):      # large weights: the norm is a kernel of its own, the projection the wide kernel
        return False
    return (w.dtype == torch.bfloat16 and m <= SKINNY_ROWS and k % 8 == 0 and head_dim % 16 == 0
            and 2 * cos.shape[1] == head_dim and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0
            and a.dtype == (torch.float32 if normed else torch.bfloat16))


def qkv_rope(a, w, q_out, positions, slots, cos, sin, kcache, vcache, heads, kv_heads, dim, page_size, norm=None, scratch=None):
    """One kernel for a decode step's projections: (RMSNorm of the float residual `a` if `norm` = (weight, eps),
    else `a` is bf16 and normed), product with w = [Wq; Wk; Wv], rotary embedding of q and k, q into
    q_out [M, heads*dim], k and v into the cache at `slots`.  kcache None: w = Wq only (a layer reading
    another layer's cache)."""
    m, k = a.shape
    has_kv = kcache is not None
    n_kv = kv_heads if has_kv else 0
    if not qkv_rope_fused_ok(a, w, dim, cos, norm is not None) or tuple(w.shape) != ((heads + 2 * n_kv) * dim, k):
        raise KernelError("qkv_rope: shape not supported by the fused kernel")
    wp, eps = (None, 0.0)
    if norm is not None:
        wp, eps = _dev(norm[0], "norm weight", torch.float32, (k,)), float(norm[1])
    kp = vp = sp = None
    if has_kv:
        pages = kcache.shape[0]
        kp = _dev(kcache, "kcache", torch.bfloat16, (pages, kv_heads, page_size, dim))
        vp = _dev(vcache, "vcache", torch.bfloat16, (pages, kv_heads, dim, page_size))
        sp = _dev(slots, "slots", torch.int32, (m,))
    max_pos = cos.shape[0]
    if norm is None and wide_ok(m, w, after_norm=True):
        need = _wide_plan(m, w.shape[0], k, False)
        work = _wide_workspace(scratch, a.device, need)
        _check(lib().cisr_qkv_rope_wide(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0),
                                        _dev(q_out, "q_out", torch.bfloat16, (m, heads * dim)), heads * dim, m, k,
                                        _dev(positions, "positions", torch.int32, (m,)), sp,
                                        _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, dim // 2)),
                                        kp, vp, heads, n_kv, dim, page_size, max_pos,
                                        None if work is None else work.data_ptr(), 0 if work is None else work.numel(),
                                        _stream()), "qkv_rope")
        return q_out
    _check(lib().cisr_qkv_rope_skinny(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0),
                                      _dev(q_out, "q_out", torch.bfloat16, (m, heads * dim)), heads * dim, m, k, wp, eps,
                                      _dev(positions, "positions", torch.int32, (m,)), sp,
                                      _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, dim // 2)),
                                      kp, vp, heads, n_kv, dim, page_size, max_pos, _stream()), "qkv_rope")
    return q_out


def attention_mfma(q, q_row_stride, kcache, vcache, tables, seg_of_row, positions, out, heads, kv_heads, dim,
                   page_size, window, scale, tasks=None, splits=1, workspace=None, waves=4, block_tiles=False,
                   item_tiles=1, row_ids=None, merge=True, key_groups=1, stream_loads=False):
    """Matrix-core attention (bf16).  tasks int32 [n, 4] = (segment, first row, rows, 0) runs tiles of
    prompt rows: one tile of 16/GC rows a block whose waves share the keys (with item_tiles=2, head sizes up to
    64: 32/GC rows, two item tiles a wave), or with `block_tiles` (head sizes up to 128) one tile of
    64 item_tiles / GC rows a block whose four waves own different rows and share keys and values through LDS
    (GC = query heads per key head, at most 16); tasks None runs one block
    per row (decode) of `waves` wavefronts (4 or 8) with `splits` blocks along the keys; splits > 1 needs
    workspace = (partials float, statistics float) and a merge.  `row_ids` (int32 [n], with tasks None): only
    the rows it lists are computed and written (negative entries are skipped): the decode rows of a mixed step.
    `merge` False (rows mode with splits > 1): the partial outputs are left unmerged in the workspace, whose first
    buffer is then bfloat16, for gemm_merged; `out` is not written.  `key_groups` 2 (block_tiles 32): a block is two
    halves that take the even and the odd 32-key steps of its items and merge at the end.  `stream_loads` (rows mode):
    keys and values are read with non-temporal loads, which the caches do not keep."""
    rows = out.shape[0]
    if not mfma_attention_supported(out.dtype, dim, page_size):
        raise KernelError(f"attention_mfma: head size {dim} / page size {page_size} / dtype {out.dtype} not supported")
    if heads % kv_heads:
        raise KernelError(f"attention: {heads} query heads do not divide into {kv_heads} key heads")
    if not scale > 0:
        raise KernelError("attention_mfma: the score scale must be positive (the maximum is taken before scaling)")
    if q.dtype != out.dtype or kcache.dtype != out.dtype or q_row_stride % 8 or q.data_ptr() % 16:
        raise KernelError("attention_mfma: q, cache and out must be bfloat16 with 16-byte aligned rows")
    if q.numel() < (rows - 1) * q_row_stride + heads * dim:
        raise KernelError("attention: q buffer too small for its stride")
    pages = kcache.shape[0]
    if kcache.numel() >= 2 ** 31 or vcache.numel() >= 2 ** 31:
        raise KernelError("attention_mfma: a layer's keys (or values) must be fewer than 2^31 elements (32-bit byte offsets)")
    dpad = -(-dim // 32) * 32
    fn = _attention_entry(dpad)
    po = pm = tp = None
    if tasks is not None:
        if item_tiles not in ((1, 2, 3, 4) if block_tiles == 32 else (1, 2)) or (item_tiles == 2 and dim > 64 and not block_tiles):
            raise KernelError("attention_mfma: two item tiles a wave need a head size of at most 64")
        if block_tiles and dpad > 128:
            raise KernelError("attention_mfma: block tiles need a head size of at most 128")
        n_tasks, splits = tasks.shape[0], 1
        mode = (2 if item_tiles == 1 else 4) if block_tiles else (3 if item_tiles == 2 else 0)
        if block_tiles == 32:
            # the 32 x 32 matrix instruction: 128/GC rows a block and four waves (item_tiles 2), or 64/GC rows and two
            if out.numel() >= 2 ** 31:
                raise KernelError("attention_mfma: the output must be fewer than 2^31 elements (32-bit offsets)")
            if page_size < 8 or dpad > 128:
                raise KernelError("attention_mfma: 32 x 32 block tiles need pages of at least 8 keys and a head size of at most 128")
            if key_groups not in (1, 2) or (key_groups == 2 and item_tiles >= 3):
                raise KernelError("attention_mfma: one or two key groups, two with 64 or 128 items a block")
            if dpad > 64 and (item_tiles == 4 or (item_tiles == 2 and key_groups == 2)):
                raise KernelError("attention_mfma: blocks of more than eight waves need a head size of at most 64")
            mode = {(1, 1): 6, (2, 1): 5, (3, 1): 10, (4, 1): 7, (1, 2): 8, (2, 2): 9}[(item_tiles, key_groups)]
        tp = _dev(tasks, "tasks", torch.int32, (n_tasks, 4))
    else:
        n_tasks, mode = rows, 1
        if row_ids is not None:
            n_tasks = row_ids.numel()
            tp = _dev(row_ids, "row_ids", torch.int32, (n_tasks,))
        if splits > 1:
            if workspace is None:
                raise KernelError("attention: split runs need a workspace")
            part_o, part_ml = workspace
            po, pm = _dev(part_o, "part_o", torch.float32 if merge else torch.bfloat16), _dev(part_ml, "part_ml", torch.float32)
            if part_o.numel() < n_tasks * heads * splits * dim or part_ml.numel() < n_tasks * heads * splits * 2:
                raise KernelError("attention: split workspace too small")
    _check(fn(q.data_ptr(), q_row_stride, _dev(kcache, "kcache", None, (pages, kv_heads, page_size, dim)),
              _dev(vcache, "vcache", None, (pages, kv_heads, dim, page_size)), _dev(tables, "tables", torch.int32),
              tables.shape[1], tp, n_tasks, _dev(seg_of_row, "seg_of_row", torch.int32, (rows,)),
              _dev(positions, "positions", torch.int32, (rows,)), _dev(out, "out", None, (rows, heads * dim)), po, pm,
              heads, kv_heads, dim, page_size.bit_length() - 1, int(window or 0), float(scale), int(splits),
              11 if mode == 1 and stream_loads else mode, int(waves),
              int(mode == 1 and splits > 1 and not merge), _stream()), "attention_mfma")
    if mode == 1 and splits > 1 and merge:
        _check(lib().cisr_attn_merge(po, pm, out.data_ptr(), n_tasks, heads, dim, int(splits), tp, _stream()), "attention_merge")
    return out


def gemm_merged_ok(m, w, heads, dim, splits):
    """Whether gemm_merged takes m rows of `splits` partial attention results of heads x dim against the bf16 weights w."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == heads * dim and w.stride(1) == 1 and w.stride(0) % 8 == 0
            and w.data_ptr() % 16 == 0 and bool(lib().cisr_gemm_merged_ok(int(m), int(w.shape[0]), int(heads), int(dim), int(splits))))


def gemm_merged(partials, heads, dim, w, out, residual):
    """out[M, N] = residual + merge(partials) . w^T in float: the output projection of a decode step whose attention
    was split over `splits` blocks along the keys and left unmerged (attention_mfma with merge=False).
    partials = (bf16 [M, heads, splits, dim] normalised partial outputs, float [M, heads, splits, 2] statistics, splits)."""
    part_o, part_ml, splits = partials
    m, n = out.shape
    if not gemm_merged_ok(m, w, heads, dim, splits) or w.shape[0] != n:
        raise KernelError("gemm_merged: shape not supported by the fused kernel")
    if out.dtype != torch.float32 or out.stride(1) != 1 or tuple(residual.shape) != (m, n) or residual.dtype != torch.float32 or residual.stride(1) != 1:
        raise KernelError("gemm_merged: float output and residual [M, N]")
    if part_o.numel() < m * heads * splits * dim or part_ml.numel() < m * heads * splits * 2:
        raise KernelError("gemm_merged: partial results too small")
    _check(lib().cisr_gemm_merged_bf16(_dev(part_o, "part_o", torch.bfloat16), _dev(part_ml, "part_ml", torch.float32), int(splits),
                                       int(heads), int(dim), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                       residual.data_ptr(), residual.stride(0), m, n, _stream()), "gemm_merged")
    return out


def mfma_attention_supported(dtype, dim, page_size):
    return (dtype == torch.bfloat16 and dim % 8 == 0 and dim <= 256 and page_size >= 8
            and page_size & (page_size - 1) == 0)



def _scatter(out, index, rows):
    """(pointer of index or None, length of out) for a token choice that writes out[index[r]]."""
    if index is None:
        _dev(out, "out", torch.int32, (rows,))
        return None, rows
    _dev(out, "out", torch.int32)
    return _dev(index, "index", torch.int32, (rows,)), out.numel()


def argmax(logits, out, index=None, scratch=None):
    """out[r] = index of the largest logit of row r (the lowest index wins a tie).  With `index`
    (int32 [R]) the result of row r goes to out[index[r]] instead, or nowhere if that is no place of out."""
    rows, vocab = logits.shape
    pool = scratch or DEFAULT_SCRATCH
    val = pool.get("argmax", rows * 32, torch.float32, logits.device)
    idx = pool.get("argmax", rows * 32, torch.int32, logits.device)
    where, out_n = _scatter(out, index, rows)
    _check(lib().cisr_argmax(_dev(logits, "logits", torch.float32), out.data_ptr(), where, out_n,
                             val.data_ptr(), idx.data_ptr(), rows, vocab, _stream()), "argmax")
    return out


def sample(logits, temperature, seeds, counters, out, index=None):
    """Temperature sampling per row; temperature <= 0 is greedy.  seeds/counters int64 [R].
    `index` as for argmax."""
    rows, vocab = logits.shape
    where, out_n = _scatter(out, index, rows)
    _check(lib().cisr_sample(_dev(logits, "logits", torch.float32), _dev(temperature, "temperature", torch.float32, (rows,)),
                             _dev(seeds, "seeds", torch.int64, (rows,)), _dev(counters, "counters", torch.int64, (rows,)),
                             out.data_ptr(), where, out_n, rows, vocab, _stream()), "sample")
    return out


def take_tokens(tokens, source, sampled):
    """tokens[r] = sampled[source[r]] for the rows whose source is a place of `sampled` (all int32)."""
    rows = tokens.numel()
    _check(lib().cisr_take_tokens(_dev(tokens, "tokens", torch.int32), _dev(source, "source", torch.int32, (rows,)),
                                  _dev(sampled, "sampled", torch.int32), rows, sampled.numel(), _stream()), "take_tokens")
    return tokens
