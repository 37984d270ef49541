"""Grouped-query attention over the paged cache.

q = h Wq^T, k = h Wk^T, v = h Wv^T; q and k take the position encoding; k and v
go into the cache at the step's slots; every row then attends to its request's
cached keys up to its own position (or the last `window` of them), scale
1/sqrt(head_dim) unless given; the result goes through Wo and is added to the
residual (reference: runtime/model.py:110-115).  The three projections run as
one product against the concatenated weight [q; k; v] (a layout choice only).

A mixer built with `own_kv` False has no k/v projections: it attends to
the cache another layer wrote.  With `bias` the q/k/v projections add
`<name>.{q,k,v}_proj.bias` before the position encoding, with `out_bias` the output
projection adds `<name>.o_proj.bias`: the products run as they are and a small kernel
adds the bias (the fused projection kernels have no bias and are not used then).
"""
import math

import torch

from ..cache.pages import KVNeed
from ..kernels import attention as kernel, ops
from .base import Mixer, TensorSpec, matrix_operand, register_part


class PagedAttention(Mixer):
    def __init__(self, name, hidden, heads, kv_heads, head_dim, position, window=None, scale=None, own_kv=True,
                 bias=False, out_bias=False, tuning=None):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads are not a multiple of {kv_heads} key/value heads")
        if head_dim % 2 or head_dim > 256:
            raise ValueError(f"head size {head_dim} must be even and at most 256")
        self.name, self.hidden, self.heads, self.kv_heads, self.head_dim = name, hidden, heads, kv_heads, head_dim
        self.position, self.window, self.own_kv = position, window, own_kv
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.bias, self.out_bias = bool(bias), bool(out_bias)
        self.w_in = self.w_out = self.b_in = self.b_out = None
        self.tuning = tuning if tuning is not None else kernel.DEFAULT_TUNING   # what the kernel's launch rules may be told

    def kernel_units(self, dtype):
        return kernel.kernel_units(self.head_dim, dtype)

    def step_arrays(self):
        return [kernel.SingleRows(self.tuning.split_single_from), kernel.RowsLongestFirst()]

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window) if self.own_kv else None

    def cache_read(self):
        return None if self.own_kv else KVNeed(self.kv_heads, self.head_dim, self.window)

    def tensor_specs(self):
        n, H, D = self.name, self.hidden, self.head_dim
        specs = [TensorSpec(f"{n}.q_proj.weight", (self.heads * D, H))]
        if self.own_kv:
            specs += [TensorSpec(f"{n}.k_proj.weight", (self.kv_heads * D, H)),
                      TensorSpec(f"{n}.v_proj.weight", (self.kv_heads * D, H))]
        specs.append(TensorSpec(f"{n}.o_proj.weight", (H, self.heads * D)))
        if self.bias:
            specs.append(TensorSpec(f"{n}.q_proj.bias", (self.heads * D,)))
            if self.own_kv:
                specs += [TensorSpec(f"{n}.k_proj.bias", (self.kv_heads * D,)), TensorSpec(f"{n}.v_proj.bias", (self.kv_heads * D,))]
        if self.out_bias:
            specs.append(TensorSpec(f"{n}.o_proj.bias", (H,)))
        return specs

    def bind(self, tensors, dtype):
        names = ["q_proj"] + (["k_proj", "v_proj"] if self.own_kv else [])
        parts = [matrix_operand(tensors[f"{self.name}.{p}.weight"], dtype) for p in names]
        self.w_in = torch.cat(parts, dim=0).contiguous() if len(parts) > 1 else parts[0]
        self.w_out = matrix_operand(tensors[f"{self.name}.o_proj.weight"], dtype)
        if self.bias:   # (a bias keeps the type it is stored in; it is added in float)
            self.b_in = torch.cat([tensors[f"{self.name}.{p}.bias"] for p in names], dim=0).contiguous()
        if self.out_bias:
            self.b_out = tensors[f"{self.name}.o_proj.bias"].contiguous()

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    @property
    def _interleaved(self):
        return getattr(self.position, "pairing", "split_half") == "interleaved"

    def _fused_projection_ok(self, a, normed):
        cos, _ = self.position.tables()
        # (the fused kernels turn split-half pairs only; another pairing takes the general rotary kernel)
        return not self._interleaved and not self.bias and ops.qkv_rope_fused_ok(a, self.w_in, self.head_dim, cos, normed)

    def fuses_norm(self, norm, residual, ctx):
        return getattr(norm, "fusable_as", None) == "rms" and self._fused_projection_ok(residual, True)

    def forward(self, h, residual, ctx, site, norm=None):
        T = residual.shape[0]
        D, nh, nkv = self.head_dim, self.heads, self.kv_heads
        gid, kcache, vcache = ctx.cache.pages_of_site(site)
        view = ctx.kv[gid]
        cos, sin = self.position.tables()
        if not self.own_kv:
            kcache_w = vcache_w = slots = None
        else:
            kcache_w, vcache_w, slots = kcache, vcache, view.slots
        if norm is not None or self._fused_projection_ok(h, False):
            # few rows: norm, projections, rotary embedding and the cache write are one kernel
            q, q_stride = ctx.buffer("attn.q", (T, nh * D), ctx.dtype), nh * D
            ops.qkv_rope(residual if norm is not None else h, self.w_in, q, ctx.positions, slots, cos, sin,
                         kcache_w, vcache_w, nh, nkv, D, view.page_size,
                         norm=(norm.weight, norm.eps) if norm is not None else None, scratch=ctx.scratch)
        else:
            q_stride = (nh + (2 * nkv if self.own_kv else 0)) * D
            q = ctx.buffer("attn.qkv", (T, q_stride), ctx.dtype)
            ops.gemm(h, self.w_in, q, scratch=ctx.scratch)
            if self.b_in is not None:
                ops.bias_add(q, self.b_in)
            ops.rope_scatter(q, ctx.positions, slots, cos, sin, kcache_w, vcache_w, nh, nkv, D, view.page_size,
                             interleaved=self._interleaved)
        out = ctx.buffer("attn.out", (T, nh * D), ctx.dtype)
        # a decode step of few rows may leave the partial results of its split keys to the output projection
        unmerged = kernel.paged_attention(ctx, q, q_stride, kcache, vcache, view, out, nh, nkv, D, self.window, self.scale,
                                          defer_merge=lambda splits: ops.gemm_merged_ok(T, self.w_out, nh, D, splits),
                                          tuning=self.tuning)
        if unmerged is not None:
            residual = ops.gemm_merged(unmerged, nh, D, self.w_out, residual, residual)
        else:
            residual = ctx.add_product(out, self.w_out, residual)
        if self.b_out is not None:
            ops.bias_add(residual, self.b_out)   # (sums commute: slices of the product that a later norm adds may still be out)
        return residual


register_part("mixer", "attention", PagedAttention)
