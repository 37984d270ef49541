"""Grouped-query attention over the paged cache.

q = h Wq^T, k = h Wk^T, v = h Wv^T; q and k take the position encoding; k and v
go into the cache at the step's slots; every row then attends to its request's
cached keys up to its own position (or the last `window` of them), scale
1/sqrt(head_dim) unless given; the result goes through Wo and is added to the
residual (reference: runtime/model.py:110-115).  The three projections run as
one product against the concatenated weight [q; k; v] (a layout choice only).

A mixer built with `reads_site_of` set has no k/v projections: it attends to
the cache another layer wrote.
"""
import math

import torch

from ..cache.pages import KVNeed
from ..kernels import ops
from .base import Mixer, TensorSpec, matrix_operand, register_part


class PagedAttention(Mixer):
    def __init__(self, name, hidden, heads, kv_heads, head_dim, position, window=None, scale=None, own_kv=True):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads are not a multiple of {kv_heads} key/value heads")
        if head_dim % 2 or head_dim > 256:
            raise ValueError(f"head size {head_dim} must be even and at most 256")
        self.name, self.hidden, self.heads, self.kv_heads, self.head_dim = name, hidden, heads, kv_heads, head_dim
        self.position, self.window, self.own_kv = position, window, own_kv
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.w_in = self.w_out = None

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window) if self.own_kv else None

    def tensor_specs(self):
        n, H, D = self.name, self.hidden, self.head_dim
        specs = [TensorSpec(f"{n}.q_proj.weight", (self.heads * D, H))]
        if self.own_kv:
            specs += [TensorSpec(f"{n}.k_proj.weight", (self.kv_heads * D, H)),
                      TensorSpec(f"{n}.v_proj.weight", (self.kv_heads * D, H))]
        return specs + [TensorSpec(f"{n}.o_proj.weight", (H, self.heads * D))]

    def bind(self, tensors, dtype):
        names = ["q_proj"] + (["k_proj", "v_proj"] if self.own_kv else [])
        parts = [matrix_operand(tensors[f"{self.name}.{p}.weight"], dtype) for p in names]
        self.w_in = torch.cat(parts, dim=0).contiguous() if len(parts) > 1 else parts[0]
        self.w_out = matrix_operand(tensors[f"{self.name}.o_proj.weight"], dtype)

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def forward(self, h, residual, ctx, site):
        T = h.shape[0]
        D, nh, nkv = self.head_dim, self.heads, self.kv_heads
        width = (nh + (2 * nkv if self.own_kv else 0)) * D
        qkv = ctx.buffer("attn.qkv", (T, width), ctx.dtype)
        ops.gemm(h, self.w_in, qkv)
        gid, kcache, vcache = ctx.cache.kv_of_site(site)
        view = ctx.kv[gid]
        cos, sin = self.position.tables()
        if self.own_kv:
            ops.rope_scatter(qkv, ctx.positions, view.slots, cos, sin, kcache, vcache, nh, nkv, D, view.page_size)
        else:
            ops.rope_scatter(qkv, ctx.positions, None, cos, sin, None, None, nh, nkv, D, view.page_size)
        out = ctx.buffer("attn.out", (T, nh * D), ctx.dtype)
        ctx.attend(qkv, width, kcache, vcache, view, out, nh, nkv, D, self.window, self.scale)
        return ops.gemm(out, self.w_out, residual, residual=residual)


register_part("mixer", "attention", PagedAttention)
