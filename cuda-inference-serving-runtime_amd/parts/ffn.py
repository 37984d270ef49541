"""Gated feed-forward (SwiGLU): x + (silu(h Wg^T) * (h Wu^T)) Wd^T
(reference: runtime/model.py:116-119).  Gate and up run as one product against
the concatenated weight [gate; up].  With `bias` every projection adds `<name>.*_proj.bias`:
the products run as they are and a small kernel adds the bias (no fused activation then)."""
import torch

from ..kernels import ops
from .base import FeedForward, TensorSpec, matrix_operand, register_part


class GatedMLP(FeedForward):
    def __init__(self, name, hidden, intermediate, activation="silu", bias=False):
        if activation != "silu":
            raise ValueError(f"activation {activation!r}: only silu has a kernel")
        self.name, self.hidden, self.intermediate = name, hidden, intermediate
        self.bias = bool(bias)
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def tensor_specs(self):
        n, H, I = self.name, self.hidden, self.intermediate
        specs = [TensorSpec(f"{n}.gate_proj.weight", (I, H)), TensorSpec(f"{n}.up_proj.weight", (I, H)),
                 TensorSpec(f"{n}.down_proj.weight", (H, I))]
        if self.bias:
            specs += [TensorSpec(f"{n}.gate_proj.bias", (I,)), TensorSpec(f"{n}.up_proj.bias", (I,)), TensorSpec(f"{n}.down_proj.bias", (H,))]
        return specs

    def bind(self, tensors, dtype):
        gate = matrix_operand(tensors[f"{self.name}.gate_proj.weight"], dtype)
        up = matrix_operand(tensors[f"{self.name}.up_proj.weight"], dtype)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = matrix_operand(tensors[f"{self.name}.down_proj.weight"], dtype)
        if self.bias:   # (a bias keeps the type it is stored in; it is added in float)
            self.b_gate_up = torch.cat([tensors[f"{self.name}.gate_proj.bias"], tensors[f"{self.name}.up_proj.bias"]], dim=0).contiguous()
            self.b_down = tensors[f"{self.name}.down_proj.bias"].contiguous()

    def fuses_norm(self, norm, residual, ctx):
        return not self.bias and getattr(norm, "fusable_as", None) == "rms" and ops.fused_norm_ok(residual, self.w_gate_up, residual.shape[0])

    def forward(self, h, residual, ctx, norm=None):
        T = residual.shape[0]
        act = ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype)
        if self.bias:
            gate_up = ops.gemm(h, self.w_gate_up, ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype), scratch=ctx.scratch)
            ops.swiglu(ops.bias_add(gate_up, self.b_gate_up), act)
            return ops.bias_add(ctx.add_product(act, self.w_down, residual), self.b_down)
        if norm is not None:
            ops.gemm_swiglu(residual, self.w_gate_up, act, norm=(norm.weight, norm.eps, None), scratch=ctx.scratch)
        elif ops.swiglu_fused_ok(h, self.w_gate_up):
            ops.gemm_swiglu(h, self.w_gate_up, act, scratch=ctx.scratch)   # one kernel: product and activation
        else:
            ops.gemm_swiglu(h, self.w_gate_up, act, gate_up=ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype), scratch=ctx.scratch)
        return ctx.add_product(act, self.w_down, residual)


register_part("ffn", "gated_mlp", GatedMLP)
