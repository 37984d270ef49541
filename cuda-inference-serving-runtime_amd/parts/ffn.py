"""Gated feed-forward (SwiGLU): x + (silu(h Wg^T) * (h Wu^T)) Wd^T
(reference: runtime/model.py:116-119).  Gate and up run as one product against
the concatenated weight [gate; up]."""
import torch

from ..kernels import ops
from .base import FeedForward, TensorSpec, matrix_operand, register_part


class GatedMLP(FeedForward):
    def __init__(self, name, hidden, intermediate, activation="silu"):
        if activation != "silu":
            raise ValueError(f"activation {activation!r}: only silu has a kernel")
        self.name, self.hidden, self.intermediate = name, hidden, intermediate
        self.w_gate_up = self.w_down = None

    def tensor_specs(self):
        n, H, I = self.name, self.hidden, self.intermediate
        return [TensorSpec(f"{n}.gate_proj.weight", (I, H)), TensorSpec(f"{n}.up_proj.weight", (I, H)),
                TensorSpec(f"{n}.down_proj.weight", (H, I))]

    def bind(self, tensors, dtype):
        gate = matrix_operand(tensors[f"{self.name}.gate_proj.weight"], dtype)
        up = matrix_operand(tensors[f"{self.name}.up_proj.weight"], dtype)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = matrix_operand(tensors[f"{self.name}.down_proj.weight"], dtype)

    def fuses_norm(self, norm, residual, ctx):
        return getattr(norm, "fusable_as", None) == "rms" and ops.fused_norm_ok(residual, self.w_gate_up, residual.shape[0])

    def forward(self, h, residual, ctx, norm=None):
        T = residual.shape[0]
        act = ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype)
        if norm is not None:
            ops.gemm_swiglu(residual, self.w_gate_up, act, norm=(norm.weight, norm.eps, None))
        elif ops.swiglu_fused_ok(h, self.w_gate_up):
            ops.gemm_swiglu(h, self.w_gate_up, act)   # one kernel: product and activation
        else:
            ops.gemm_swiglu(h, self.w_gate_up, act, scratch=ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype))
        return ctx.add_product(act, self.w_down, residual)


register_part("ffn", "gated_mlp", GatedMLP)
