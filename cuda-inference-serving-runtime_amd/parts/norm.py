"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w in float
(reference: runtime/reference.py:5-6, kernels/ops.cu:3-19)."""
import torch

from ..kernels import ops
from .base import Part, TensorSpec, register_part


class RMSNorm(Part):
    # What a kernel that takes over this norm must compute: "rms" = x * rsqrt(mean(x^2) + eps) * weight, with the
    # attributes `weight` (float [dim]) and `eps`.  A mixer, feed-forward or head fuses any norm that says so.
    fusable_as = "rms"
    adds_partials = True    # forward adds the partial sums of a product left unfinished before it (ctx.add_product)

    def __init__(self, name, dim, eps):
        self.name, self.dim, self.eps = name, dim, float(eps)
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name + ".weight", (self.dim,), init="one_plus_normal")]

    def bind(self, tensors, dtype):
        self.weight = tensors[self.name + ".weight"].to(torch.float32).contiguous()  # exact widening

    def forward(self, x, ctx, rows=None, tag="norm"):
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = ctx.buffer(tag, (n_out, self.dim), ctx.dtype)
        partials = ctx.take_unfinished(x)
        if partials is not None:
            # the product before was left as partial sums: they, the residual and the norm are one kernel
            if rows is None and ops.partials_ok(x):
                return ops.rmsnorm_partials(x, partials, self.weight, out, self.eps)
            ops.add_partials(x, partials)
        return ops.rmsnorm(x, self.weight, out, self.eps, rows)


register_part("norm", "rmsnorm", RMSNorm)
