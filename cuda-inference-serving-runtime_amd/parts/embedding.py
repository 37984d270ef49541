"""Token embedding and output head.

x0[r] = E[token_r] with no scaling (reference: runtime/model.py:105); logits =
h . W^T with W the head's own matrix or, when tied, the embedding matrix
(reference: runtime/checkpoint.py:38-39).  Logits are always float.
"""
import torch

from ..kernels import ops
from .base import Part, TensorSpec, matrix_operand


class TokenEmbedding(Part):
    def __init__(self, name, vocab, hidden):
        self.name, self.vocab, self.hidden = name, vocab, hidden
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name + ".weight", (self.vocab, self.hidden))]

    def bind(self, tensors, dtype):
        self.weight = matrix_operand(tensors[self.name + ".weight"], dtype)

    def forward(self, ctx):
        out = ctx.buffer("residual", (ctx.tokens.shape[0], self.hidden), torch.float32)
        return ops.embedding(ctx.tokens, self.weight, out)


class LMHead(Part):
    def __init__(self, name, vocab, hidden, tied_to=None):
        self.name, self.vocab, self.hidden, self.tied_to = name, vocab, hidden, tied_to
        self.weight = None

    def tensor_specs(self):
        return [] if self.tied_to is not None else [TensorSpec(self.name + ".weight", (self.vocab, self.hidden))]

    def bind(self, tensors, dtype):
        self.weight = self.tied_to.weight if self.tied_to is not None else matrix_operand(tensors[self.name + ".weight"], dtype)

    def fuses_norm(self, norm, residual, rows):
        return getattr(norm, "fusable_as", None) == "rms" and ops.fused_norm_ok(residual, self.weight, rows.shape[0])

    def forward(self, h, ctx, norm=None, residual=None):
        """Logits of the normed rows h; or, with `norm`, of RMSNorm(residual[ctx.logit_rows]) in one kernel."""
        n = ctx.logit_rows.shape[0] if norm is not None else h.shape[0]
        logits = ctx.buffer("logits", (n, self.vocab), torch.float32)
        if norm is not None:
            return ops.gemm_normed(residual, (norm.weight, norm.eps, ctx.logit_rows), self.weight, logits)
        return ops.gemm(h, self.weight, logits, after_norm=True, scratch=ctx.scratch)
