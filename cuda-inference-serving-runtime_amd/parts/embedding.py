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

    def forward(self, h, ctx):
        logits = ctx.buffer("logits", (h.shape[0], self.vocab), torch.float32)
        return ops.gemm(h, self.weight, logits)
