"""Arrangement of parts in a layer.  PreNormBlock is the Llama arrangement
(reference: runtime/model.py:106-119): x = x + mixer(norm1(x)); x = x + ffn(norm2(x)),
the residual stream x kept in float."""
from .base import Part, register_part


class PreNormBlock(Part):
    def __init__(self, mixer_norm, mixer, ffn_norm, ffn):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype):
        for p in self.parts():
            p.bind(tensors, dtype)

    def prepare(self, device, dtype):
        for p in self.parts():
            p.prepare(device, dtype)

    def forward(self, residual, ctx, site):
        if self.mixer.fuses_norm(self.mixer_norm, residual, ctx):
            residual = self.mixer.forward(None, residual, ctx, site, norm=self.mixer_norm)
        else:
            residual = self.mixer.forward(self.mixer_norm.forward(residual, ctx), residual, ctx, site)
        if self.ffn.fuses_norm(self.ffn_norm, residual, ctx):
            return self.ffn.forward(None, residual, ctx, norm=self.ffn_norm)
        return self.ffn.forward(self.ffn_norm.forward(residual, ctx), residual, ctx)


register_part("block", "prenorm", PreNormBlock)
