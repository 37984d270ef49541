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

    # What the block keeps between steps, asked of the block (not of a part inside it): one mixer here, so one need
    # of each kind; an arrangement with more parts that keep something answers for all of them.
    def cache_need(self):
        return self.mixer.cache_need()

    def cache_read(self):
        return self.mixer.cache_read() if hasattr(self.mixer, "cache_read") else None

    def state_need(self):
        return self.mixer.state_need()

    def kernel_units(self, dtype):
        """Shared objects beside the core that the parts need (names of kernels.library.units())."""
        return [u for p in self.parts() if hasattr(p, "kernel_units") for u in p.kernel_units(dtype)]

    def step_arrays(self):
        """Step arrays that the parts want every step's metadata to carry from the start (engine.context.StepArray)."""
        return [a for p in self.parts() if hasattr(p, "step_arrays") for a in p.step_arrays()]

    def first_norm(self):
        """The norm that reads the residual stream first: the block before may leave its last product to it."""
        return self.mixer_norm

    def forward(self, residual, ctx, site):
        # ctx.next_norm names the norm that reads the residual stream after the part that runs: a part's last
        # product may be left to it (ctx.add_product); on entry it is the norm after this block
        after = ctx.next_norm
        ffn_fuses = self.ffn.fuses_norm(self.ffn_norm, residual, ctx)
        ctx.next_norm = None if ffn_fuses else self.ffn_norm
        if self.mixer.fuses_norm(self.mixer_norm, residual, ctx):
            ctx.settle(residual)
            residual = self.mixer.forward(None, residual, ctx, site, norm=self.mixer_norm)
        else:
            residual = self.mixer.forward(self.mixer_norm.forward(residual, ctx), residual, ctx, site)
        if ffn_fuses:
            ctx.settle(residual)
            ctx.next_norm = after
            return self.ffn.forward(None, residual, ctx, norm=self.ffn_norm)
        h = self.ffn_norm.forward(residual, ctx)
        ctx.settle(residual)       # (a norm that adds no partial sums)
        ctx.next_norm = after
        return self.ffn.forward(h, residual, ctx)


register_part("block", "prenorm", PreNormBlock)
