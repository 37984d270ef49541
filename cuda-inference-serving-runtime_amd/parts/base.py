"""Interfaces of the parts a layer is put together from, and their registry.

A part knows its own sizes and constants (constructor parameters), the tensors
it owns (names, shapes), and how to run on a step's rows.  It does not know
which model it is in.  Kinds of part:

  norm      forward(x_float[T, H], ctx, rows=None) -> activations [T or R, H]
  position  tables(device) -> (cos, sin) float [max_pos, rot/2] used by mixers
  mixer     forward(h[T, H], residual[T, H] float, ctx, site, norm=None) -> residual
  ffn       forward(h[T, H], residual[T, H] float, ctx, norm=None) -> residual
  block     forward(residual, ctx, site) -> residual  (the arrangement of the four)

Mixers and feed-forwards add their result to the float residual stream
themselves (their last matrix product does it in its epilogue) and return it.
A mixer or feed-forward may take over the norm in front of it: if its
`fuses_norm(norm, residual, ctx)` says so for a step, the block passes h=None
and the norm part, and the part applies the norm inside its first kernel.  Which
norms can be taken over is a capability the norm states (`fusable_as`: "rms"
with `weight` and `eps`), not a class.
A mixer states what it keeps between steps: `cache_need()` (pages of keys and
values) and/or `state_need()` (a fixed-size state per request), or neither.
"""
from ..weights.loader import TensorSpec  # noqa: F401  (parts import it from here)

_PARTS = {}

KINDS = ("norm", "position", "mixer", "ffn", "block")


def register_part(kind, name, factory):
    if kind not in KINDS:
        raise ValueError(f"unknown kind of part {kind!r}; kinds: {KINDS}")
    if (kind, name) in _PARTS:
        raise ValueError(f"{kind} {name!r} is already registered")
    _PARTS[(kind, name)] = factory


def unregister_part(kind, name):
    _PARTS.pop((kind, name), None)


def make_part(kind, family, /, **params):
    """Build the part registered as (kind, family) with its own parameters."""
    try:
        factory = _PARTS[(kind, family)]
    except KeyError:
        known = sorted(n for k, n in _PARTS if k == kind)
        raise KeyError(f"no {kind} named {family!r}; registered: {known}") from None
    return factory(**params)


class Part:
    """Base of every part."""

    def tensor_specs(self):
        return []

    def bind(self, tensors, dtype):
        """Take the loaded tensors this part declared (dict by full name).
        `dtype` is the compute dtype (torch.float32 or torch.bfloat16)."""

    def prepare(self, device, dtype):
        """Build tables and the like on the device (no weights involved)."""


class Mixer(Part):
    def cache_need(self):
        return None

    def cache_read(self):
        """What a mixer that keeps no cache expects of the cache the order of layers lets it read (a KVNeed: heads,
        head size, and the window it looks back over; None: it reads none, or cannot say).  The model checks it
        against what the layer it reads keeps."""
        return None

    def state_need(self):
        return None

    def fuses_norm(self, norm, residual, ctx):
        return False

    def forward(self, h, residual, ctx, site, norm=None):
        raise NotImplementedError


class FeedForward(Part):
    def fuses_norm(self, norm, residual, ctx):
        return False

    def forward(self, h, residual, ctx, norm=None):
        raise NotImplementedError


def matrix_operand(t, dtype):
    """A stored matrix as a GEMM operand of the compute dtype.  bf16 -> float
    widening is exact; a 32-bit matrix run in bf16 is rounded to nearest even by
    the conversion kernel."""
    import torch
    from ..kernels import ops
    if t.dtype == dtype:
        return t.contiguous()
    if dtype == torch.float32:
        return t.to(torch.float32).contiguous()
    if t.dtype == torch.float32 and dtype == torch.bfloat16:
        return ops.f32_to_bf16(t.contiguous(), torch.empty_like(t, dtype=torch.bfloat16))
    raise TypeError(f"cannot use a {t.dtype} matrix in {dtype} arithmetic")
