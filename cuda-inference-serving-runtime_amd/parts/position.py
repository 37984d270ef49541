"""Position encodings applied to queries and keys before keys are cached.

RotaryEmbedding is the split-half rotary embedding: coordinate pair
(i, i + rot/2) of a head turns by pos * theta^(-2i/rot)
(reference: runtime/reference.py:9-15, kernels/ops.cu:21-33).  Angles are
computed on the host in float64 and stored as float cosine/sine tables, so the
kernels do no transcendental arithmetic.  NoPosition turns nothing.

What a position part gives a mixer: `tables() -> (cos, sin)` float
[max_positions, pairs], and `pairing`: which two coordinates of a head pair i
is, "split_half" (i, i + pairs) or "interleaved" (2i, 2i + 1).  A part without
the attribute is split-half.
"""
import numpy as np
import torch

from .base import Part, register_part


class RotaryEmbedding(Part):
    def __init__(self, head_dim, theta, max_positions, rotary_dim=None, pairing="split_half"):
        if pairing not in ("split_half", "interleaved"):
            raise ValueError(f"pairing {pairing!r} is neither split_half nor interleaved")
        self.pairing = pairing
        self.head_dim, self.theta, self.max_positions = head_dim, float(theta), int(max_positions)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary size {self.rotary_dim} must be even and at most the head size {head_dim}")
        self._tables = None

    def angles(self):
        half = self.rotary_dim // 2
        inv_freq = np.float64(self.theta) ** (-np.arange(half, dtype=np.float64) * 2.0 / self.rotary_dim)
        return np.arange(self.max_positions, dtype=np.float64)[:, None] * inv_freq[None, :]

    def prepare(self, device, dtype):
        if self._tables is not None and self._tables[0].device == torch.device(device):
            return                      # one part may serve many layers: its tables are built once
        a = self.angles()
        self._tables = (torch.from_numpy(np.cos(a).astype(np.float32)).to(device).contiguous(),
                        torch.from_numpy(np.sin(a).astype(np.float32)).to(device).contiguous())

    def tables(self):
        return self._tables


class NoPosition(Part):
    """Identity: a one-pair table with angle zero."""
    pairing = "split_half"

    def __init__(self, head_dim, max_positions=1, **_):
        self.head_dim, self.max_positions = head_dim, int(max_positions)
        self._tables = None

    def prepare(self, device, dtype):
        if self._tables is not None and self._tables[0].device == torch.device(device):
            return
        self._tables = (torch.ones(self.max_positions, 1, dtype=torch.float32, device=device),
                        torch.zeros(self.max_positions, 1, dtype=torch.float32, device=device))

    def tables(self):
        return self._tables


register_part("position", "rotary", RotaryEmbedding)
register_part("position", "none", NoPosition)
