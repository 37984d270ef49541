"""Choosing the next token from float logits on the GPU.

Greedy is the reference's only rule (argmax, runtime/engine.py:99; the lowest
index wins a tie).  Temperature sampling draws from softmax(logits / T) by
inverse CDF with a random number that is a function of (request seed, index of
the generated token) only, so what a request samples does not depend on what
else is in the batch or how its prompt was cut.  T <= 0 means greedy.
"""
import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


def _splitmix64(x):
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform01(seed, counter):
    """Host twin of the kernel's random number in [0, 1) (24 bits)."""
    h = _splitmix64(_splitmix64(seed & _MASK) ^ ((counter * 0xD1342543DE82EF95) & _MASK))
    return (h >> 40) / 16777216.0


def _as_i64(value):
    value &= _MASK
    return value - (1 << 64) if value >= (1 << 63) else value


class Sampler:
    """pick(logits, params) -> list of token ids.  params: one (temperature, seed, counter) per row."""

    def pick(self, logits, params):
        rows = logits.shape[0]
        if rows == 0:
            return []
        if len(params) != rows:
            raise ValueError("one (temperature, seed, counter) per row of logits is required")
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        if all(not (p[0] > 0) for p in params):
            ops.argmax(logits, out)
        else:
            dev = logits.device
            temperature = torch.tensor([float(p[0]) for p in params], dtype=torch.float32, device=dev)
            seeds = torch.tensor([_as_i64(int(p[1])) for p in params], dtype=torch.int64, device=dev)
            counters = torch.tensor([_as_i64(int(p[2])) for p in params], dtype=torch.int64, device=dev)
            ops.sample(logits, temperature, seeds, counters, out)
        return out.cpu().tolist()
