"""Plain temperature sampling for the tests: float64 softmax(logits / T) and an inverse-CDF draw.

The reference picks greedily only (runtime/engine.py:99: argmax, lowest index on a tie), so the sampling rule
is this engine's own definition, restated here from its description and sharing no code with it:
  u      = uniform01(seed, index of the generated token), 24 random bits in [0, 1)
  token  = the first index whose cumulative probability exceeds u.
uniform01 is splitmix64 applied twice: h = mix(mix(seed) xor (index * 0xD1342543DE82EF95)), u = (h >> 40) / 2^24.
"""
import numpy as np

_M = (1 << 64) - 1


def mix(x):
    x = (x + 0x9E3779B97F4A7C15) & _M
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _M
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _M
    return x ^ (x >> 31)


def uniform01(seed, index):
    return (mix(mix(seed & _M) ^ ((index * 0xD1342543DE82EF95) & _M)) >> 40) / float(1 << 24)


def cdf(logits, temperature):
    z = np.asarray(logits, np.float64) / temperature
    p = np.exp(z - z.max())
    return np.cumsum(p / p.sum())


def draw(logits, temperature, seed, index):
    """(token, distance of u from the nearest edge of the token's interval of the CDF)."""
    c = cdf(logits, temperature)
    u = uniform01(seed, index)
    token = int(np.searchsorted(c, u, side="right"))
    token = min(token, len(c) - 1)
    lower = c[token - 1] if token > 0 else 0.0
    return token, min(u - lower, c[token] - u)
