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
    """pick(logits, params) -> list of token ids.  params: one (temperature, seed, counter) per row.

    With `out` and `index` (int32 on the device) the token of row r is left at out[index[r]] on the
    device instead, nothing is returned and the host does not wait: the next step can take its tokens
    from there while the host reads them later."""

    def __init__(self):
        self._staging = {}    # device -> [pinned int64 host buffers, device buffer, events, next]
        self._scratch = ops.ScratchPool()   # the argmax kernel's slice winners

    def _params(self, params, device):
        """(temperature, seeds, counters) on the device, through pinned memory so the host does not wait."""
        rows = len(params)
        entry = self._staging.get(device)
        if entry is None or entry[1][0].numel() < 5 * rows:
            cap = max(320, 5 << (rows - 1).bit_length())
            entry = self._staging[device] = [[torch.empty(cap, dtype=torch.int32, pin_memory=True) for _ in range(4)],
                                             [torch.empty(cap, dtype=torch.int32, device=device) for _ in range(4)],
                                             [None] * 4, 0]
        slot = entry[3] % 4
        entry[3] += 1
        if entry[2][slot] is not None:
            entry[2][slot].synchronize()      # the copy that last read this buffer is over
        host, dev = entry[0][slot], entry[1][slot]
        # seeds and counters as int64 (two int32 each), then the temperatures as float
        host[:2 * rows].view(torch.int64)[:] = torch.tensor([_as_i64(int(p[1])) for p in params], dtype=torch.int64)
        host[2 * rows:4 * rows].view(torch.int64)[:] = torch.tensor([_as_i64(int(p[2])) for p in params], dtype=torch.int64)
        host[4 * rows:5 * rows].view(torch.float32)[:] = torch.tensor([float(p[0]) for p in params], dtype=torch.float32)
        dev[:5 * rows].copy_(host[:5 * rows], non_blocking=True)
        entry[2][slot] = torch.cuda.Event()
        entry[2][slot].record()
        return (dev[4 * rows:5 * rows].view(torch.float32), dev[:2 * rows].view(torch.int64),
                dev[2 * rows:4 * rows].view(torch.int64))

    def pick(self, logits, params, out=None, index=None):
        rows = logits.shape[0]
        if (out is None) != (index is None):
            raise ValueError("out and index come together")
        if rows == 0:
            return [] if out is None else None
        if len(params) != rows:
            raise ValueError("one (temperature, seed, counter) per row of logits is required")
        keep = out is not None
        if not keep:
            out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        if all(not (p[0] > 0) for p in params):
            ops.argmax(logits, out, index, scratch=self._scratch)
        else:
            temperature, seeds, counters = self._params(params, logits.device)
            ops.sample(logits, temperature, seeds, counters, out, index)
        return None if keep else out.cpu().tolist()
