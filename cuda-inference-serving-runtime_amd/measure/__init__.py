"""Measurements of the machine and of single kernels, apart from the engine: the kernels of `csrc/measure.hip`
(a shared object of its own that no step ever loads) and, as `python -m runtime.measure <workload>`, the sweeps
that settled the launch rules of `kernels/attention.py`.  The benchmark of the engine itself is `bench.py`."""
import ctypes as C

import torch

from ..kernels import library
from ..kernels.ops import KernelError, _check, _dev, _stream

_handle = None


def _lib():
    global _handle
    if _handle is None:
        h = library.load(library.MEASURE)
        p, i, ll = C.c_void_p, C.c_int, C.c_longlong
        for name, args in {"cisr_idle": [i, p], "cisr_stream_read": [p, ll, p, i, p],
                           "cisr_grid_meet": [p, p, i, i, i, C.c_uint, p]}.items():
            fn = getattr(h, name)
            fn.argtypes, fn.restype = args, C.c_int
        _handle = h
    return _handle


def idle(blocks=1):
    """Launches a kernel of `blocks` blocks that does nothing (the cost of a launch)."""
    _check(_lib().cisr_idle(int(blocks), _stream()), "idle")


def stream_read(buffer, sink, blocks=512):
    """Reads every byte of `buffer` once and keeps nothing (the read bandwidth of the memory).
    `sink`: a GPU tensor of at least 4 bytes."""
    nbytes = buffer.numel() * buffer.element_size()
    if not buffer.is_contiguous() or nbytes % 16 or buffer.data_ptr() % 16:
        raise KernelError("stream_read: a contiguous buffer of a multiple of 16 bytes, 16-byte aligned")
    _check(_lib().cisr_stream_read(buffer.data_ptr(), nbytes, _dev(sink, "sink"), int(blocks), _stream()), "stream_read")


def grid_meet(blocks, rounds, exchange=0, spin_limit=1 << 22):
    """One kernel of `blocks` blocks (a multiple of 32, at most 512, all resident at once) that all meet `rounds`
    times, passing `exchange` floats through memory at each meeting (what a barrier over the whole grid costs beside
    a launch).  Returns the words it counted in: [0] the number of groups of 32 blocks that arrived, over all rounds,
    [-1] is set when a block gave up waiting after `spin_limit` polls."""
    if blocks <= 0 or blocks % 32 or blocks > 512 or rounds * blocks >= 1 << 31 or exchange < 0:
        raise KernelError(f"grid_meet: {blocks} blocks must be a multiple of 32, at most 512, and {rounds} rounds few enough to count")
    device = torch.device("cuda", torch.cuda.current_device())
    words = torch.zeros(1024, dtype=torch.int32, device=device)
    passed = torch.empty(max(2 * exchange, 1), dtype=torch.float32, device=device)
    _check(_lib().cisr_grid_meet(words.data_ptr(), passed.data_ptr(), int(exchange), int(blocks), int(rounds), int(spin_limit),
                                 _stream()), "grid_meet")
    return words
