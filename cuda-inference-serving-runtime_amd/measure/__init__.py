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
                           "cisr_grid_meet": [p, p, i, i, i, C.c_uint, p],
                           "cisr_chain_phase": [p, p, p, i, i, p, C.c_uint, p, p, i, p],
                           "cisr_one_launch_step": [p, i, i, i, i, p, ll, p, p, i, i, C.c_uint, p]}.items():
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


def chain_phase(w, x, y, counters=None, wait=False):
    """y = squash(w . x): one link of a chain of dependent matrix-vector products, the leanest kernel a decode step of
    one request could be made of.  w bf16 [N, K] (N a multiple of 4, K 512 or 1536), x float [K], y float [N].
    `wait`: the kernel polls counters[0] until counters[1] blocks have arrived before it reads x (straight from
    memory), and every block bumps counters[2] after its store; counters = (int32 word in, expected, int32 word out or
    None, int32 error word)."""
    n, k = w.shape
    if w.dtype != torch.bfloat16 or x.dtype != torch.float32 or y.dtype != torch.float32 or x.numel() < k or y.numel() < n:
        raise KernelError("chain_phase: bf16 weights [N, K], float vectors of K and N elements")
    cin, expect, cout, err = counters if counters is not None else (None, 0, None, None)
    _check(_lib().cisr_chain_phase(_dev(w, "w"), x.data_ptr(), y.data_ptr(), n, k, None if cin is None else cin.data_ptr(), int(expect),
                                   None if cout is None else cout.data_ptr(), None if err is None else err.data_ptr(), int(bool(wait)),
                                   _stream()), "chain_phase")


def one_launch_step(weights, layers, hidden, qkv, intermediate, kv, kv_words, scratch, words, blocks=32, active=8, spin_limit=200000):
    """A mock decode step as ONE launch: the blocks of each die (XCD) meet inside the kernel through that die's L2, the
    first `active` dies each run the step of a request of their own (30 x five matrix-vector passes with the traffic
    of the real ones).  weights: bf16, layers x ((qkv + hidden + 2 intermediate) hidden + hidden intermediate)
    elements; kv: 8 x layers x kv_words 16-byte words; scratch: 8 x 16384 floats; words: 1024 int32, zeroed before
    every launch ([1023] is set when a block gave up waiting)."""
    need = layers * ((qkv + hidden + 2 * intermediate) * hidden + hidden * intermediate)
    if weights.dtype != torch.bfloat16 or weights.numel() < need or kv.numel() * kv.element_size() < 8 * layers * kv_words * 16:
        raise KernelError("one_launch_step: weights or keys and values too small for the sizes")
    if scratch.dtype != torch.float32 or scratch.numel() < 8 * 16384 or words.dtype != torch.int32 or words.numel() < 1024:
        raise KernelError("one_launch_step: scratch of 8 x 16384 floats and 1024 int32 words")
    _check(_lib().cisr_one_launch_step(_dev(weights, "weights"), int(layers), int(hidden), int(qkv), int(intermediate), _dev(kv, "kv"),
                                       int(kv_words), scratch.data_ptr(), words.data_ptr(), int(blocks), int(active), int(spin_limit),
                                       _stream()), "one_launch_step")
