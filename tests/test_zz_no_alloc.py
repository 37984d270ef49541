"""The greedy pick that allocates nothing (cisr_argmax_noalloc), called through ctypes as a caller
without an allocator would, against the entry point that takes its buffers from the caller
(cisr_argmax): two calls in a row, the second with a smaller input, so that what the first call
left in the library's fixed array must not show."""
import ctypes as C

import pytest

pytestmark = pytest.mark.gpu


def _library():
    from runtime.kernels import library
    h = library.load()
    p, i = C.c_void_p, C.c_int
    h.cisr_argmax_noalloc.argtypes = [p, p, i, i, p]
    h.cisr_argmax_noalloc.restype = i
    h.cisr_argmax.argtypes = [p, p, p, i, p, p, i, i, p]
    h.cisr_argmax.restype = i
    h.cisr_noalloc_init.argtypes = []
    h.cisr_noalloc_init.restype = i
    h.cisr_argmax_noalloc_max_rows.argtypes = []
    h.cisr_argmax_noalloc_max_rows.restype = i
    return h


def test_argmax_without_allocation_matches_the_one_with_buffers():
    import torch
    h = _library()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    assert h.cisr_noalloc_init() == 0
    limit = h.cisr_argmax_noalloc_max_rows()
    assert limit == 1024
    stream = torch.cuda.current_stream().cuda_stream
    generator = torch.Generator(device="cpu").manual_seed(11)
    for rows, vocab in ((37, 49152), (5, 1003)):          # the second call is smaller: stale slice winners must not show
        logits = torch.randn(rows, vocab, generator=generator).to(device)
        logits[0, 7] = logits[0, vocab - 3] = 9.0         # a tie: the lowest index wins
        logits[rows - 1, vocab - 1] = 11.0                # the last place of the last slice
        got = torch.full((rows,), -1, dtype=torch.int32, device=device)
        want = torch.full((rows,), -1, dtype=torch.int32, device=device)
        val = torch.empty(rows * 32, dtype=torch.float32, device=device)
        idx = torch.empty(rows * 32, dtype=torch.int32, device=device)
        # everything is allocated before the call under test; from here on only the two entry points run
        assert h.cisr_argmax_noalloc(logits.data_ptr(), got.data_ptr(), rows, vocab, stream) == 0
        assert h.cisr_argmax(logits.data_ptr(), want.data_ptr(), None, rows, val.data_ptr(), idx.data_ptr(), rows, vocab, stream) == 0
        torch.cuda.synchronize()
        assert got.tolist() == want.tolist()
        assert got.tolist() == logits.argmax(dim=-1).tolist()
        assert got[0].item() == 7 and got[rows - 1].item() == vocab - 1
    # sizes beyond the fixed array are refused before anything is launched
    out = torch.full((4,), -5, dtype=torch.int32, device=device)
    big = torch.zeros(4, 8, device=device)
    assert h.cisr_argmax_noalloc(big.data_ptr(), out.data_ptr(), limit + 1, 8, stream) != 0
    assert h.cisr_argmax_noalloc(big.data_ptr(), out.data_ptr(), 4, 0, stream) != 0
    assert h.cisr_argmax_noalloc(None, out.data_ptr(), 4, 8, stream) != 0
    torch.cuda.synchronize()
    assert out.tolist() == [-5] * 4
    assert h.cisr_argmax_noalloc(big.data_ptr(), out.data_ptr(), 0, 8, stream) == 0      # no rows: nothing to do
