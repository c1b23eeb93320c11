"""The argmax entry point that allocates nothing (tqk_argmax_static), called through ctypes
as a caller without torch's wrappers would, against tqk_argmax with a scratch buffer of the
caller's: two calls in a row, the second with a smaller input, so that what the first call
left in the library's own array must not show."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from tq_kv_amd import kernels as K
    lib = K.library()
    lib.tqk_last_error.restype = ctypes.c_char_p
    return lib


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, logits):
    rows, vocab = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    scratch = torch.empty((lib.tqk_argmax_scratch_floats(rows, vocab),), dtype=torch.float32, device="cuda")
    assert lib.tqk_argmax(_ptr(logits), rows, vocab, _ptr(want), _ptr(scratch), stream) == 0, lib.tqk_last_error()
    got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    assert lib.tqk_argmax_static(_ptr(logits), rows, vocab, _ptr(got), stream) == 0, lib.tqk_last_error()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_argmax_static_equals_argmax_on_two_calls_in_a_row():
    lib = _lib()
    assert lib.tqk_argmax_static_prepare() == 0, lib.tqk_last_error()
    g = torch.Generator().manual_seed(5)
    big = torch.randn((9, 152064), generator=g).cuda()
    big[3, 151000] = 50.0                 # the best of a late chunk
    big[4, 17] = 50.0
    big[4, 90017] = 50.0                  # equal values: the lowest index wins
    got, want = _both(lib, big)
    assert torch.equal(got, want) and torch.equal(want.long(), big.cpu().argmax(dim=1))
    assert got[3] == 151000 and got[4] == 17
    # a smaller input right after: fewer rows, fewer chunks, the last chunk not full
    small = torch.randn((2, 5000), generator=g).cuda()
    small[1, 4999] = 40.0
    got, want = _both(lib, small)
    assert torch.equal(got, want) and torch.equal(want.long(), small.cpu().argmax(dim=1))
    assert got[1] == 4999


def test_argmax_static_refuses_what_its_array_cannot_hold():
    lib = _lib()
    most = lib.tqk_argmax_static_max_pairs()
    rows = most // 2 + 1                  # two chunks a row: one pair too many
    logits = torch.zeros((rows, 4097), device="cuda")
    out = torch.zeros((rows,), dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.tqk_argmax_static(_ptr(logits), rows, 4097, _ptr(out), stream) == -1
    assert b"scratch entries" in lib.tqk_last_error()
    assert lib.tqk_argmax_static(_ptr(logits), most // 2, 4097, _ptr(out), stream) == 0, lib.tqk_last_error()
    torch.cuda.synchronize()
    assert int(out[: most // 2].abs().sum()) == 0
