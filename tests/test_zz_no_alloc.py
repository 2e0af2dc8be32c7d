"""The entry point that allocates nothing (tp_argmax_no_alloc), called through ctypes as a caller outside Python
would: its output against tp_argmax's on two calls in a row, the second with a smaller input, so that what the
first call left in the library's fixed scratch array must not show."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from trapetum_amd.kernels import build
    lib = ctypes.CDLL(build.build_core())
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.tp_last_error.restype = ctypes.c_char_p
    lib.tp_argmax_no_alloc.argtypes = [P, I, I, P, P]
    lib.tp_argmax_no_alloc.restype = I
    lib.tp_argmax.argtypes = [P, I, I, P, P, P]
    lib.tp_argmax.restype = I
    lib.tp_argmax_workspace_bytes.argtypes = [I, I]
    lib.tp_argmax_workspace_bytes.restype = ctypes.c_long
    return lib


def test_no_alloc_argmax_equals_argmax_twice_in_a_row():
    lib = _lib()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream(dev).cuda_stream
    g = torch.Generator().manual_seed(11)
    for rows, vocab in ((8, 256000), (3, 50021)):          # the second call is smaller: stale winners lie beyond it
        z = torch.randn((rows, vocab), generator=g).to(dev)
        z[1, vocab - 1] = 9.0                                # the last part holds a row's winner
        z[2, 77] = z[2, vocab // 2] = 8.0                   # a tie: the smaller index wins
        want = torch.empty(rows, dtype=torch.int32, device=dev)
        ws = torch.empty(lib.tp_argmax_workspace_bytes(rows, vocab), dtype=torch.uint8, device=dev)
        assert lib.tp_argmax(z.data_ptr(), rows, vocab, want.data_ptr(), ws.data_ptr(), stream) == 0, lib.tp_last_error()
        got = torch.full((rows,), -1, dtype=torch.int32, device=dev)
        assert lib.tp_argmax_no_alloc(z.data_ptr(), rows, vocab, got.data_ptr(), stream) == 0, lib.tp_last_error()
        torch.cuda.synchronize(dev)
        assert got.tolist() == want.tolist()
        assert got.tolist() == z.cpu().argmax(dim=-1).tolist()[:2] + [77] + z.cpu().argmax(dim=-1).tolist()[3:]


def test_no_alloc_argmax_refuses_what_the_scratch_cannot_hold():
    lib = _lib()
    dev = torch.device("cuda:0")
    z = torch.zeros((257, 8), device=dev)
    out = torch.zeros(257, dtype=torch.int32, device=dev)
    assert lib.tp_argmax_no_alloc(z.data_ptr(), 257, 8, out.data_ptr(), None) != 0
    assert b"256" in lib.tp_last_error()
    assert lib.tp_argmax_no_alloc(z.data_ptr(), 0, 8, out.data_ptr(), None) != 0
