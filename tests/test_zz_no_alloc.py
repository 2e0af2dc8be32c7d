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
    lib.tp_argmax_no_alloc_prepare.argtypes = []
    lib.tp_argmax_no_alloc_prepare.restype = I
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


def test_no_alloc_argmax_inside_a_captured_graph():
    """What the header names as a caller: after tp_argmax_no_alloc_prepare() (outside the capture) two calls, a large one
    and then a smaller one, are captured into one HIP graph; every replay, with other work and synchronisations of the
    program between the replays and new logits each time, gives what tp_argmax gives."""
    lib = _lib()
    dev = torch.device("cuda:0")
    assert lib.tp_argmax_no_alloc_prepare() == 0, lib.tp_last_error()
    shapes = ((8, 256000), (3, 50021))
    z = [torch.zeros(s, device=dev) for s in shapes]
    got = [torch.full((s[0],), -1, dtype=torch.int32, device=dev) for s in shapes]
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            st = torch.cuda.current_stream(dev).cuda_stream
            for t, o in zip(z, got):
                assert lib.tp_argmax_no_alloc(t.data_ptr(), t.shape[0], t.shape[1], o.data_ptr(), st) == 0, lib.tp_last_error()
    torch.cuda.current_stream(dev).wait_stream(side)
    g = torch.Generator().manual_seed(12)
    stream = torch.cuda.current_stream(dev).cuda_stream
    for replay in range(4):
        for t in z:
            t.copy_(torch.randn(t.shape, generator=g))
            t[1, (replay * 7919) % t.shape[1]] = 9.0
        graph.replay()
        torch.cuda.synchronize(dev)
        for t, o in zip(z, got):
            want = torch.empty(t.shape[0], dtype=torch.int32, device=dev)
            ws = torch.empty(lib.tp_argmax_workspace_bytes(*t.shape), dtype=torch.uint8, device=dev)
            assert lib.tp_argmax(t.data_ptr(), t.shape[0], t.shape[1], want.data_ptr(), ws.data_ptr(), stream) == 0
            torch.cuda.synchronize(dev)
            assert o.tolist() == want.tolist(), replay
            assert o.tolist()[1] == (replay * 7919) % t.shape[1]
            o.fill_(-1)
