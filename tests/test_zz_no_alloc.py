"""hapmi_sumsq_static: the entry point that allocates nothing (its partial sums live in a device array inside the
library), called through the C ABI and compared bit for bit with hapmi_sumsq, whose partial sums go to a workspace
of the caller, on two calls in a row, the second with a smaller input; plus its size limit, the empty input, and the
call recorded into a HIP graph (the use it exists for) and replayed on changing inputs."""
import ctypes
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    lib = ctypes.CDLL(os.path.join(ROOT, "hap_amd", "libhapmi.so"))
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    lib.hapmi_sumsq.argtypes = [vp, i64, vp, vp, i64, vp]
    lib.hapmi_sumsq_static.argtypes = [vp, i64, vp, vp]
    lib.hapmi_sumsq_workspace_elems.argtypes = [i64, ctypes.POINTER(i64)]
    lib.hapmi_last_error.restype = ctypes.c_char_p
    assert lib.hapmi_init() == 0, lib.hapmi_last_error()
    return lib


def test_sumsq_static_equals_sumsq_with_a_workspace(cuda):
    lib = _lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator().manual_seed(5)
    for n in (3_000_017, 70_001):                          # the second, smaller call finds the first call's partial sums in the array
        g = (torch.randn(n, generator=gen) * 3).to(cuda)
        need = ctypes.c_int64()
        assert lib.hapmi_sumsq_workspace_elems(n, ctypes.byref(need)) == 0
        ws = torch.full((need.value,), float("nan"), device=cuda)
        want = torch.full((1,), -1.0, device=cuda)
        got = torch.full((1,), -2.0, device=cuda)
        assert lib.hapmi_sumsq(g.data_ptr(), n, want.data_ptr(), ws.data_ptr(), ws.numel(), stream) == 0, lib.hapmi_last_error()
        allocated = torch.cuda.memory_allocated()
        assert lib.hapmi_sumsq_static(g.data_ptr(), n, got.data_ptr(), stream) == 0, lib.hapmi_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == allocated
        assert torch.equal(got, want), (n, got.item(), want.item())
        ref = g.double().pow(2).sum().item()
        assert abs(got.item() - ref) <= 1e-6 * ref
    # empty input: the result is 0
    got = torch.full((1,), 5.0, device=cuda)
    assert lib.hapmi_sumsq_static(None, 0, got.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert got.item() == 0.0
    # beyond the built-in scratch (2^30 elements): refused before anything is read or launched
    assert lib.hapmi_sumsq_static(g.data_ptr(), (1 << 30) + 1, got.data_ptr(), stream) == -5
    assert b"exceed the built-in scratch" in lib.hapmi_last_error()
    torch.cuda.synchronize()
    assert got.item() == 0.0


def test_sumsq_static_under_stream_capture(cuda):
    """The call only enqueues kernels (the scratch address was looked up by hapmi_init), so it can be recorded into a
    HIP graph; every replay, with the program's own eager work and synchronisations between the replays, gives the
    bits of an eager hapmi_sumsq on the same input."""
    lib = _lib()
    gen = torch.Generator().manual_seed(9)
    n = 1_000_003
    g = torch.zeros(n, device=cuda)
    got = torch.full((1,), -2.0, device=cuda)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                          # one eager call on the capture stream first
        assert lib.hapmi_sumsq_static(g.data_ptr(), n, got.data_ptr(), ctypes.c_void_p(side.cuda_stream)) == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.hapmi_sumsq_static(g.data_ptr(), n, got.data_ptr(), st) == 0, lib.hapmi_last_error()
    need = ctypes.c_int64()
    assert lib.hapmi_sumsq_workspace_elems(n, ctypes.byref(need)) == 0
    ws = torch.empty(need.value, device=cuda)
    want = torch.empty(1, device=cuda)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for rep in range(4):
        g.copy_((torch.randn(n, generator=gen) * (rep + 1)).to(cuda))
        got.fill_(-2.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert lib.hapmi_sumsq(g.data_ptr(), n, want.data_ptr(), ws.data_ptr(), ws.numel(), stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), (rep, got.item(), want.item())
