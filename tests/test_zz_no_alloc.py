"""hb_argmax_noalloc, the entry point that allocates nothing, through ctypes: the same indices
as hb_argmax with a workspace, on two calls in a row of which the second is smaller (it reads
nothing that the first left in the library's scratch), and a clear refusal beyond the scratch."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_argmax_without_allocation_gives_what_argmax_gives():
    from herbert_rs_amd.kernels import lib, ops
    so = lib.load("sampling")
    fn = so.hb_argmax_noalloc
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    fn.restype = ctypes.c_int
    so.hb_argmax_noalloc_setup.argtypes = []
    so.hb_argmax_noalloc_setup.restype = ctypes.c_int
    assert so.hb_argmax_noalloc_setup() == 0, so.hb_last_error()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator().manual_seed(77)
    for R, V in ((64, 151936), (3, 40000), (5, 9000)):        # the second and third are smaller
        logits = torch.randn(R, V, generator=gen)
        logits[0, V - 1] = 30.0                                # the last stretch's last value
        logits[1, 17] = logits[1, V // 2 + 5] = 31.0           # equal maxima in different stretches: the first wins
        logits[2] = -float("inf")                              # nothing above -inf: index 0
        dev = logits.cuda()
        want = torch.full((R,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((R,), -2, dtype=torch.int32, device="cuda")
        ops.argmax(dev, want)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        rc = fn(dev.data_ptr(), V, R, V, got.data_ptr(), stream)
        assert rc == 0, so.hb_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert got.tolist() == want.tolist()
        assert got.tolist()[:3] == [V - 1, 17, 0]
        assert got.tolist()[3:] == logits[3:].argmax(-1).tolist()
    # more partial results than the library's scratch holds: refused, nothing launched
    R, V = 300, 151936
    dev = torch.zeros(R, V, device="cuda")
    got = torch.full((R,), -2, dtype=torch.int32, device="cuda")
    rc = fn(dev.data_ptr(), V, R, V, got.data_ptr(), stream)
    torch.cuda.synchronize()
    assert rc != 0 and b"scratch holds 4096" in so.hb_last_error()
    assert got.tolist() == [-2] * R
    assert fn(dev.data_ptr(), V, 0, V, got.data_ptr(), stream) != 0      # bad sizes are refused too
