"""The entry point that allocates nothing (``tq_sample_topp_static``, csrc/no_alloc.h), called through ctypes and
compared with ``tq_sample_topp``, whose caller brings the scratch memory: two calls in a row, the second with a
smaller input, so that what the first call left in the library's array would show if anything depended on it."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_sampling_without_allocation_equals_sampling_with_brought_scratch():
    from turboquant_cpp_amd.csrc import build, ops
    ops.library("bfloat16")                                   # builds the library if it is not there
    lib = ctypes.CDLL(build.find_library("bfloat16"))
    fn = lib.tq_sample_topp_static
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_void_p,
                   ctypes.c_void_p, ctypes.c_void_p]
    lib.tq_sample_topp_static_init.restype = ctypes.c_int
    dev = "cuda:0"
    torch.cuda.set_device(0)
    assert lib.tq_sample_topp_static_init() == 0
    g = torch.Generator().manual_seed(11)
    stream = torch.cuda.current_stream().cuda_stream
    for R, V, temperature, top_p in ((13, 151936, 0.7, 0.9), (5, 1001, 1.3, 0.5), (64, 32000, 0.7, 0.9), (1, 7, 0.2, 1.0)):
        logits = (3.0 * torch.randn((R, V), generator=g)).to(dev)
        uniforms = torch.rand((R,), generator=g).to(dev)
        want = ops.sample_topp(logits, temperature, top_p, uniforms, "bfloat16")
        out = torch.full((R,), -1, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        rc = fn(logits.data_ptr(), R, V, temperature, top_p, uniforms.data_ptr(), out.data_ptr(), stream)
        torch.cuda.synchronize()
        assert rc == 0
        assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the amount of free device memory"
        assert torch.equal(out, want), (R, V)
        assert 0 <= int(out.min()) and int(out.max()) < V
    # beyond the stated maximum: refused, nothing launched, out untouched
    out = torch.full((65,), -1, dtype=torch.int32, device=dev)
    small = torch.zeros((65, 8), device=dev)
    assert fn(small.data_ptr(), 65, 8, 0.7, 0.9, small.data_ptr(), out.data_ptr(), stream) == -2
    assert fn(small.data_ptr(), 14, 151936, 0.7, 0.9, small.data_ptr(), out.data_ptr(), stream) == -2      # R * V > 2^21
    assert fn(small.data_ptr(), 2, 8, 0.0, 0.9, small.data_ptr(), out.data_ptr(), stream) == -1
    torch.cuda.synchronize()
    assert bool((out == -1).all())
