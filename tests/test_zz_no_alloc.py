"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes: two calls in a
row on one GPU, the second with a smaller input, each against the entry point with a workspace;
sizes beyond its fixed array are refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_sampling_without_allocation_matches_the_entry_point_with_a_workspace():
    from tests import backends
    if backends.ACTIVE.name != "hip":
        pytest.skip("the device array and its address are what this test is about: GPU only")
    from sparseengine_amd.kernels import library
    from sparseengine_amd.kernels.hip_ops import HipKernels
    lib = library.load("sampling")
    fn = lib.se_sample_unfiltered_no_alloc
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                   ctypes.c_void_p, ctypes.c_void_p]
    hip = HipKernels()
    g = torch.Generator().manual_seed(3)
    stream = torch.cuda.current_stream().cuda_stream
    for rows, vocab in ((13, 20011), (5, 4097)):          # the second call is smaller: stale slots must not matter
        logits = (torch.randn(rows, vocab, generator=g) * 2).cuda()
        temperature = torch.tensor([0.0, 0.7, 1.0, 1.5, 0.3] * 3)[:rows].contiguous().cuda()
        seeds = (torch.arange(rows, dtype=torch.int64) * 7919 + 1).cuda()
        expected = torch.empty(rows, dtype=torch.int32, device="cuda")
        hip.sample(logits, temperature, None, None, seeds, expected)
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        status = fn(logits.data_ptr(), logits.stride(0), rows, vocab, temperature.data_ptr(), seeds.data_ptr(),
                    got.data_ptr(), stream)
        assert status == 0
        torch.cuda.synchronize()
        assert torch.equal(got, expected)
        # "allocates nothing": the device's own count of free bytes (which sees every hipMalloc, not only the
        # tensor library's) and the tensor library's count are the same before and after a further call; the
        # call above has asked for the array's address already, so this one is a call like every later one
        got.fill_(-1)
        torch.cuda.synchronize()
        free_before, allocations_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_stats()["allocation.all.allocated"]
        status = fn(logits.data_ptr(), logits.stride(0), rows, vocab, temperature.data_ptr(), seeds.data_ptr(),
                    got.data_ptr(), stream)
        assert status == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == allocations_before
        assert torch.equal(got, expected)
        assert int(got[0]) == int(logits[0].argmax())
        # greedy, no temperature and no seeds
        status = fn(logits.data_ptr(), logits.stride(0), rows, vocab, None, None, got.data_ptr(), stream)
        assert status == 0
        torch.cuda.synchronize()
        assert torch.equal(got.long(), logits.argmax(-1))
    # beyond the fixed array: refused, nothing launched
    wide = torch.zeros(70, 262144, device="cuda")
    out = torch.full((70,), -5, dtype=torch.int32, device="cuda")
    assert fn(wide.data_ptr(), wide.stride(0), 70, 262144, None, None, out.data_ptr(), stream) == -1
    torch.cuda.synchronize()
    assert bool((out == -5).all())
