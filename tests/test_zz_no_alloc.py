"""The entry point that allocates nothing (fmsa_lora_grad_static: partial sums in a buffer inside the
library's device image) against fmsa_lora_grad with a caller-provided workspace: same kernels, same order
of the sums, so the results must be bit-identical -- also on a second call with a smaller input, which
re-uses the buffer with the first call's partial sums still in it."""
import ctypes

import pytest
import torch

from tests.helpers import randn

pytestmark = pytest.mark.gpu


def _both(M, C, r, transpose_out, out_dtype, dtype, seed, check_allocations=False):
    import fmsa_hip

    L = randn((M, r), seed, dtype).cuda()
    R = randn((M, C), seed + 1, dtype).cuda()
    ref = fmsa_hip.lora_grad(L, R, 0.5, transpose_out, out_dtype)
    out = torch.full_like(ref, float("nan"))
    # straight through the C ABI: the caller owns inputs and output, the library brings its own scratch
    lib = fmsa_hip.lib()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    allocs_before = torch.cuda.memory_stats()["allocation.all.allocated"]
    rc = lib.fmsa_lora_grad_static(ctypes.c_void_p(L.data_ptr()), L.stride(0), ctypes.c_void_p(R.data_ptr()), R.stride(0), M, C, r,
                                   ctypes.c_float(0.5), int(transpose_out), fmsa_hip.act_enum(dtype),
                                   {torch.float32: fmsa_hip.F32, torch.bfloat16: fmsa_hip.BF16, torch.float16: fmsa_hip.F16}[out_dtype],
                                   ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, fmsa_hip.lib().fmsa_strerror(rc)
    torch.cuda.synchronize()
    if check_allocations:
        # what the entry point exists for: neither the device's free memory (driver-level allocations: hipMalloc, module
        # loads) nor torch's allocation count moves across the call, and a second query agrees
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == allocs_before
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.mem_get_info()[0] == free_before
    return out, ref


def test_static_scratch_matches_workspace_entry_point_twice():
    # first call: the largest shape of the benchmark layer (8192 tokens x 14336 columns, rank 16: 8.3 MB of partial sums)
    out, ref = _both(8192, 14336, 16, False, torch.float32, torch.bfloat16, 1)
    assert torch.equal(out, ref)
    # second call, smaller and ragged (fewer splits, fewer columns, other rank): stale partial sums must not leak in
    # (from here on the code object is loaded and the buffer's address known: the calls must not allocate)
    out, ref = _both(1000, 1024 + 32, 8, True, torch.bfloat16, torch.bfloat16, 3, check_allocations=True)
    assert torch.equal(out, ref)
    out, ref = _both(4096, 4096, 64, True, torch.float32, torch.float16, 5, check_allocations=True)
    assert torch.equal(out, ref)


def test_static_scratch_rejects_requests_beyond_its_size():
    import fmsa_hip

    M, C, r = 8192, 14336, 64  # 4 x the 16 MiB of the first case above
    assert fmsa_hip.lib().fmsa_lora_grad_workspace(M, C, r) > fmsa_hip.LORA_GRAD_STATIC_BYTES
    L = torch.zeros((M, r), dtype=torch.bfloat16, device="cuda")
    R = torch.zeros((M, C), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((r, C), dtype=torch.float32, device="cuda")
    with pytest.raises(fmsa_hip.FmsaError, match="workspace"):
        fmsa_hip.lora_grad_static(L, R, 1.0, False, out)
