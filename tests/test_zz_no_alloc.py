"""ksq_w4a16_gemm_static_scratch (the entry point that allocates nothing: its split-K partial tiles and re-encoded
activations live in a device array inside the library) against ksq_w4a16_gemm with a caller's workspace: the two
must agree bit for bit, and both must meet the parity bar against the oracle, on calls in a row that share the one
scratch array, each smaller than the one before."""
import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import W4Case, W4Device, capi_dtype, torch_dtype

pytestmark = pytest.mark.gpu


def _both(gpu, case):
    import torch

    from ksanallm_amd import capi

    dev = W4Device(case, gpu)
    assert dev.workspace_bytes > 0, "the case must be one whose kernels use scratch"
    want = dev.gemm()
    out = torch.full((case.M, case.N), float("nan"), dtype=torch_dtype(case.dtype), device=gpu)
    capi.w4a16_gemm_static_scratch(capi_dtype(case.dtype), out, dev.act, dev.weight, dev.sz, case.M, case.N, case.K,
                                   case.g)
    torch.cuda.synchronize()
    return out, want


def test_static_scratch_matches_workspace_entry_point(gpu):
    import torch

    print("\n[case] static scratch: bf16 M=200 K=12288 N=528, then f16 M=40 K=2304 N=1040, then f16 M=16 K=8192 N=272",
          flush=True)
    cases = [
        W4Case(7001, 200, 12288, 528, kind="awq", dtype="bf16"),   # re-encoded activations + split-K partial tiles
        W4Case(7002, 40, 2304, 1040, kind="awq", dtype="f16"),     # smaller: split-K of the 17 <= M <= 64 kernel
        W4Case(7003, 16, 8192, 272, kind="gptq", dtype="f16"),     # smaller again: split-K of the M <= 16 kernel
    ]
    for case in cases:
        got, want = _both(gpu, case)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"M={case.M}: entry points differ"
        orc.assert_parity(got.float().cpu().numpy(), case.oracle(), f"static scratch M={case.M}")


def test_static_scratch_rejects_oversized_shapes(gpu):
    import torch

    from ksanallm_amd import capi

    m, k, n = 4096, 11008, 4096
    assert capi.w4a16_workspace_bytes(m, n, k) > capi.STATIC_SCRATCH_BYTES
    dummy = torch.zeros(4096, dtype=torch.uint8, device=gpu)
    with pytest.raises(capi.KsqError) as e:
        capi.w4a16_gemm_static_scratch(capi.BF16, dummy, dummy, dummy, dummy, m, n, k, 128)
    assert e.value.code == capi.ERR_WORKSPACE and "static scratch" in str(e.value)
