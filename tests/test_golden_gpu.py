"""The HIP path, through the C ABI, against the committed golden vectors of tests/golden (float64 truth from an
independent numpy statement of the formats): layouts and FP8 quantisation bit-exact, GEMMs to the parity bar
(max relative error <= 1e-2 with the denominator floored at the RMS of the truth, mean absolute error <= 2e-3 RMS)."""
import os

import numpy as np
import pytest

from oracle import oracle as orc
from tests.test_golden import W4_CASES, load

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


@pytest.mark.parametrize("name", W4_CASES)
def test_w4a16_golden(gpu, name):
    import torch

    from ksanallm_amd import capi

    f = load(name)
    bf16 = bool(int(f["bf16"]))
    cdt, tdt = (capi.BF16, torch.bfloat16) if bf16 else (capi.F16, torch.float16)
    g = int(f["group"])
    K, N = f["u"].shape
    M = f["act_bits"].shape[0]
    qweight = torch.from_numpy(f["qweight"]).to(gpu)
    scales = torch.from_numpy(f["scales_bits"].view(np.int16)).to(gpu)
    wb, sb = capi.w4a16_repack_sizes(K, N, g)
    weight = torch.empty(wb, dtype=torch.uint8, device=gpu)
    sz = torch.empty(sb // 4, dtype=torch.int32, device=gpu)
    if "qzeros" in f.files:
        qzeros = torch.from_numpy(f["qzeros"]).to(gpu)
        capi.w4a16_repack(capi.W4_AWQ_INT32_NPACK, qweight, capi.ZERO_AWQ_INT32, qzeros, scales, cdt, K, N, g, weight, sz)
    else:
        capi.w4a16_repack(capi.W4_GPTQ_INT32_KPACK, qweight, capi.ZERO_NONE, None, scales, cdt, K, N, g, weight, sz)
    act = torch.from_numpy(f["act_bits"].view(np.int16)).to(gpu).view(tdt)
    wsb = capi.w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=gpu)
    for use_ws in (True, False):
        out = torch.full((M, N), float("nan"), dtype=tdt, device=gpu)
        capi.w4a16_gemm(cdt, out, act, weight, sz, M, N, K, g, ws if use_ws else None, wsb if use_ws else 0)
        torch.cuda.synchronize()
        orc.assert_parity(out.float().cpu().numpy(), f["out"], f"{name} workspace={use_ws}")


def test_fp8_golden(gpu):
    import torch

    from ksanallm_amd import capi

    f = load("fp8_8x256x64")
    M, K = f["x_bits"].shape
    N = f["wq"].shape[0]
    x = torch.from_numpy(f["x_bits"].view(np.int16)).to(gpu).view(torch.float16)
    aq = torch.zeros((M, K), dtype=torch.uint8, device=gpu)
    a_scale = torch.zeros(M, dtype=torch.float32, device=gpu)
    capi.fp8_quantize(capi.F16, x, M, K, capi.FP8_PER_TOKEN_DYNAMIC, aq, a_scale)
    torch.cuda.synchronize()
    assert np.array_equal(a_scale.cpu().numpy(), f["a_scale"])
    got_q, want_q = aq.cpu().numpy(), f["aq"]
    nz = (want_q & 0x7F) != 0
    assert np.array_equal(got_q[nz], want_q[nz]) and np.all((got_q[~nz] & 0x7F) == 0)
    wq = torch.from_numpy(f["wq"]).to(gpu)
    w_scale = torch.from_numpy(f["w_scale"]).to(gpu)
    wsb = capi.fp8_workspace_bytes(M, N, K)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=gpu)
    for odt, tdt in ((capi.F16, torch.float16), (capi.BF16, torch.bfloat16)):
        out = torch.full((M, N), float("nan"), dtype=tdt, device=gpu)
        capi.fp8_gemm(odt, out, aq, a_scale, M, wq, w_scale, N, M, N, K, ws, wsb)
        torch.cuda.synchronize()
        orc.assert_parity(out.float().cpu().numpy(), f["out"], "fp8 golden")
