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
        if not use_ws and K % 128:
            continue  # the padded copy of the activation rows lives in the workspace
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


@pytest.mark.parametrize("source", ["cutlass80", "cutlass90", "marlin", "desc_act", "silu_mul", "bias"])
def test_w4a16_next_golden(gpu, source):
    """The widened entry points against the float64 vectors: weights as the other back ends leave them, a desc_act
    checkpoint, and the two epilogues."""
    import torch

    from ksanallm_amd import capi

    f = load("w4a16_next_f16_12x256x128")
    K, N = f["u"].shape
    M, g = f["act_bits"].shape[0], int(f["group"])
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)  # noqa: E731
    wb, sb = capi.w4a16_repack_sizes(K, N, g)
    weight = torch.empty(wb, dtype=torch.uint8, device=gpu)
    sz = torch.empty(sb // 4, dtype=torch.int32, device=gpu)
    scales = dev(f["scales_bits"].view(np.int16))
    lay, src, zk, zeros, perm, order = capi.W4_AWQ_INT32_NPACK, f["qweight_awq"], capi.ZERO_AWQ_INT32, f["qzeros_awq"], None, 0
    epi, bias, want, cols = capi.EPILOGUE_NONE, None, f["out"], N
    if source == "cutlass80":
        lay, src, zk, zeros = capi.W4_CUTLASS_SM80_INTERLEAVED, f["cutlass80"], capi.ZERO_UINT8, f["z"]
    elif source == "cutlass90":
        lay, src, zk, zeros = capi.W4_CUTLASS_SM90_COLMAJOR, f["cutlass90"], capi.ZERO_UINT8, f["z"]
    elif source == "marlin":
        lay, src, zk, zeros = capi.W4_MARLIN, f["marlin"], capi.ZERO_MARLIN_INT32, f["marlin_zp"]
        scales = dev(f["marlin_scales_bits"].view(np.int16))
    elif source == "desc_act":
        lay, src, zk, zeros, perm, want = capi.W4_GPTQ_INT32_KPACK, f["qweight_gptq"], capi.ZERO_NONE, None, dev(f["perm"]), f["out_desc"]
    elif source == "silu_mul":
        order, epi, want, cols = capi.COLS_HALVES_INTERLEAVED, capi.EPILOGUE_SILU_MUL, f["out_silu"], N // 2
    elif source == "bias":
        epi, bias, want = capi.EPILOGUE_BIAS, dev(f["bias_bits"].view(np.int16)), f["out_bias"]
    capi.w4a16_repack_ex(lay, dev(src), zk, None if zeros is None else dev(zeros), scales, capi.F16, K, N, g, perm, order,
                         weight, sz)
    act = dev(f["act_bits"].view(np.int16)).view(torch.float16)
    wsb = capi.w4a16_workspace_bytes_ex(M, N, K, perm is not None)
    ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device=gpu)
    out = torch.full((M, cols), float("nan"), dtype=torch.float16, device=gpu)
    capi.w4a16_gemm_ex(capi.F16, out, act, weight, sz, M, N, K, g, perm, epi, bias, ws, wsb)
    torch.cuda.synchronize()
    orc.assert_parity(out.float().cpu().numpy(), want, f"next golden {source}")
