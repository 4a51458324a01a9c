"""GPU parity tests of what widens the path on either side of the GEMM: already-preprocessed weight layouts and
desc_act checkpoints on the load side, bias and SiLU-mul epilogues on the store side.  Everything goes through the
C ABI; the oracle (fp32 dequantize-then-GEMM, then the epilogue in double precision) is the checker.  Tolerance: the
parity bar of the plain GEMM (max relative error 1e-2 with the denominator floored at the RMS, mean absolute error
<= 2e-3 x RMS)."""
import os

import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import ORC_DT, W4Case, W4Device, capi_dtype, torch_dtype

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


class _env:
    def __init__(self, **kv):
        self.kv = kv

    def __enter__(self):
        self.old = {k: os.environ.get(k) for k in self.kv}
        for k, v in self.kv.items():
            os.environ[k] = str(v)

    def __exit__(self, *a):
        for k, v in self.old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def _dev(a, gpu):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to(gpu)


def _bits(a, dtype, gpu):
    import torch

    return torch.from_numpy(a.view(np.int16)).to(gpu).view(torch_dtype(dtype))


def _repack_ex(case, gpu, layout="gptq", perm=None, order=0):
    """Device repack of the case; returns (weight, sz) tensors."""
    import torch

    from ksanallm_amd import capi

    c = case
    wb, sb = capi.w4a16_repack_sizes(c.K, c.N, c.g)
    w = torch.zeros(wb, dtype=torch.uint8, device=gpu)
    sz = torch.zeros(sb // 4, dtype=torch.int32, device=gpu)
    if layout == "gptq":
        src, lay = c.gptq_qweight(), capi.W4_GPTQ_INT32_KPACK
    elif layout == "awq":
        src, lay = c.awq_qweight(), capi.W4_AWQ_INT32_NPACK
    elif layout == "cutlass80":
        src, lay = orc.cutlass_preprocess(c.rowmajor(), 80), capi.W4_CUTLASS_SM80_INTERLEAVED
    elif layout == "cutlass90":
        src, lay = orc.cutlass_preprocess(c.rowmajor(), 90), capi.W4_CUTLASS_SM90_COLMAJOR
    elif layout == "marlin":
        lay = capi.W4_MARLIN
        if c.kind == "gptq":
            src = orc.marlin_repack(c.gptq_qweight(), c.K, c.N, "gptq")
        else:
            src = orc.marlin_repack(c.awq_qweight(), c.K, c.N, "awq")
    else:
        src, lay = c.rowmajor(), capi.W4_ROWMAJOR_INT4_SIGNED
    zk, zeros = (capi.ZERO_NONE, None) if c.z is None else (capi.ZERO_UINT8, _dev(c.z, gpu))
    scales = _dev(c.scales.view(np.int16), gpu)
    if layout == "marlin":
        scales = _dev(orc.marlin_permute_scales(c.scales, c.K, c.g).view(np.int16), gpu)
        if c.z is not None:
            zk, zeros = capi.ZERO_MARLIN_INT32, _dev(orc.marlin_zero_points(c.z), gpu)
    p = None if perm is None else _dev(perm.astype(np.int32), gpu)
    capi.w4a16_repack_ex(lay, _dev(src, gpu), zk, zeros, scales, capi_dtype(c.dtype), c.K, c.N, c.g, p, order, w, sz)
    torch.cuda.synchronize()
    return w, sz


def _gemm_ex(case, gpu, w, sz, perm=None, epilogue=0, bias=None, act_order_ws=False, out_cols=None):
    import torch

    from ksanallm_amd import capi

    c = case
    act = _bits(c.act, c.dtype, gpu)
    ws_bytes = capi.w4a16_workspace_bytes_ex(max(c.M, 1), c.N, c.K, perm is not None or act_order_ws)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=gpu)
    out = torch.full((c.M, out_cols or c.N), float("nan"), dtype=torch_dtype(c.dtype), device=gpu)
    p = None if perm is None else _dev(perm.astype(np.int32), gpu)
    capi.w4a16_gemm_ex(capi_dtype(c.dtype), out, act, w, sz, c.M, c.N, c.K, c.g, p, epilogue, bias, ws, ws_bytes)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


# ------------------------------------------------------------------------------------------------ load side

@pytest.mark.parametrize("layout", ["cutlass80", "cutlass90", "awq"])
@pytest.mark.parametrize("order", [0, 1])
def test_device_repack_ex_matches_host(gpu, layout, order):
    from ksanallm_amd import capi

    case = W4Case(2000, 1, 512, 96, g=64, kind="awq", dtype="f16")
    perm = np.random.default_rng(2001).permutation(case.K).astype(np.int32)
    w, sz = _repack_ex(case, gpu, layout=layout, perm=perm, order=order)
    c = case
    src = {"cutlass80": lambda: orc.cutlass_preprocess(c.rowmajor(), 80),
           "cutlass90": lambda: orc.cutlass_preprocess(c.rowmajor(), 90), "awq": c.awq_qweight}[layout]()
    lay = {"cutlass80": capi.W4_CUTLASS_SM80_INTERLEAVED, "cutlass90": capi.W4_CUTLASS_SM90_COLMAJOR,
           "awq": capi.W4_AWQ_INT32_NPACK}[layout]
    hw = np.zeros(c.K * c.N // 8, dtype=np.uint32)
    hsz = np.zeros((c.K // c.g) * c.N, dtype=np.uint32)
    capi.w4a16_repack_ex_host(lay, src, capi.ZERO_UINT8, c.z, c.scales, capi_dtype(c.dtype), c.K, c.N, c.g, perm, order,
                              hw, hsz)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), hw)
    assert np.array_equal(sz.cpu().numpy().view(np.uint32), hsz)


@pytest.mark.parametrize("layout", ["cutlass80", "cutlass90"])
@pytest.mark.parametrize("dtype,M", [("f16", 16), ("bf16", 70)])
def test_gemm_from_preprocessed_weights(gpu, layout, dtype, M):
    """What the loader's CUTLASS back end leaves in the weight tensor is accepted as it is."""
    case = W4Case(2010 + M, M, 768, 208, g=128, kind="awq", dtype=dtype)
    w, sz = _repack_ex(case, gpu, layout=layout)
    got = _gemm_ex(case, gpu, w, sz)
    orc.assert_parity(got, case.oracle(), f"{layout} {dtype} M={M}")


@pytest.mark.parametrize("kind,dtype,M,g", [("gptq", "f16", 16, 128), ("awq", "bf16", 40, 64), ("awq", "f16", 150, 128)])
def test_gemm_from_marlin_weights(gpu, kind, dtype, M, g):
    """What the loader's Marlin back end leaves behind (weight tiles, permuted scales, Marlin zero points)."""
    case = W4Case(2015 + M, M, 768, 192, g=g, kind=kind, dtype=dtype)
    w, sz = _repack_ex(case, gpu, layout="marlin")
    got = _gemm_ex(case, gpu, w, sz)
    orc.assert_parity(got, case.oracle(), f"marlin {kind} {dtype} M={M}")


def test_desc_act_marlin_weights(gpu):
    """The Marlin repack of a desc_act checkpoint already stores the rows in sorted order (has_perm,
    gptq_marlin_repack.cu:100-114): no row permutation at repack, the loader's perm at run time."""
    from ksanallm_amd import capi

    K, N, g, M = 512, 128, 128, 20
    rng = np.random.default_rng(2017)
    case = W4Case(2018, M, K, N, g=g, kind="gptq", dtype="f16")
    order = rng.permutation(K)
    g_idx = np.empty(K, dtype=np.int32)
    g_idx[order] = np.arange(K, dtype=np.int32) // g
    perm = np.empty(K, dtype=np.int32)
    capi.gptq_act_order_perm(g_idx, K, g, perm)
    sorted_case = W4Case(2018, M, K, N, g=g, kind="gptq", dtype="f16")
    sorted_case.u = np.ascontiguousarray(case.u[perm])  # what gptq_marlin_repack reads through perm
    w, sz = _repack_ex(sorted_case, gpu, layout="marlin")
    got = _gemm_ex(case, gpu, w, sz, perm=perm)
    s = orc.from_bits(case.scales, orc.F16)
    wdq = (s[g_idx] * (case.u.astype(np.float32) - 8.0)).astype(np.float32)
    want = orc.gemm_f32(orc.from_bits(case.act, orc.F16), wdq)
    orc.assert_parity(got, want, "desc_act through Marlin weights")


def test_one_hot_rows_through_cutlass_layout_are_exact(gpu):
    """Layout end to end with no tolerance: one-hot activations return dequantised rows exactly."""
    K, N, g = 256, 64, 128
    rows = [0, 1, 31, 32, 33, 63, 64, 127, 128, 200, 255]
    act = np.zeros((len(rows), K), dtype=np.float32)
    for i, k in enumerate(rows):
        act[i, k] = 1.0
    case = W4Case(2020, len(rows), K, N, g=g, kind="awq", dtype="f16", act=act)
    w, sz = _repack_ex(case, gpu, layout="cutlass80")
    got = _gemm_ex(case, gpu, w, sz)
    want = orc.from_bits(orc.to_bits(case.dequantized()[rows], orc.F16), orc.F16)
    assert np.array_equal(got, want)


def test_permute_columns_and_interleave_halves(gpu):
    import torch

    from ksanallm_amd import capi

    rng = np.random.default_rng(2030)
    m, k = 37, 1024
    x = rng.integers(0, 65536, size=(m, k), dtype=np.uint16)
    perm = rng.permutation(k).astype(np.int32)
    out = torch.zeros((m, k), dtype=torch.int16, device=gpu)
    capi.permute_columns(out, _dev(x.view(np.int16), gpu), _dev(perm, gpu), m, k)
    rows, row_bytes = 96, 136
    y = rng.integers(0, 256, size=(rows, row_bytes), dtype=np.uint8)
    out2 = torch.zeros((rows, row_bytes), dtype=torch.uint8, device=gpu)
    capi.interleave_halves(out2, _dev(y, gpu), rows, row_bytes)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), x[:, perm])
    want = np.empty_like(y)
    want[0::2] = y[: rows // 2]
    want[1::2] = y[rows // 2:]
    assert np.array_equal(out2.cpu().numpy(), want)


@pytest.mark.parametrize("dtype,M,g", [("f16", 1, 128), ("f16", 16, 64), ("bf16", 48, 128), ("bf16", 150, 128)])
def test_desc_act_checkpoint(gpu, dtype, M, g):
    """GPTQ act-order: row k belongs to group g_idx[k].  The oracle dequantises with the gathered scales; the library
    sorts the rows by group at load time and gathers the activations' columns at run time."""
    from ksanallm_amd import capi

    K, N = 1024, 272
    rng = np.random.default_rng(2040 + M)
    case = W4Case(2041 + M, M, K, N, g=g, kind="gptq", dtype=dtype)
    order = rng.permutation(K)
    g_idx = np.empty(K, dtype=np.int32)
    g_idx[order] = np.arange(K, dtype=np.int32) // g
    perm = np.empty(K, dtype=np.int32)
    capi.gptq_act_order_perm(g_idx, K, g, perm)
    w, sz = _repack_ex(case, gpu, layout="gptq", perm=perm)
    got = _gemm_ex(case, gpu, w, sz, perm=perm)
    s = orc.from_bits(case.scales, ORC_DT[dtype])                       # [G, N]
    wdq = (s[g_idx] * (case.u.astype(np.float32) - 8.0)).astype(np.float32)  # [K, N], row-wise group lookup
    want = orc.gemm_f32(orc.from_bits(case.act, ORC_DT[dtype]), wdq)
    orc.assert_parity(got, want, f"desc_act {dtype} M={M} g={g}")


def test_act_perm_without_workspace_is_refused(gpu):
    import torch

    from ksanallm_amd import capi

    case = W4Case(2050, 4, 256, 64, kind="gptq", dtype="f16")
    w, sz = _repack_ex(case, gpu)
    perm = _dev(np.arange(case.K, dtype=np.int32), gpu)
    out = torch.zeros((4, 64), dtype=torch.float16, device=gpu)
    with pytest.raises(capi.KsqError) as e:
        capi.w4a16_gemm_ex(capi.F16, out, _bits(case.act, "f16", gpu), w, sz, 4, 64, 256, 128, perm, 0, None, None, 0)
    assert e.value.code == capi.ERR_WORKSPACE
    with pytest.raises(capi.KsqError) as e:
        capi.w4a16_gemm_ex(capi.F16, out, _bits(case.act, "f16", gpu), w, sz, 4, 64, 256, 128, None, capi.EPILOGUE_BIAS,
                           None, None, 0)
    assert e.value.code == capi.ERR_INVALID_ARGUMENT


# ------------------------------------------------------------------------------------------------ store side

ROUTES = {
    "auto": {},
    "kstat": {"KSQ_W4_ASTREAM": 0},
    "astream": {"KSQ_W4_ASTREAM": 1},
    "astream_splitk": {"KSQ_W4_ASTREAM": 1, "KSQ_W4_ASTREAM_KSPLIT": 2},
    "astream_lds": {"KSQ_W4_ASTREAM": 1, "KSQ_W4_ASTREAM_LDS": 1, "KSQ_W4_ASTREAM_KSPLIT": 3},
    "stream": {"KSQ_W4_ASTREAM": 0, "KSQ_W4_KSTAT": 0, "KSQ_W4_FORCE_STREAM": 1},
    "stream_splitk": {"KSQ_W4_ASTREAM": 0, "KSQ_W4_KSTAT": 0, "KSQ_W4_FORCE_STREAM": 1, "KSQ_W4_KSPLIT": 3},
    "rows64": {"KSQ_W4_PREFILL_ROWS": 64, "KSQ_W4_PREFILL_KSPLIT": 1},
    "rows64_splitk": {"KSQ_W4_PREFILL_ROWS": 64, "KSQ_W4_PREFILL_KSPLIT": 3},
    "rows128": {"KSQ_W4_PREFILL_ROWS": 128},
}
EPI_CASES = [("auto", 1), ("auto", 16), ("kstat", 24), ("astream", 24), ("kstat", 64), ("astream", 64), ("astream_splitk", 24), ("astream_splitk", 64), ("astream_lds", 40), ("stream", 9),
             ("stream", 100), ("stream_splitk", 33), ("rows64", 100), ("rows64_splitk", 100), ("rows128", 200), ("auto", 300)]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("route,M", EPI_CASES)
def test_silu_mul_epilogue(gpu, dtype, route, M):
    """Fused gate/up: the [K, 2H] weight [gate | up] is repacked with its column pairs interleaved and the GEMM stores
    silu(gate) * up, [M, H]."""
    from ksanallm_amd import capi

    K, N = 1152, 544  # 9 k tiles, 34 column tiles
    case = W4Case(2100 + M, M, K, N, g=128, kind="awq", dtype=dtype)
    w, sz = _repack_ex(case, gpu, layout="awq", order=capi.COLS_HALVES_INTERLEAVED)
    with _env(**ROUTES[route]):
        got = _gemm_ex(case, gpu, w, sz, epilogue=capi.EPILOGUE_SILU_MUL, out_cols=N // 2)
        again = _gemm_ex(case, gpu, w, sz, epilogue=capi.EPILOGUE_SILU_MUL, out_cols=N // 2)
    want = orc.silu_mul(case.oracle())
    orc.assert_parity(got, want, f"silu_mul {dtype} {route} M={M}")
    assert np.array_equal(got, again)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("route,M", EPI_CASES)
def test_bias_epilogue(gpu, dtype, route, M):
    from ksanallm_amd import capi

    K, N = 1152, 544
    case = W4Case(2200 + M, M, K, N, g=128, kind="awq", dtype=dtype)
    w, sz = _repack_ex(case, gpu, layout="awq")
    bias_bits = orc.to_bits(np.random.default_rng(2201).standard_normal(N).astype(np.float32) * 3, ORC_DT[dtype])
    with _env(**ROUTES[route]):
        got = _gemm_ex(case, gpu, w, sz, epilogue=capi.EPILOGUE_BIAS, bias=_bits(bias_bits, dtype, gpu))
    want = case.oracle() + orc.from_bits(bias_bits, ORC_DT[dtype])[None, :]
    orc.assert_parity(got, want, f"bias {dtype} {route} M={M}")


def _fp8_case(seed, M, K, N, per_channel):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    a_bits, w_bits = orc.to_bits(a, orc.BF16), orc.to_bits(w, orc.BF16)
    if per_channel:
        a_s = orc.fp8_compute_scale(a_bits, orc.BF16, M, K)
        w_s = orc.fp8_compute_scale(w_bits, orc.BF16, N, K)
        aq = orc.fp8_quantize(a_bits, orc.BF16, a_s, M, K)
        wq = orc.fp8_quantize(w_bits, orc.BF16, w_s, N, K)
    else:
        a_s = orc.fp8_compute_scale(a_bits, orc.BF16, 1, M * K)
        w_s = orc.fp8_compute_scale(w_bits, orc.BF16, 1, N * K)
        aq = orc.fp8_quantize(a_bits, orc.BF16, a_s, 1, M * K).reshape(M, K)
        wq = orc.fp8_quantize(w_bits, orc.BF16, w_s, 1, N * K).reshape(N, K)
    return aq.reshape(M, K), a_s, wq.reshape(N, K), w_s


@pytest.mark.parametrize("out_dtype", ["f16", "bf16"])
@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("M,kstat,K", [(1, 1, 1024), (16, 1, 1024), (16, 0, 1024), (40, 1, 1024), (64, 1, 1024),
                                       (100, 1, 1024), (256, 1, 1024), (100, 1, 4096), (300, 1, 4096)])
@pytest.mark.parametrize("epilogue", ["bias", "silu_mul"])
def test_fp8_epilogues(gpu, out_dtype, per_channel, M, kstat, K, epilogue):
    """The same two epilogues on the FP8 GEMM (k-stationary, streaming and large-M kernels; with K = 4096 the large-M
    kernel splits K over its few tiles and the reduction kernel applies the epilogue).  For SiLU-mul the weight
    rows [gate ; up] and their scales are interleaved with ksq_interleave_halves."""
    import torch

    from ksanallm_amd import capi

    N = 544
    aq, a_s, wq, w_s = _fp8_case(2300 + M + K, M, K, N, per_channel)
    acc = orc.fp8_gemm(aq, a_s, wq, w_s)
    d_wq, d_ws = _dev(wq, gpu), _dev(w_s, gpu)
    bias = None
    if epilogue == "silu_mul":
        il = torch.zeros_like(d_wq)
        capi.interleave_halves(il, d_wq, N, K)
        d_wq = il
        if per_channel:
            ils = torch.zeros_like(d_ws)
            capi.interleave_halves(ils, d_ws, N, 4)
            d_ws = ils
        want, epi, cols = orc.silu_mul(acc), capi.EPILOGUE_SILU_MUL, N // 2
    else:
        bias_bits = orc.to_bits(np.random.default_rng(2301).standard_normal(N).astype(np.float32), ORC_DT[out_dtype])
        bias = _bits(bias_bits, out_dtype, gpu)
        want, epi, cols = acc + orc.from_bits(bias_bits, ORC_DT[out_dtype])[None, :], capi.EPILOGUE_BIAS, N
    ws_bytes = capi.fp8_workspace_bytes(M, N, K)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=gpu)
    out = torch.full((M, cols), float("nan"), dtype=torch_dtype(out_dtype), device=gpu)
    with _env(KSQ_FP8_KSTAT=kstat):
        capi.fp8_gemm_ex(capi_dtype(out_dtype), out, _dev(aq, gpu), _dev(a_s, gpu), a_s.size, d_wq, d_ws, w_s.size, M, N,
                         K, epi, bias, ws, ws_bytes)
    torch.cuda.synchronize()
    orc.assert_parity(out.float().cpu().numpy(), want, f"fp8 {epilogue} M={M} per_channel={per_channel}")


# ---- F2, producer side: row maxima out of the GEMM's epilogue, consumed by the per-token FP8 quantiser ------------------
ROWMAX_CASES = [("kstat", 5, {}), ("kstat", 16, {}), ("kstat_splitk", 16, {"KSQ_W4_KSPLIT": 2}),
                ("astream", 40, {"KSQ_W4_ASTREAM": 1}), ("astream_lds", 64, {"KSQ_W4_ASTREAM": 1, "KSQ_W4_ASTREAM_LDS": 1}),
                ("stream", 9, {"KSQ_W4_KSTAT": 0}), ("rows64", 100, {"KSQ_W4_PREFILL_ROWS": 64}),
                ("rows64_splitk", 100, {"KSQ_W4_PREFILL_ROWS": 64, "KSQ_W4_PREFILL_KSPLIT": 2}),
                ("rows128", 200, {"KSQ_W4_PREFILL_ROWS": 128}), ("auto", 300, {})]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("epilogue", ["none", "silu_mul"])
@pytest.mark.parametrize("route,M,env", ROWMAX_CASES)
def test_w4a16_gemm_row_maxima_feed_the_quantiser(gpu, dtype, epilogue, route, M, env):
    """ksq_w4a16_gemm_rowmax: the output equals the plain GEMM's bit for bit, row_absmax is exactly the largest |out| of
    every row as stored, and the one-pass quantiser fed with it writes the bytes and scales of the two-pass one."""
    import torch

    from ksanallm_amd import capi

    case = W4Case(2300 + M, M, 1024, 544, g=128, kind="awq", dtype=dtype)
    dev = W4Device(case, gpu)
    big = torch.empty(16 << 20, dtype=torch.uint8, device=gpu)
    epi = capi.EPILOGUE_SILU_MUL if epilogue == "silu_mul" else capi.EPILOGUE_NONE
    cols = case.N // 2 if epi == capi.EPILOGUE_SILU_MUL else case.N
    tdt, cdt = torch_dtype(dtype), capi_dtype(dtype)
    ref = torch.full((M, cols), float("nan"), dtype=tdt, device=gpu)
    out = torch.full((M, cols), float("nan"), dtype=tdt, device=gpu)
    rowmax = torch.full((M,), 123.0, dtype=torch.float32, device=gpu)
    with _env(**env):
        capi.w4a16_gemm_ex(cdt, ref, dev.act, dev.weight, dev.sz, M, case.N, case.K, case.g, None, epi, None, big, big.numel())
        capi.fill_zero_f32(rowmax, M)
        capi.w4a16_gemm_rowmax(cdt, out, dev.act, dev.weight, dev.sz, M, case.N, case.K, case.g, rowmax, epi, None, big,
                               big.numel())
    torch.cuda.synchronize()
    assert torch.equal(ref.view(torch.int16), out.view(torch.int16)), route
    want = out.float().abs().max(dim=1).values
    assert torch.equal(rowmax, want), (route, rowmax[:4], want[:4])
    # consumer: one pass with the known maxima == max pass + quantise
    q1 = torch.empty((M, cols), dtype=torch.uint8, device=gpu)
    s1 = torch.empty(M, dtype=torch.float32, device=gpu)
    q2, s2 = torch.empty_like(q1), torch.empty_like(s1)
    capi.fp8_quantize(cdt, out, M, cols, capi.FP8_PER_TOKEN_DYNAMIC, q1, s1)
    capi.fp8_quantize_rows_from_absmax(cdt, out, M, cols, rowmax, q2, s2)
    torch.cuda.synchronize()
    assert torch.equal(s1, s2) and torch.equal(q1, q2), route


@pytest.mark.parametrize("out_dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M,K,env", [(1, 1024, {}), (16, 1024, {}), (16, 1024, {"KSQ_FP8_KSTAT": 0}), (40, 1024, {}),
                                     (100, 1024, {}), (300, 1024, {}), (300, 4096, {"KSQ_FP8_TAIL_KSPLIT": 2}),
                                     (130, 1024, {"KSQ_FP8_PREFILL_TILE": 128}), (7, 1008, {})])
def test_fp8_gemm_row_maxima(gpu, out_dtype, M, K, env):
    import torch

    from ksanallm_amd import capi

    rng = np.random.default_rng(2400 + M)
    N = 528
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    xq = codes[rng.integers(0, len(codes), size=(M, K))] & np.uint8(0xBF)
    wq = codes[rng.integers(0, len(codes), size=(N, K))] & np.uint8(0xBF)
    xs = ((rng.random(M) + 0.5) * 1e-2).astype(np.float32)
    ws = ((rng.random(N) + 0.5) * 1e-2).astype(np.float32)
    tdt, cdt = torch_dtype(out_dtype), capi_dtype(out_dtype)
    dx, dw = torch.from_numpy(xq).to(gpu), torch.from_numpy(wq).to(gpu)
    dxs, dws = torch.from_numpy(xs).to(gpu), torch.from_numpy(ws).to(gpu)
    wsb = capi.fp8_workspace_bytes(M, N, K)
    wk = torch.empty(max(wsb, 256), dtype=torch.uint8, device=gpu)
    ref = torch.full((M, N), float("nan"), dtype=tdt, device=gpu)
    out = torch.full((M, N), float("nan"), dtype=tdt, device=gpu)
    rowmax = torch.zeros(M, dtype=torch.float32, device=gpu)
    with _env(**env):
        capi.fp8_gemm_ex(cdt, ref, dx, dxs, M, dw, dws, N, M, N, K, capi.EPILOGUE_NONE, None, wk, wsb)
        capi.fp8_gemm_rowmax(cdt, out, dx, dxs, M, dw, dws, N, M, N, K, rowmax, capi.EPILOGUE_NONE, None, wk, wsb)
    torch.cuda.synchronize()
    assert torch.equal(ref.view(torch.int16), out.view(torch.int16))
    assert torch.equal(rowmax, out.float().abs().max(dim=1).values)
