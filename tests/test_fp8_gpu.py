"""FP8 e4m3 parity tests: quantise / rescale / weight conversion must match the oracle bit for bit (the oracle is
pinned by the closed forms of the reference's own unit test); the GEMM is held to the parity bar against the
oracle's fp32 accumulation."""
import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import ORC_DT, bits_of, capi_dtype, torch_dtype
from tests.test_w4a16_gpu import _env

pytestmark = pytest.mark.gpu

REF_SHAPES = [(1, 31), (1, 16383), (16383, 7), (7, 16383), (16383, 1), (31, 1)]  # LU/utils_test.cu:30,64


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def _upload_bits(bits, dtype, gpu):
    import torch

    if dtype == "f32":  # the oracle's "bits" of fp32 are the floats themselves
        return torch.from_numpy(np.ascontiguousarray(bits, dtype=np.float32)).to(gpu)
    return torch.from_numpy(bits.view(np.int16)).to(gpu).view(torch_dtype(dtype))


def _quantize(gpu, xbits, dtype, mode, static_scale=None):
    import torch

    from ksanallm_amd import capi

    m, k = xbits.shape
    x = _upload_bits(xbits, dtype, gpu)
    q = torch.zeros((m, k), dtype=torch.uint8, device=gpu)
    nscale = m if mode == capi.FP8_PER_TOKEN_DYNAMIC else 1
    scale = torch.full((nscale,), -1.0, dtype=torch.float32, device=gpu)
    if static_scale is not None:
        scale.fill_(float(static_scale))
    capi.fp8_quantize(capi_dtype(dtype), x, m, k, mode, q, scale)
    torch.cuda.synchronize()
    return q.cpu().numpy(), scale.cpu().numpy()


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("shape", REF_SHAPES)
def test_per_channel_quantize_reference_shapes(gpu, dtype, shape):
    from ksanallm_amd import capi

    C, L = shape
    rng = np.random.default_rng(300)
    x = orc.to_bits((rng.random((C, L), dtype=np.float32) * 0.2 - 0.1), ORC_DT[dtype])
    q, s = _quantize(gpu, x, dtype, capi.FP8_PER_TOKEN_DYNAMIC)
    want_s = orc.fp8_compute_scale(x, ORC_DT[dtype], C, L)
    assert np.array_equal(s, want_s)
    assert np.array_equal(q, orc.fp8_quantize(x, ORC_DT[dtype], want_s, C, L))


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("m,k", [(1, 4096), (16, 8192), (64, 1000), (300, 512)])
def test_per_tensor_dynamic_and_static(gpu, dtype, m, k):
    from ksanallm_amd import capi

    rng = np.random.default_rng(301)
    xv = rng.standard_normal((m, k)).astype(np.float32)
    xv[0, 0] = 7.5  # a clear maximum
    x = orc.to_bits(xv, ORC_DT[dtype])
    q, s = _quantize(gpu, x, dtype, capi.FP8_PER_TENSOR_DYNAMIC)
    want_s = orc.fp8_compute_scale(x, ORC_DT[dtype], 1, m * k)
    assert np.array_equal(s, want_s)
    assert np.array_equal(q.reshape(1, -1), orc.fp8_quantize(x, ORC_DT[dtype], want_s, 1, m * k))
    st = np.array([0.0123], dtype=np.float32)  # static: values beyond 448 * scale must saturate
    q2, s2 = _quantize(gpu, x, dtype, capi.FP8_PER_TENSOR_STATIC, static_scale=st[0])
    assert np.array_equal(s2, st)
    assert np.array_equal(q2.reshape(1, -1), orc.fp8_quantize(x, ORC_DT[dtype], st, 1, m * k))


def test_quantize_special_values(gpu):
    from ksanallm_amd import capi

    vals = np.array([0.0, -0.0, 448.0, -448.0, 500.0, 1e-8, 2.0**-9, 2.0**-10, 3 * 2.0**-10, 0.0175, 464.0, 65504.0],
                    dtype=np.float32)
    x = orc.to_bits(np.tile(vals, 4)[None, :], orc.F16)
    st = np.array([1.0], dtype=np.float32)
    q, _ = _quantize(gpu, x, "f16", capi.FP8_PER_TENSOR_STATIC, static_scale=1.0)
    want = orc.fp8_quantize(x, orc.F16, st, 1, x.shape[1])
    assert np.array_equal(q & 0x7F, want & 0x7F)  # sign of zero is not significant
    nz = (want & 0x7F) != 0
    assert np.array_equal(q[nz], want[nz])
    zeros = np.zeros((3, 64), dtype=np.uint16)
    _, s = _quantize(gpu, zeros, "f16", capi.FP8_PER_TOKEN_DYNAMIC)
    assert np.array_equal(s, np.full(3, np.float32(1.0) / 448 / 512, dtype=np.float32))


@pytest.mark.parametrize("n", [1, 7, 31, 16383])
def test_rescale(gpu, n):
    import torch

    from ksanallm_amd import capi

    rng = np.random.default_rng(302)
    q = rng.integers(0, 256, size=n, dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0x21
    s_in, s_out = np.float32(0.37), np.float32(0.11)
    dq = torch.from_numpy(q).to(gpu)
    out = torch.zeros_like(dq)
    si = torch.tensor([s_in], dtype=torch.float32, device=gpu)
    so = torch.tensor([s_out], dtype=torch.float32, device=gpu)
    capi.fp8_rescale(dq, out, n, si, so)
    torch.cuda.synchronize()
    want = orc.fp8_rescale(q, s_in, s_out)
    got = out.cpu().numpy()
    nz = (want & 0x7F) != 0
    assert np.array_equal(got[nz], want[nz]) and np.all((got[~nz] & 0x7F) == 0)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_convert_weight(gpu, dtype):
    import torch

    from ksanallm_amd import capi

    rng = np.random.default_rng(303)
    K, N = 200, 136
    w = orc.to_bits(rng.standard_normal((K, N)).astype(np.float32) * 0.02, ORC_DT[dtype])
    dw = _upload_bits(w, dtype, gpu)
    wq = torch.zeros((N, K), dtype=torch.uint8, device=gpu)
    ws = torch.zeros(1, dtype=torch.float32, device=gpu)
    capi.fp8_convert_weight(capi_dtype(dtype), dw, K, N, wq, ws)
    torch.cuda.synchronize()
    want_q, want_s = orc.fp8_convert_weight(w, ORC_DT[dtype])
    assert np.array_equal(ws.cpu().numpy(), want_s)
    got = wq.cpu().numpy()
    nz = (want_q & 0x7F) != 0
    assert np.array_equal(got[nz], want_q[nz]) and np.all((got[~nz] & 0x7F) == 0)


def _fp8_case(seed, M, K, N):
    """configs[4] recipe: W = quantise(N(0,1) * 0.02, per-channel absmax / 448); activations N(0,1) in bf16 quantised
    per token."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    w_scale = orc.fp8_compute_scale(w, orc.F32, N, K)
    wq = orc.fp8_quantize(w, orc.F32, w_scale, N, K)
    x = orc.to_bits(rng.standard_normal((M, K)).astype(np.float32), orc.BF16)
    x_scale = orc.fp8_compute_scale(x, orc.BF16, M, K)
    xq = orc.fp8_quantize(x, orc.BF16, x_scale, M, K)
    return xq, x_scale, wq, w_scale


def _run_gemm(gpu, xq, x_scale, wq, w_scale, out_dtype, use_workspace=True):
    import torch

    from ksanallm_amd import capi

    M, K = xq.shape
    N = wq.shape[0]
    dx, dw = torch.from_numpy(xq).to(gpu), torch.from_numpy(wq).to(gpu)
    dxs, dws = torch.from_numpy(x_scale).to(gpu), torch.from_numpy(w_scale).to(gpu)
    out = torch.full((M, N), float("nan"), dtype=torch_dtype(out_dtype), device=gpu)
    wsb = capi.fp8_workspace_bytes(M, N, K) if use_workspace else 0
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=gpu)
    capi.fp8_gemm(capi_dtype(out_dtype), out, dx, dxs, x_scale.size, dw, dws, w_scale.size, M, N, K,
                  ws if use_workspace else None, wsb)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("out_dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("M", [1, 3, 16, 17, 64, 65, 130])
def test_gemm_rowwise_scales(gpu, out_dtype, M):
    xq, xs, wq, ws = _fp8_case(400 + M, M, 1024, 272)
    got = _run_gemm(gpu, xq, xs, wq, ws, out_dtype)
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), f"fp8 M={M} {out_dtype}")


def test_gemm_per_tensor_scales_and_ragged_shapes(gpu):
    # per-tensor scalars are what the reference layer passes; N not a multiple of 16 and K a multiple of 16 only
    xq, xs, wq, ws = _fp8_case(401, 5, 1008, 100)
    xs1, ws1 = xs[:1].copy(), ws[:1].copy()
    got = _run_gemm(gpu, xq, xs1, wq, ws1, "bf16")
    orc.assert_parity(got, orc.fp8_gemm(xq, xs1, wq, ws1), "fp8 per-tensor ragged")
    got = _run_gemm(gpu, xq, xs, wq, ws, "bf16", use_workspace=False)
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), "fp8 ragged no workspace")


@pytest.mark.parametrize("M,K,N", [(128, 1024, 256), (300, 1008, 264), (257, 2048, 520)])
def test_gemm_large_m_ragged(gpu, M, K, N):
    """M >= 128: ragged M and N through the MFMA-tiled kernel; K not a multiple of 128 through the streaming kernel."""
    xq, xs, wq, ws = _fp8_case(410 + M, M, K, N)
    got = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), f"fp8 large M={M} K={K} N={N}")
    got1 = _run_gemm(gpu, xq, xs[:1].copy(), wq, ws[:1].copy(), "f16")
    orc.assert_parity(got1, orc.fp8_gemm(xq, xs[:1].copy(), wq, ws[:1].copy()), f"fp8 large per-tensor M={M}")


@pytest.mark.parametrize("tile", [128, 256])
@pytest.mark.parametrize("M,K,N", [(300, 1024, 264), (257, 2048, 520), (512, 384, 768), (128, 128, 256)])
def test_gemm_large_m_both_tiles(gpu, tile, M, K, N):
    """The MFMA-tiled kernel in both workgroup tiles (128 x 256 and 256 x 256), whichever the planner would pick."""
    import os

    xq, xs, wq, ws = _fp8_case(430 + M, M, K, N)
    old = os.environ.get("KSQ_FP8_PREFILL_TILE")
    os.environ["KSQ_FP8_PREFILL_TILE"] = str(tile)
    try:
        got = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
        got2 = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
    finally:
        if old is None:
            os.environ.pop("KSQ_FP8_PREFILL_TILE", None)
        else:
            os.environ["KSQ_FP8_PREFILL_TILE"] = old
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), f"fp8 tile={tile} M={M} K={K} N={N}")
    assert np.array_equal(got, got2)


@pytest.mark.parametrize("ksplit", [0, 1, 2, 3])
@pytest.mark.parametrize("M,K,N", [(300, 4096, 9208), (300, 4096, 2600), (2048, 4096, 9216), (2040, 4096, 11256)])
def test_gemm_large_m_split_last_round(gpu, ksplit, M, K, N):
    """256 x 256 tiles that do not fill whole rounds of one tile per compute unit.  352 tiles on 256 units: the last
    96 go out as a launch of their own with K split (0 = the planner's own count, 1 = no split), partial tiles through
    the workspace, a reduction kernel behind it.  288 tiles: the last 32 cover at most a quarter of the units and go
    out as column quarters (256 x 64, four workgroups to a tile) instead.  72 and 22 tiles (the latter not a multiple
    of eight: the grid is rounded up): a single round that leaves most units empty, so the whole grid is the split
    launch.  Ragged M and N; twice, bit for bit; and without a workspace (no K split)."""
    import os

    xq, xs, wq, ws = _fp8_case(450 + M, M, K, N)
    old = os.environ.get("KSQ_FP8_TAIL_KSPLIT")
    if ksplit:
        os.environ["KSQ_FP8_TAIL_KSPLIT"] = str(ksplit)
    try:
        got = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
        got2 = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
    finally:
        if old is None:
            os.environ.pop("KSQ_FP8_TAIL_KSPLIT", None)
        else:
            os.environ["KSQ_FP8_TAIL_KSPLIT"] = old
    rows = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(M).choice(M, size=40, replace=False)]))
    want = orc.fp8_gemm(xq[rows], xs[rows], wq, ws)
    orc.assert_parity(got[rows], want, f"fp8 tail split {ksplit} M={M} K={K} N={N}")
    assert np.array_equal(got, got2)
    got3 = _run_gemm(gpu, xq, xs, wq, ws, "bf16", use_workspace=False)
    orc.assert_parity(got3[rows], want, f"fp8 no workspace M={M}")


def test_gemm_large_m_small_integers_exact(gpu):
    rng = np.random.default_rng(420)
    M, K, N = 256, 384, 256
    codes = orc.e4m3_encode(np.arange(-4, 5, dtype=np.float32))
    xq = codes[rng.integers(0, 9, size=(M, K))]
    wq = codes[rng.integers(0, 9, size=(N, K))]
    one = np.ones(1, dtype=np.float32)
    got = _run_gemm(gpu, xq, one, wq, one, "f16")
    want = orc.e4m3_decode(xq).astype(np.int64) @ orc.e4m3_decode(wq).astype(np.int64).T
    assert np.array_equal(orc.to_bits(got, orc.F16), orc.to_bits(want.astype(np.float32), orc.F16))


def test_gemm_small_integers_exact(gpu):
    rng = np.random.default_rng(402)
    M, K, N = 16, 512, 64
    codes = orc.e4m3_encode(np.arange(-4, 5, dtype=np.float32))
    xq = codes[rng.integers(0, 9, size=(M, K))]
    wq = codes[rng.integers(0, 9, size=(N, K))]
    one = np.ones(1, dtype=np.float32)
    got = _run_gemm(gpu, xq, one, wq, one, "f16")
    want = orc.e4m3_decode(xq).astype(np.int64) @ orc.e4m3_decode(wq).astype(np.int64).T
    assert np.array_equal(orc.to_bits(got, orc.F16), orc.to_bits(want.astype(np.float32), orc.F16))


@pytest.mark.parametrize("wide", [0, 1])
@pytest.mark.parametrize("M,K,N", [(1, 1024, 272), (5, 8208, 100), (16, 9600, 528), (9, 29568, 272)])
def test_gemm_one_row_tile_both_workgroup_shapes(gpu, wide, M, K, N):
    """M <= 16 with 16 waves x 4 stages and with 8 waves x 8 stages per workgroup (what the planner takes for K above
    8192), including K that is split over workgroups and K that is not a multiple of 128; twice, bit for bit."""
    import os

    xq, xs, wq, ws = _fp8_case(440 + M, M, K, N)
    old = os.environ.get("KSQ_FP8_WIDE")
    os.environ["KSQ_FP8_WIDE"] = str(wide)
    try:
        got = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
        got2 = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
    finally:
        if old is None:
            os.environ.pop("KSQ_FP8_WIDE", None)
        else:
            os.environ["KSQ_FP8_WIDE"] = old
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), f"fp8 wide={wide} M={M} K={K} N={N}")
    assert np.array_equal(got, got2)


@pytest.mark.parametrize("M,K,N,env", [
    (5, 1024, 272, {}),                                   # decode kernel
    (3, 4224, 528, {"KSQ_FP8_KPHASE": 1}),                # K in phases inside the workgroup
    (40, 1008, 100, {}),                                  # K % 128 != 0: streaming kernel
    (70, 1024, 264, {"KSQ_FP8_KSTAT": 0, "KSQ_FP8_PREFILL_MIN_M": 1000}),  # streaming kernel, several row tiles
    (300, 1024, 264, {}),                                 # 256 x 256 tiles
    (300, 4096, 2600, {"KSQ_FP8_TAIL_KSPLIT": 2}),        # ... with K split and the reduction kernel
    (300, 4096, 9208, {"KSQ_FP8_TAIL_KSPLIT": 1}),        # ... with a last round of column quarters
    (130, 1024, 520, {"KSQ_FP8_PREFILL_TILE": 128}),      # 128 x 256 tiles
])
def test_gemm_fp32_results_every_route(gpu, M, K, N, env):
    """out_dtype = fp32 (what the reference's Fp8MatMulLayer<float> gets from its GEMM) through every kernel family:
    the result is the fp32 accumulator times the scales, so it must agree with the oracle far inside the tolerance
    of the 16-bit outputs; twice, bit for bit."""
    xq, xs, wq, ws = _fp8_case(480 + M, M, K, N)
    with _env(**env):
        got = _run_gemm(gpu, xq, xs, wq, ws, "f32")
        got2 = _run_gemm(gpu, xq, xs, wq, ws, "f32")
    want = orc.fp8_gemm(xq, xs, wq, ws)
    orc.assert_parity(got, want, f"fp8 fp32 out M={M} K={K} N={N} {env}")
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert float(np.max(np.abs(got - want))) <= 2e-5 * rms * np.sqrt(K), "fp32 results carry no 16-bit rounding"
    assert np.array_equal(got, got2)


@pytest.mark.parametrize("M", [1, 8, 70])
def test_gemm_dynamic_fp32(gpu, M):
    """fp32 activations in, fp32 results out: per-token quantisation (bit-identical to the oracle's, through the
    element-wise kernels) and the GEMM as one call, with a bias row in fp32."""
    import torch

    from ksanallm_amd import capi

    K, N = 1024, 272
    rng = np.random.default_rng(490 + M)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    w_scale = orc.fp8_compute_scale(w, orc.F32, N, K)
    wq = orc.fp8_quantize(w, orc.F32, w_scale, N, K)
    x_scale = orc.fp8_compute_scale(x, orc.F32, M, K)
    xq = orc.fp8_quantize(x, orc.F32, x_scale, M, K)
    want = orc.fp8_gemm(xq, x_scale, wq, w_scale) + bias[None, :]
    dx, dw, dws, db = (torch.from_numpy(a).to(gpu) for a in (x, wq, w_scale, bias))
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device=gpu)
    wsb = capi.fp8_gemm_dynamic_workspace_bytes(M, N, K)
    ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device=gpu)
    capi.fp8_gemm_dynamic(capi.F32, out, dx, dw, dws, N, M, N, K, capi.EPILOGUE_BIAS, db, ws, wsb)
    torch.cuda.synchronize()
    orc.assert_parity(out.cpu().numpy(), want, f"fp8 dynamic fp32 M={M}")


@pytest.mark.parametrize("per_channel", [True, False])
@pytest.mark.parametrize("M,K,N", [(1, 256, 272), (3, 4224, 528), (4, 8320, 264), (5, 2176, 1040), (8, 8208, 272),
                                   (2, 1008, 4104), (7, 640, 8200), (1, 29568, 272), (6, 4096, 16)])
def test_gemm_k_phases_inside_the_workgroup(gpu, per_channel, M, K, N):
    """One to eight rows with K walked in phases inside the workgroup (what a long K gets instead of a split across
    workgroups): whole and partial last phases, K that is not a multiple of 128, one to four column tiles per
    workgroup, a ragged last workgroup and a ragged last column tile; no workspace needed; two runs bit for bit."""
    import os

    from ksanallm_amd import capi

    xq, xs, wq, ws = _fp8_case(470 + M, M, K, N)
    if not per_channel:
        xs, ws = xs[:1].copy(), ws[:1].copy()
    old = os.environ.get("KSQ_FP8_KPHASE")
    os.environ["KSQ_FP8_KPHASE"] = "1"
    capi.set_launch_log(True)
    try:
        got = _run_gemm(gpu, xq, xs, wq, ws, "bf16", use_workspace=False)
        assert "fp8_kphase_kernel" in capi.last_launch(), capi.last_launch()
        got2 = _run_gemm(gpu, xq, xs, wq, ws, "f16")
        got3 = _run_gemm(gpu, xq, xs, wq, ws, "f16")
    finally:
        capi.set_launch_log(False)
        if old is None:
            os.environ.pop("KSQ_FP8_KPHASE", None)
        else:
            os.environ["KSQ_FP8_KPHASE"] = old
    want = orc.fp8_gemm(xq, xs, wq, ws)
    orc.assert_parity(got, want, f"fp8 k phases M={M} K={K} N={N}")
    orc.assert_parity(got2, want, f"fp8 k phases f16 M={M} K={K} N={N}")
    assert np.array_equal(got2, got3)


@pytest.mark.parametrize("seed", [21, 22, 23, 24])
def test_gemm_random_shapes(gpu, seed):
    """Ten shapes per seed from a seeded random walk over every family of M, N from 8 to a few thousand (ragged column
    tiles included) and K from 16 to 2500 in steps of 16 (the streaming kernel for K % 128 != 0, the decode and tile
    kernels otherwise), per-token x per-channel and per-tensor scales, with and without a workspace."""
    rng = np.random.default_rng(seed)
    for i in range(10):
        M = int(rng.choice([rng.integers(1, 17), rng.integers(17, 65), rng.integers(65, 300)]))
        N = 8 * int(rng.choice([rng.integers(1, 17), rng.integers(17, 300)]))
        K = 16 * int(rng.choice([rng.integers(1, 9), rng.integers(9, 160)])) if rng.integers(0, 2) else 128 * int(rng.integers(1, 20))
        xq, xs, wq, ws = _fp8_case(4000 + 100 * seed + i, M, K, N)
        if rng.integers(0, 2):
            xs, ws = xs[:1].copy(), ws[:1].copy()
        want = orc.fp8_gemm(xq, xs, wq, ws)
        got = _run_gemm(gpu, xq, xs, wq, ws, "bf16" if i % 2 else "f16")
        orc.assert_parity(got, want, f"fp8 random seed {seed} #{i}: M={M} K={K} N={N} scales={len(xs)}x{len(ws)}")
        got = _run_gemm(gpu, xq, xs, wq, ws, "bf16", use_workspace=False)
        orc.assert_parity(got, want, f"fp8 random seed {seed} #{i}, no workspace")


@pytest.mark.parametrize("M", [1, 64])
def test_config4_qwen72b_shape(gpu, M):
    xq, xs, wq, ws = _fp8_case(403, M, 8192, 8192)
    got = _run_gemm(gpu, xq, xs, wq, ws, "bf16")
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), f"cfg4 8192x8192 M={M}")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_convert_weight_per_channel(gpu, dtype):
    import torch

    from ksanallm_amd import capi

    rng = np.random.default_rng(440)
    K, N = 200, 136
    wv = (rng.standard_normal((K, N)) * np.exp2(rng.integers(-8, 3, size=N))[None, :]).astype(np.float32)
    wv[:, 5] = 0.0
    w = orc.to_bits(wv, ORC_DT[dtype])
    dw = _upload_bits(w, dtype, gpu)
    wq = torch.zeros((N, K), dtype=torch.uint8, device=gpu)
    ws = torch.full((N,), -1.0, dtype=torch.float32, device=gpu)
    capi.fp8_convert_weight_per_channel(capi_dtype(dtype), dw, K, N, wq, ws)
    torch.cuda.synchronize()
    want_q, want_s = orc.fp8_convert_weight_per_channel(w, ORC_DT[dtype])
    assert np.array_equal(ws.cpu().numpy(), want_s)
    got = wq.cpu().numpy()
    nz = (want_q & 0x7F) != 0
    assert np.array_equal(got[nz], want_q[nz]) and np.all((got[~nz] & 0x7F) == 0)


def test_merge_qkv_scales(gpu):
    """Max merge bit-exact against the oracle; the per-channel merge leaves the bytes alone and the fused GEMM then
    equals the three separate GEMMs exactly."""
    import torch

    from ksanallm_amd import capi

    rng = np.random.default_rng(441)
    nq, nk, nv, K, M = 64, 32, 32, 256, 5
    wq = rng.integers(0, 256, size=(nq + nk + nv, K), dtype=np.uint8)
    wq[(wq & 0x7F) == 0x7F] = 0x2a
    scales = [np.array([v], dtype=np.float32) for v in (0.021, 0.0503, 0.0127)]
    d_scales = [torch.from_numpy(x).to(gpu) for x in scales]
    dw = torch.from_numpy(wq.copy()).to(gpu)  # rescaled in place: never the host array itself
    out_s = torch.zeros(1, dtype=torch.float32, device=gpu)
    capi.fp8_merge_qkv_scales(capi.FP8_MERGE_MAX, *d_scales, nq, nk, nv, dw, K, out_s)
    torch.cuda.synchronize()
    want_w, want_s = orc.fp8_merge_qkv_max(wq, scales[0][0], scales[1][0], scales[2][0], nq, nk, nv)
    assert np.array_equal(out_s.cpu().numpy(), want_s)
    got = dw.cpu().numpy()
    nz = (want_w & 0x7F) != 0
    assert np.array_equal(got[nz], want_w[nz]) and np.all((got[~nz] & 0x7F) == 0)

    dw2 = torch.from_numpy(wq.copy()).to(gpu)
    chan = torch.zeros(nq + nk + nv, dtype=torch.float32, device=gpu)
    capi.fp8_merge_qkv_scales(capi.FP8_MERGE_PER_CHANNEL, *d_scales, nq, nk, nv, None, K, chan)
    torch.cuda.synchronize()
    want_chan = np.concatenate([np.full(nq, scales[0][0]), np.full(nk, scales[1][0]), np.full(nv, scales[2][0])])
    assert np.array_equal(chan.cpu().numpy(), want_chan.astype(np.float32))
    xq = rng.integers(0, 120, size=(M, K), dtype=np.uint8)
    xs = (rng.random(M).astype(np.float32) * 0.01 + 1e-3).astype(np.float32)
    fused = _run_gemm(gpu, xq, xs, wq, want_chan.astype(np.float32), "f16")
    row = 0
    for rows, sc in ((nq, scales[0]), (nk, scales[1]), (nv, scales[2])):
        part = _run_gemm(gpu, xq, xs, np.ascontiguousarray(wq[row:row + rows]), sc, "f16")
        assert np.array_equal(fused[:, row:row + rows], part)
        row += rows


def _run_dynamic(gpu, x_bits, wq, w_scale, dtype, use_workspace=True, epilogue=0, bias_bits=None):
    """ksq_fp8_gemm_dynamic on activations given as 16-bit patterns of `dtype`."""
    import torch

    from ksanallm_amd import capi

    M, K = x_bits.shape
    N = wq.shape[0]
    dx = _upload_bits(x_bits, dtype, gpu)
    dw, dws = torch.from_numpy(wq).to(gpu), torch.from_numpy(w_scale).to(gpu)
    cols = N // 2 if epilogue == capi.EPILOGUE_SILU_MUL else N
    out = torch.full((M, cols), float("nan"), dtype=torch_dtype(dtype), device=gpu)
    wsb = capi.fp8_gemm_dynamic_workspace_bytes(M, N, K) if use_workspace else 0
    ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device=gpu)
    bias = _upload_bits(bias_bits, dtype, gpu) if bias_bits is not None else None
    capi.fp8_gemm_dynamic(capi_dtype(dtype), out, dx, dw, dws, w_scale.size, M, N, K, epilogue, bias,
                          ws if use_workspace else None, wsb)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("M", [1, 2, 3, 5, 8, 9, 40])
@pytest.mark.parametrize("K,N", [(1024, 272), (8192, 528), (9600, 1040), (4096, 4112)])
def test_gemm_dynamic_quantises_inside(gpu, dtype, M, K, N):
    """Per-token quantisation folded into the GEMM (one launch up to eight rows, two beyond): parity against the
    oracle's quantise-then-GEMM, agreement with the library's own two calls, twice bit for bit; K = 9600 is split over
    workgroups, N = 4112 gives a workgroup several batches."""
    import os

    rng = np.random.default_rng(460 + M + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    ws = orc.fp8_compute_scale(w, orc.F32, N, K)
    wq = orc.fp8_quantize(w, orc.F32, ws, N, K)
    xv = rng.standard_normal((M, K)).astype(np.float32) * np.exp2(rng.integers(-6, 7, size=(M, 1))).astype(np.float32)
    x = orc.to_bits(xv, ORC_DT[dtype])
    os.environ["KSQ_FP8_FUSED_QUANT"] = "1"  # the single-launch form for every m <= 8 (by default it serves m = 1 only)
    try:
        got = _run_dynamic(gpu, x, wq, ws, dtype)
        got2 = _run_dynamic(gpu, x, wq, ws, dtype)
        got3 = _run_dynamic(gpu, x, wq, ws, dtype, use_workspace=False) if M <= 8 and K <= 8192 else None
    finally:
        os.environ.pop("KSQ_FP8_FUSED_QUANT", None)
    xs = orc.fp8_compute_scale(x, ORC_DT[dtype], M, K)
    xq = orc.fp8_quantize(x, ORC_DT[dtype], xs, M, K)
    want = orc.fp8_gemm(xq, xs, wq, ws)
    orc.assert_parity(got.float().cpu().numpy(), want, f"fp8 dynamic M={M} K={K} N={N} {dtype}")
    assert np.array_equal(bits_of(got), bits_of(got2))
    two = _run_gemm(gpu, xq, xs, wq, ws, dtype).astype(np.float64)
    diff = np.abs(got.float().cpu().numpy().astype(np.float64) - two)
    assert np.all(diff <= 2.0 ** -7 * np.maximum(np.abs(two), 1e-6)), "differs from quantise + GEMM by more than an output ulp"
    if got3 is not None:  # no workspace: still one launch (a longer K is split over workgroups and needs one)
        orc.assert_parity(got3.float().cpu().numpy(), want, f"fp8 dynamic, no workspace M={M}")
    dflt = _run_dynamic(gpu, x, wq, ws, dtype)  # the default route choice
    orc.assert_parity(dflt.float().cpu().numpy(), want, f"fp8 dynamic default route M={M}")
    os.environ["KSQ_FP8_FUSED_QUANT"] = "0"
    try:
        got4 = _run_dynamic(gpu, x, wq, ws, dtype)
    finally:
        os.environ.pop("KSQ_FP8_FUSED_QUANT", None)
    assert np.array_equal(got4.float().cpu().numpy().astype(np.float64), two), "two-launch route must equal the two calls"


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("M", [1, 4, 8])
def test_gemm_dynamic_quantiser_is_the_quantise_kernels(gpu, dtype, M):
    """An identity weight (e4m3 1.0 on the diagonal, scale 1) turns the GEMM into out[m, k] = T(float(q[m, k]) * scale[m]):
    the quantised bytes and scales inside the fused kernel, compared exactly with the oracle's."""
    K = N = 1024
    rng = np.random.default_rng(470 + M)
    xv = rng.standard_normal((M, K)).astype(np.float32) * np.exp2(rng.integers(-10, 11, size=(M, 1))).astype(np.float32)
    xv[0, :5] = [0.0, -0.0, 1e-30, -3.0e4 if dtype == "f16" else -3.0e30, 7.5]
    x = orc.to_bits(xv, ORC_DT[dtype])
    wq = np.zeros((N, K), dtype=np.uint8)
    wq[np.arange(N), np.arange(N)] = orc.e4m3_encode(np.array([1.0], dtype=np.float32))[0]
    import os

    os.environ["KSQ_FP8_FUSED_QUANT"] = "1"
    try:
        got = _run_dynamic(gpu, x, wq, np.ones(1, dtype=np.float32), dtype)
    finally:
        os.environ.pop("KSQ_FP8_FUSED_QUANT", None)
    xs = orc.fp8_compute_scale(x, ORC_DT[dtype], M, K)
    xq = orc.fp8_quantize(x, ORC_DT[dtype], xs, M, K)
    want = orc.e4m3_decode(xq) * xs[:, None]
    gb, wb = bits_of(got), orc.to_bits(want.astype(np.float32), ORC_DT[dtype])
    same = (gb == wb) | (((gb & 0x7FFF) == 0) & ((wb & 0x7FFF) == 0))  # the sign of zero is not significant
    assert np.all(same)


def test_gemm_dynamic_epilogues_and_errors(gpu):
    import torch

    from ksanallm_amd import capi

    rng = np.random.default_rng(480)
    M, K, N = 4, 1024, 256
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    ws = orc.fp8_compute_scale(w, orc.F32, N, K)
    wq = orc.fp8_quantize(w, orc.F32, ws, N, K)
    x = orc.to_bits(rng.standard_normal((M, K)).astype(np.float32), orc.BF16)
    xs = orc.fp8_compute_scale(x, orc.BF16, M, K)
    xq = orc.fp8_quantize(x, orc.BF16, xs, M, K)
    acc = orc.fp8_gemm(xq, xs, wq, ws)
    bias = orc.to_bits(rng.standard_normal(N).astype(np.float32), orc.BF16)
    import os

    os.environ["KSQ_FP8_FUSED_QUANT"] = "1"
    got = _run_dynamic(gpu, x, wq, ws, "bf16", epilogue=capi.EPILOGUE_BIAS, bias_bits=bias)
    orc.assert_parity(got.float().cpu().numpy(), acc + orc.from_bits(bias, orc.BF16)[None, :], "fp8 dynamic + bias")
    # rows [gate ; up] interleaved gate / up (what ksq_interleave_halves builds): row 2i = gate i, row 2i + 1 = up i
    il = np.empty_like(wq)
    il[0::2], il[1::2] = wq[: N // 2], wq[N // 2:]
    ils = np.empty_like(ws)
    ils[0::2], ils[1::2] = ws[: N // 2], ws[N // 2:]
    got = _run_dynamic(gpu, x, il, ils, "bf16", epilogue=capi.EPILOGUE_SILU_MUL)
    orc.assert_parity(got.float().cpu().numpy(), orc.silu_mul(acc), "fp8 dynamic + SiLU-mul")
    os.environ.pop("KSQ_FP8_FUSED_QUANT", None)
    big = orc.to_bits(rng.standard_normal((12, K)).astype(np.float32), orc.BF16)
    with pytest.raises(capi.KsqError) as e:
        _run_dynamic(gpu, big, wq, ws, "bf16", use_workspace=False)
    assert e.value.code == capi.ERR_WORKSPACE
