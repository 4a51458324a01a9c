"""W4A16 parity tests proper: the HIP path through the C ABI against the CPU oracle on the same seeded bytes.
Bar: max relative error <= 1e-2 (denominator floored at RMS of the oracle output) and mean absolute error
<= 2e-3 x RMS, fp32 accumulation; integer and one-hot cases must match bit for bit."""
import os

import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import ORC_DT, W4Case, W4Device, bits_of

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def _env(**kv):
    class _Ctx:
        def __enter__(self):
            self.old = {k: os.environ.get(k) for k in kv}
            for k, v in kv.items():
                os.environ[k] = str(v)

        def __exit__(self, *a):
            for k, v in self.old.items():
                if v is None:
                    os.environ.pop(k, None)
                else:
                    os.environ[k] = v

    return _Ctx()


@pytest.mark.parametrize("layout", ["gptq", "awq", "rowmajor"])
def test_device_repack_matches_host_repack(gpu, layout):
    from ksanallm_amd import capi

    case = W4Case(100, 4, 512, 96, g=64, kind="awq", dtype="f16")
    dev = W4Device(case, gpu, layout=layout)
    wb, sb = capi.w4a16_repack_sizes(case.K, case.N, case.g)
    hw = np.zeros(wb // 4, dtype=np.uint32)
    hs = np.zeros(sb // 4, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_GPTQ_INT32_KPACK, case.gptq_qweight(), capi.ZERO_UINT8, case.z, case.scales,
                           capi.F16, case.K, case.N, case.g, hw, hs)
    assert np.array_equal(dev.weight.cpu().numpy().view(np.uint32), hw)
    assert np.array_equal(dev.sz.cpu().numpy().view(np.uint32), hs)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("kind,g", [("gptq", 128), ("awq", 128), ("awq", 64)])
def test_one_hot_rows_return_dequantized_rows_exactly(gpu, dtype, kind, g):
    K, N = 512, 128
    rows = [0, 1, 7, 8, 31, 32, 63, 64, 127, 128, 255, 256, 300, 383, 510, 511]
    act = np.zeros((len(rows), K), dtype=np.float32)
    for i, k in enumerate(rows):
        act[i, k] = 1.0
    case = W4Case(101, len(rows), K, N, g=g, kind=kind, dtype=dtype, act=act)
    out = W4Device(case, gpu).gemm()
    want = orc.to_bits(case.dequantized()[rows], ORC_DT[dtype])
    assert np.array_equal(bits_of(out), want)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_integer_case_is_exact(gpu, dtype):
    M, K, N = 7, 256, 64
    rng = np.random.default_rng(102)
    act = rng.integers(-3, 4, size=(M, K)).astype(np.float32)
    case = W4Case(102, M, K, N, kind="awq", dtype=dtype, act=act, scales=np.ones((K // 128, N), dtype=np.float32))
    got = W4Device(case, gpu).gemm_f32()
    want = act.astype(np.int64) @ (case.u.astype(np.int64) - np.repeat(case.z, 128, axis=0).astype(np.int64))
    # the fp32 sums are exact integers; the output rounding to T is the same round-to-nearest-even on both sides
    want_bits = orc.to_bits(want.astype(np.float32), ORC_DT[dtype])
    assert np.array_equal(orc.to_bits(got, ORC_DT[dtype]), want_bits)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 100, 128, 200])
def test_m_sweep_small_shape(gpu, dtype, M):
    case = W4Case(1000 + M, M, 1024, 320, kind="awq", dtype=dtype)
    got = W4Device(case, gpu).gemm_f32()
    orc.assert_parity(got, case.oracle(), f"M={M} {dtype}")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("route", [0, 1])
@pytest.mark.parametrize("M", [17, 32, 33, 48, 64])
def test_m_sweep_both_decode_routes(gpu, dtype, route, M):
    """17 <= M <= 64 is served by the k-stationary kernel (two or four row tiles) or by the accumulator-stationary
    one, chosen per shape: force each."""
    case = W4Case(1050 + M, M, 1024, 320, kind="awq", dtype=dtype)
    with _env(KSQ_W4_ASTREAM=route):
        got = W4Device(case, gpu).gemm_f32()
    orc.assert_parity(got, case.oracle(), f"M={M} {dtype} route={route}")


@pytest.mark.parametrize("dtype,g", [("f16", 128), ("bf16", 64)])
@pytest.mark.parametrize("tpw_max", [1, 2, 3, 4])
@pytest.mark.parametrize("M,K", [(1, 8192), (16, 7168), (9, 2048)])
def test_k_tiles_per_wave(gpu, dtype, g, tpw_max, M, K):
    """One row tile with 1..4 k tiles per wave (a smaller maximum forces a split of K across workgroups; four covers
    K = 8192 inside one workgroup with a ring of a single column tile)."""
    case = W4Case(1400 + K // 128 + M, M, K, 336, g=g, kind="awq", dtype=dtype)
    dev = W4Device(case, gpu)
    with _env(KSQ_W4_KSTAT_TPW_MAX=tpw_max):
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"tpw_max={tpw_max} {dtype} M={M} K={K}")
    assert np.array_equal(got1, got2)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("kind,g", [("gptq", 128), ("gptq", 64), ("awq", 64)])
def test_group_sizes_and_kinds(gpu, dtype, kind, g):
    case = W4Case(1100, 9, 768, 208, g=g, kind=kind, dtype=dtype)
    orc.assert_parity(W4Device(case, gpu).gemm_f32(), case.oracle(), f"{kind} g={g} {dtype}")


@pytest.mark.parametrize("ksplit", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("nt,slices", [(1, 1), (1, 2), (1, 4), (2, 1), (2, 2), (4, 1)])
@pytest.mark.parametrize("dtype,M", [("f16", 16), ("bf16", 33), ("bf16", 7)])
def test_forced_split_k_and_tile_widths(gpu, dtype, M, ksplit, nt, slices):
    case = W4Case(1200 + ksplit, M, 1408, 272, kind="awq", dtype=dtype)  # 11 k tiles, 17 column tiles: ragged
    dev = W4Device(case, gpu)
    import torch

    big = torch.empty(64 << 20, dtype=torch.uint8, device=gpu)
    dev.workspace, dev.workspace_bytes = big, big.numel()
    with _env(KSQ_W4_KSPLIT=ksplit, KSQ_W4_NT=nt, KSQ_W4_SLICES=slices):
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()  # counters must have returned to zero
    want = case.oracle()
    orc.assert_parity(got1, want, f"ksplit={ksplit} nt={nt} slices={slices}")
    assert np.array_equal(got1, got2), "split-K result must be deterministic and repeatable"


@pytest.mark.parametrize("waves,ct", [(4, 4), (8, 4), (4, 3), (8, 3), (4, 2), (8, 2), (4, 1), (8, 1)])
@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 128, 384, 528),    # odd number of k tiles, 33 column tiles: ragged in N for both widths
    ("bf16", "awq", 128, 333, 512, 1040),  # ragged rows, three column blocks of 512
    ("f16", "gptq", 64, 257, 256, 272),    # two groups per k tile
    ("bf16", "gptq", 64, 130, 640, 512),
])
def test_prefill_kernel_widths(gpu, waves, ct, dtype, kind, g, M, K, N):
    """The large-M kernel in its four workgroup widths (four or eight waves side by side, four or three column tiles
    per wave: 128 x 256, 512, 192, 384), whichever the planner would pick."""
    case = W4Case(1250 + waves + M, M, K, N, g=g, kind=kind, dtype=dtype)
    dev = W4Device(case, gpu)
    with _env(KSQ_W4_PREFILL_ROWS=128, KSQ_W4_PREFILL_WAVES=waves, KSQ_W4_PREFILL_CT=ct):
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"prefill waves={waves} {dtype} {kind} g={g} M={M}")
    assert np.array_equal(got1, got2)


@pytest.mark.parametrize("K", [8192, 17408, 28672, 33792])
def test_prefill_bf16_long_rows(gpu, K):
    """bf16 activations on the large-M route are re-encoded row by row as fp16 x 2^e: rows of up to 16384 and up to
    32768 elements stay in registers between the row maximum and the conversion, longer ones are read twice.  Rows
    with very different magnitudes, so that the per-row exponent matters."""
    M, N = 70, 64
    case = W4Case(1250 + K // 128, M, K, N, g=128, kind="gptq", dtype="bf16")
    act = orc.from_bits(case.act, orc.BF16)
    act *= np.exp2(np.random.default_rng(K).integers(-20, 21, size=(M, 1))).astype(np.float32)
    case.act = orc.to_bits(act, orc.BF16)
    dev = W4Device(case, gpu)
    got1 = dev.gemm_f32()
    got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"prefill bf16 rows of {K}")
    assert np.array_equal(got1, got2)


@pytest.mark.parametrize("rows,nt", [(64, 1), (64, 2), (64, 4), (128, 4)])
@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 65, 640, 528),     # five k tiles: the four-deep ring wraps with a remainder
    ("bf16", "awq", 128, 200, 1024, 272),
    ("f16", "gptq", 64, 130, 384, 512),
    ("bf16", "gptq", 64, 96, 128, 256),    # a single k tile
])
def test_prefill_row_tiles(gpu, rows, nt, dtype, kind, g, M, K, N):
    """The large-M path with 64-row (1, 2 or 4 column tiles per wave) and 128-row workgroup tiles, whichever the
    planner would pick."""
    case = W4Case(1260 + rows + M, M, K, N, g=g, kind=kind, dtype=dtype)
    dev = W4Device(case, gpu)
    with _env(KSQ_W4_PREFILL_ROWS=rows, KSQ_W4_PREFILL_NT=nt):
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"prefill rows={rows} {dtype} {kind} g={g} M={M}")
    assert np.array_equal(got1, got2)


@pytest.mark.parametrize("kg,ct", [(1, 4), (2, 4), (2, 3)])
@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 65, 640, 528),      # five k tiles: the second k group's last step has no tile
    ("bf16", "awq", 128, 200, 1024, 272),   # eight k tiles, two row blocks, ragged rows and columns
    ("f16", "gptq", 64, 130, 384, 512),     # three k tiles, two groups per tile
    ("bf16", "gptq", 64, 300, 256, 256),    # two k tiles: one step per k group
])
def test_prefill_128_rows_k_groups(gpu, kg, ct, dtype, kind, g, M, K, N):
    """The 128-row kernel with four waves side by side, as one group or as two groups that take the even and the odd
    k tiles and add their accumulators through LDS at the end (what the planner picks for grids of at most one
    workgroup per compute unit); twice, bit for bit."""
    case = W4Case(1270 + kg + M, M, K, N, g=g, kind=kind, dtype=dtype)
    dev = W4Device(case, gpu)
    with _env(KSQ_W4_PREFILL_ROWS=128, KSQ_W4_PREFILL_WAVES=4, KSQ_W4_PREFILL_KG=kg, KSQ_W4_PREFILL_CT=ct):
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"prefill 128 rows kg={kg} {dtype} {kind} g={g} M={M}")
    assert np.array_equal(got1, got2)


@pytest.mark.parametrize("ksplit,waves,kg,ct", [(2, 4, 2, 4), (3, 4, 2, 3), (8, 4, 1, 4), (2, 8, 1, 3), (5, 4, 2, 4), (4, 4, 2, 2),
                                                (3, 4, 2, 1), (2, 4, 1, 1)])
@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 130, 1152, 528),    # nine k tiles: splits of one to five tiles, odd ones for the two k groups
    ("bf16", "awq", 128, 200, 2048, 272),
    ("f16", "gptq", 64, 128, 4096, 512),
    ("bf16", "gptq", 64, 300, 1024, 256),
])
def test_prefill_128_rows_split_k(gpu, ksplit, waves, kg, ct, dtype, kind, g, M, K, N):
    """The 128-row kernel with K split over workgroups (each split's fp32 tile through the workspace, summed in split
    order by the reduction kernel), in every form of the workgroup; twice, bit for bit, and with a workspace that holds
    no partial tiles."""
    from ksanallm_amd import capi

    case = W4Case(1290 + ksplit + M, M, K, N, g=g, kind=kind, dtype=dtype)
    forms = dict(KSQ_W4_PREFILL_ROWS=128, KSQ_W4_PREFILL_WAVES=waves, KSQ_W4_PREFILL_KG=kg, KSQ_W4_PREFILL_CT=ct)
    with _env(KSQ_W4_PREFILL_KSPLIT=ksplit, **forms):
        dev = W4Device(case, gpu)   # sizes the workspace for the split
        got1 = dev.gemm_f32()
        capi.set_launch_log(True)
        got2 = dev.gemm_f32()
        log = capi.last_launch()
        capi.set_launch_log(False)
    assert f"kg={kg},ct={ct}> grid=(" in log and f",{ksplit})" in log and "w4a16_splitk_reduce_kernel" in log, log
    with _env(KSQ_W4_PREFILL_KSPLIT=1, **forms):
        front = capi.w4a16_workspace_bytes(M, N, K)
    assert dev.workspace_bytes > front
    dev.workspace_bytes = front
    with _env(KSQ_W4_PREFILL_KSPLIT=ksplit, **forms):
        got3 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"prefill 128 rows ksplit={ksplit} kg={kg} ct={ct} {dtype} {kind} g={g} M={M}")
    assert np.array_equal(got1, got2)
    orc.assert_parity(got3, case.oracle(), f"prefill 128 rows one split {dtype} {kind} g={g} M={M}")


@pytest.mark.parametrize("ksplit", [2, 3, 8])
@pytest.mark.parametrize("nt", [1, 4])
@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 65, 1152, 528),     # nine k tiles: splits of one to five tiles, ragged rows and columns
    ("bf16", "awq", 128, 200, 2048, 272),
    ("f16", "gptq", 64, 130, 4096, 512),    # whole groups of four tiles per split (the steady-state loop)
    ("bf16", "gptq", 64, 512, 1024, 256),
])
def test_prefill_split_k(gpu, ksplit, nt, dtype, kind, g, M, K, N):
    """The 64-row large-M kernel with K split over workgroups (fp32 partial tiles through the workspace, summed in split
    order by a second kernel): parity, bit-identical repeats, and the fall-back to one split when the workspace holds
    nothing beyond the bf16 front part."""
    from ksanallm_amd import capi

    case = W4Case(1280 + ksplit + M, M, K, N, g=g, kind=kind, dtype=dtype)
    with _env(KSQ_W4_PREFILL_ROWS=64, KSQ_W4_PREFILL_NT=nt, KSQ_W4_PREFILL_KSPLIT=ksplit):
        dev = W4Device(case, gpu)   # sizes the workspace for the split
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()
    with _env(KSQ_W4_PREFILL_ROWS=64, KSQ_W4_PREFILL_NT=nt, KSQ_W4_PREFILL_KSPLIT=1):
        front = capi.w4a16_workspace_bytes(M, N, K)
    assert dev.workspace_bytes > front
    dev.workspace_bytes = front
    with _env(KSQ_W4_PREFILL_ROWS=64, KSQ_W4_PREFILL_NT=nt, KSQ_W4_PREFILL_KSPLIT=ksplit):
        got3 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"prefill ksplit={ksplit} nt={nt} {dtype} {kind} g={g} M={M}")
    assert np.array_equal(got1, got2)
    orc.assert_parity(got3, case.oracle(), f"prefill one split {dtype} {kind} g={g} M={M}")


@pytest.mark.parametrize("lds", [0, 1])
@pytest.mark.parametrize("cnt", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 17, 640, 528),      # five k tiles over eight waves: three waves idle, odd slices
    ("bf16", "awq", 128, 32, 1152, 272),    # nine k tiles: slices of two with a remainder
    ("f16", "gptq", 64, 33, 384, 512),
    ("bf16", "gptq", 64, 64, 128, 4112),    # a single k tile, more column tiles than compute units
    ("f16", "awq", 64, 48, 2048, 1040),
])
def test_accumulator_stationary_route(gpu, lds, cnt, dtype, kind, g, M, K, N):
    """The 17 <= M <= 64 kernel that keeps only accumulators and streams both operands, with every number of column
    tiles per workgroup (0 = the launcher's own choice) and the activations through registers + lane permutation or
    through LDS; twice, bit for bit."""
    case = W4Case(1300 + cnt + M, M, K, N, g=g, kind=kind, dtype=dtype)
    dev = W4Device(case, gpu)
    env = dict(KSQ_W4_ASTREAM=1, KSQ_W4_ASTREAM_LDS=lds)
    if cnt:
        env["KSQ_W4_ASTREAM_CNT"] = cnt
    with _env(**env):
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"astream cnt={cnt} {dtype} {kind} g={g} M={M}")
    assert np.array_equal(got1, got2)


@pytest.mark.parametrize("lds", [0, 1])
@pytest.mark.parametrize("ksplit", [2, 3, 4])
@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 17, 640, 528),      # five k tiles: splits of one and two tiles, most waves idle
    ("bf16", "awq", 128, 32, 1152, 272),
    ("f16", "gptq", 64, 64, 2048, 1040),
    ("bf16", "gptq", 64, 48, 4096, 272),    # splits of eight to eleven k tiles: odd and even slices per wave
])
def test_accumulator_stationary_split_k(gpu, lds, ksplit, dtype, kind, g, M, K, N):
    """The same kernel with K split over workgroups as well (partial tiles through the workspace, summed in split
    order by the last workgroup to arrive): parity, bit-identical repeats (the arrival counters return to zero), and
    the fall-back to one split when the caller gives no workspace."""
    case = W4Case(1340 + ksplit + M, M, K, N, g=g, kind=kind, dtype=dtype)
    with _env(KSQ_W4_ASTREAM=1, KSQ_W4_ASTREAM_LDS=lds, KSQ_W4_ASTREAM_KSPLIT=ksplit):
        dev = W4Device(case, gpu)   # sizes the workspace for the split
        assert dev.workspace_bytes >= ksplit * (N // 16) * (2 if M <= 32 else 4) * 1024
        got1 = dev.gemm_f32()
        got2 = dev.gemm_f32()
        got3 = dev.gemm_f32(use_workspace=False)
    orc.assert_parity(got1, case.oracle(), f"astream ksplit={ksplit} {dtype} {kind} g={g} M={M}")
    assert np.array_equal(got1, got2)
    orc.assert_parity(got3, case.oracle(), f"astream no workspace {dtype} {kind} g={g} M={M}")


@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "awq", 128, 40, 2304, 1040),     # 18 k tiles, 65 column tiles, four row tiles: K split in two by the planner
    ("bf16", "gptq", 64, 24, 10240, 272),    # 80 k tiles with two row tiles: split
    ("f16", "gptq", 128, 24, 2048, 4112),    # one column tile per CU and a bit: activations through registers
    ("bf16", "awq", 128, 64, 1152, 16400),   # four tiles per workgroup: activations through LDS, bf16 with CNT = 4
    ("f16", "awq", 128, 100, 12288, 528),    # M >= 65, K >= 96 M: the 64-row kernel with K split in two
    ("bf16", "gptq", 128, 128, 12288, 272),
])
def test_planner_choices_without_overrides(gpu, dtype, kind, g, M, K, N):
    """Shapes picked so that the launch planners, left alone, take the split-K and LDS forms of the kernels for
    17 <= M <= 64 and the split-K form of the 64-row large-M kernel; twice, bit for bit, and without a workspace."""
    case = W4Case(1400 + M + N, M, K, N, g=g, kind=kind, dtype=dtype)
    dev = W4Device(case, gpu)
    got1 = dev.gemm_f32()
    got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"planner {dtype} {kind} g={g} M={M} K={K} N={N}")
    assert np.array_equal(got1, got2)
    if not (dtype == "bf16" and M >= 65):  # the bf16 large-M route needs its workspace and falls back to a slower kernel
        orc.assert_parity(dev.gemm_f32(use_workspace=False), case.oracle(), f"planner, no workspace {dtype} M={M}")


@pytest.mark.parametrize("dtype,kind,g,M,K,N", [
    ("f16", "gptq", 128, 512, 11008, 4096),   # Llama-2-7B down: 64 workgroups of 128 x 256, K split in four
    ("bf16", "awq", 128, 256, 8192, 8192),    # Llama-3-70B o
    ("f16", "awq", 128, 200, 4096, 12288),    # Llama-2-7B qkv, ragged rows: 192 tiles of 128 x 128, no split
    ("bf16", "gptq", 128, 96, 4096, 4096),    # Llama-2-7B o, one row block: 128 x 64 tiles, K split
])
def test_planner_splits_k_over_128_row_tiles(gpu, dtype, kind, g, M, K, N):
    """Full-size shapes with few output tiles, where the planner, left alone, takes the 128-row kernel in its
    one-workgroup-per-CU form, with K split over workgroups where K is long; twice, bit for bit."""
    from ksanallm_amd import capi

    case = W4Case(1450 + M, M, K, N, g=g, kind=kind, dtype=dtype)
    dev = W4Device(case, gpu)
    got1 = dev.gemm_f32()
    capi.set_launch_log(True)
    got2 = dev.gemm_f32()
    log = capi.last_launch()
    capi.set_launch_log(False)
    assert "w4a16_prefill_kernel" in log and "kg=2" in log, log
    if K >= 8192:
        assert "w4a16_splitk_reduce_kernel" in log, log
    orc.assert_parity(got1, case.oracle(), f"planner, 128-row split {dtype} {kind} M={M} K={K} N={N}")
    assert np.array_equal(got1, got2)


def _random_w4_shapes(seed, count):
    """Shapes of a seeded random walk over what the planners distinguish: every family of M, widths from one column
    tile to a few thousand columns (ragged last workgroups included), K from one k tile up, both group sizes (K = 64 x
    odd with g = 64), both layouts and element types."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        M = int(rng.choice([rng.integers(1, 17), rng.integers(17, 33), rng.integers(33, 65), rng.integers(65, 300)]))
        N = 16 * int(rng.choice([rng.integers(1, 9), rng.integers(9, 140)]))
        g = int(rng.choice([64, 128]))
        K = g * int(rng.choice([rng.integers(1, 5), rng.integers(5, 20)]))
        if K % 128 == 64 and g == 128:
            K += 64
        out.append((M, K, N, g, str(rng.choice(["awq", "gptq"])), str(rng.choice(["f16", "bf16"]))))
    return out


@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16])
def test_random_shapes(gpu, seed):
    """Twelve shapes per seed from a seeded random walk (and, with the first seed, the shape that used to read past the
    weights: one k tile under the two-row-tile decode kernel), each through the planner's own choice with a workspace
    and without one, against the oracle."""
    shapes = _random_w4_shapes(seed, 12)
    if seed == 11:
        shapes += [(24, 128, 272, 128, "awq", "f16"), (32, 128, 16, 64, "gptq", "bf16")]
    for i, (M, K, N, g, kind, dtype) in enumerate(shapes):
        case = W4Case(3000 + 100 * seed + i, M, K, N, g=g, kind=kind, dtype=dtype)
        dev = W4Device(case, gpu)
        want = case.oracle()
        orc.assert_parity(dev.gemm_f32(), want, f"random seed {seed} #{i}: M={M} K={K} N={N} g={g} {kind} {dtype}")
        if K % 128 == 0 and not (dtype == "bf16" and M >= 65):  # K = 64 x odd needs the padded copy in the workspace
            orc.assert_parity(dev.gemm_f32(use_workspace=False), want, f"random seed {seed} #{i}, no workspace")


def test_prefill_bf16_row_magnitudes(gpu):
    """bf16 activations go through a per-row power-of-two re-encoding on the large-M route: rows of very different
    magnitude (up to 2^100, down to 2^-60, an all-zero row) must each keep full relative accuracy."""
    M, K, N = 160, 512, 256
    rng = np.random.default_rng(1270)
    act = rng.standard_normal((M, K)).astype(np.float32)
    exps = rng.integers(-60, 101, size=M)
    act *= np.exp2(exps.astype(np.float64)).astype(np.float32)[:, None]
    act[7, :] = 0.0
    case = W4Case(1271, M, K, N, kind="awq", dtype="bf16", act=act)
    got = W4Device(case, gpu).gemm_f32()
    want = case.oracle()
    assert np.all(got[7] == 0.0)
    for row in range(M):  # every row against its own scale
        if row != 7:
            orc.assert_parity(got[row:row + 1], want[row:row + 1], f"row {row} (2^{exps[row]})")


@pytest.mark.parametrize("M", [16, 65, 600])
def test_bf16_scales_far_outside_the_fp16_range(gpu, M):
    """bf16 group scales from 1e-6 to 1e5, different per column block and with a wide spread inside some columns: the
    decode kernels (M = 16) keep scales in fp32, the 64-row and 128-row kernels (M = 65, 600) run their matrix
    instructions in fp16 and must still be right, column block by column block."""
    K, N = 1024, 1024
    rng = np.random.default_rng(1290 + M)
    G = K // 128
    base = np.repeat(np.array([1e-6, 3e-5, 1e-3, 0.02, 7.0, 3e3, 1e5, 2e-2], dtype=np.float32), N // 8)[None, :]
    sv = base * (1 + rng.random((G, N), dtype=np.float32))
    sv[:, -128:] *= np.exp2(rng.integers(-10, 1, size=(G, 128))).astype(np.float32)  # spread inside a column
    case = W4Case(1291, M, K, N, kind="awq", dtype="bf16", scales=sv)
    got = W4Device(case, gpu).gemm_f32()
    want = case.oracle()
    assert np.all(np.isfinite(got))
    for b in range(8):
        cols = slice(b * N // 8, (b + 1) * N // 8)
        orc.assert_parity(got[:, cols], want[:, cols], f"M={M} column block {b} (scale ~ {base[0, b * N // 8]:g})")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("kind", ["awq", "gptq"])
@pytest.mark.parametrize("M,K,N", [(1, 192, 272), (16, 1088, 528), (40, 448, 1040), (100, 1088, 272), (600, 704, 512)])
def test_k_odd_multiple_of_64(gpu, dtype, kind, M, K, N):
    """Group size 64 with K = 64 * odd, which the reference's kernels accept (k % 64 == 0): the repack pads the last
    k tile, the GEMM pads the activation rows in its workspace; every kernel family by M; without a workspace the
    call must refuse."""
    from ksanallm_amd import capi

    case = W4Case(1500 + M + K, M, K, N, g=64, kind=kind, dtype=dtype)
    dev = W4Device(case, gpu)
    assert dev.workspace_bytes >= M * (K + 64) * 2
    got1 = dev.gemm_f32()
    got2 = dev.gemm_f32()
    orc.assert_parity(got1, case.oracle(), f"K={K} g=64 {kind} {dtype} M={M}")
    assert np.array_equal(got1, got2)
    with pytest.raises(capi.KsqError) as e:
        dev.gemm(use_workspace=False)
    assert e.value.code == capi.ERR_WORKSPACE


@pytest.mark.parametrize("dtype,g", [("f16", 128), ("bf16", 64), ("f16", 64), ("bf16", 128)])
@pytest.mark.parametrize("M,K,N", [(1, 256, 272), (3, 2176, 528), (4, 4224, 272), (5, 2176, 1040), (8, 8320, 272),
                                   (2, 384, 4112), (7, 640, 8208), (4, 384, 12304), (1, 256, 16)])
def test_k_phases_inside_the_workgroup(gpu, dtype, g, M, K, N):
    """One to eight rows with K walked in phases inside the workgroup (what long K gets instead of a split across
    workgroups): whole and partial last phases, one to four column tiles per workgroup, a ragged last workgroup; no
    workspace needed; two runs bit for bit."""
    from ksanallm_amd import capi

    case = W4Case(1900 + M + K // 128, M, K, N, g=g, kind="awq", dtype=dtype)
    dev = W4Device(case, gpu)
    capi.set_launch_log(True)
    try:
        with _env(KSQ_W4_KPHASE=1):
            got1 = dev.gemm_f32(use_workspace=False)
            assert "w4a16_kphase_kernel" in capi.last_launch(), capi.last_launch()
            got2 = dev.gemm_f32()
    finally:
        capi.set_launch_log(False)
    orc.assert_parity(got1, case.oracle(), f"k phases M={M} K={K} N={N} {dtype} g={g}")
    assert np.array_equal(got1, got2)


def test_caller_bound_split_k_counters_and_launch_log(gpu):
    """Split-K with the arrival counters in the caller's memory: same bits as with the library's, the memory is back at
    zero after every launch, and the launch log names the kernel and its split."""
    import torch

    from ksanallm_amd import capi

    case = W4Case(1777, 16, 1408, 272, kind="awq", dtype="f16")
    dev = W4Device(case, gpu)
    big = torch.empty(8 << 20, dtype=torch.uint8, device=gpu)
    dev.workspace, dev.workspace_bytes = big, big.numel()
    capi.set_launch_log(True)
    try:
        with _env(KSQ_W4_KSPLIT=3):
            ref = dev.gemm_f32()
            assert "w4a16_kstat_kernel" in capi.last_launch() and ",3)" in capi.last_launch(), capi.last_launch()
            mine = torch.zeros(capi.SPLITK_COUNTER_BYTES + 256, dtype=torch.uint8, device=gpu)
            mine = mine[(-mine.data_ptr()) % 256:][:capi.SPLITK_COUNTER_BYTES]
            capi.bind_splitk_counters(None, mine)
            try:
                got1, got2 = dev.gemm_f32(), dev.gemm_f32()
            finally:
                capi.bind_splitk_counters(None, None)
            again = dev.gemm_f32()
    finally:
        capi.set_launch_log(False)
    assert int(mine.to(torch.int32).abs().sum().item()) == 0, "the counters did not return to zero"
    assert np.array_equal(ref, got1) and np.array_equal(ref, got2) and np.array_equal(ref, again)
    orc.assert_parity(ref, case.oracle(), "bound counters")
    with pytest.raises(capi.KsqError):
        capi.bind_splitk_counters(None, mine, 1024)  # too small


def test_no_workspace_still_correct(gpu):
    case = W4Case(1300, 16, 4096, 512, kind="gptq", dtype="f16")
    dev = W4Device(case, gpu)
    a = dev.gemm_f32(use_workspace=True)
    b = dev.gemm_f32(use_workspace=False)
    want = case.oracle()
    orc.assert_parity(a, want, "with workspace")
    orc.assert_parity(b, want, "without workspace")


def test_config0_gptq_m16_4096x4096(gpu):
    case = W4Case(0, 16, 4096, 4096, kind="gptq", dtype="f16")
    m = orc.assert_parity(W4Device(case, gpu).gemm_f32(), case.oracle(), "cfg0")
    print("cfg0 metrics", m)


SHAPES_7B = [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]


@pytest.mark.parametrize("K,N", SHAPES_7B)
def test_config1_awq_decode_sweep(gpu, K, N):
    import torch

    case = W4Case(1000 + K + N, 64, K, N, kind="awq", dtype="f16")
    dev = W4Device(case, gpu)
    want = case.oracle()
    for M in (1, 4, 16, 64):
        got = dev.gemm(act=dev.act[:M].contiguous()).float().cpu().numpy()
        orc.assert_parity(got, want[:M], f"cfg1 K={K} N={N} M={M}")
    del dev
    torch.cuda.empty_cache()


@pytest.mark.parametrize("K,N", [(4096, 4096), (11008, 4096)])
def test_config2_awq_bf16_prefill_rows_subset(gpu, K, N):
    """M = 512 through the product path; the oracle checks a seeded subset of rows (the full product is the
    bench's job)."""
    case = W4Case(2000 + K + N, 512, K, N, kind="awq", dtype="bf16")
    got = W4Device(case, gpu).gemm_f32()
    rows = np.random.default_rng(5).choice(512, size=24, replace=False)
    rows.sort()
    orc.assert_parity(got[rows], case.oracle(rows=rows), f"cfg2 K={K} N={N}")


@pytest.mark.parametrize("K,N", [(8192, 8192), (28672, 8192)])
def test_config3_gptq_70b_rows_subset(gpu, K, N):
    """The o and down projections of Llama-2-70B (configs[3]) at M = 32, 64 and 256 through the product path: these
    are the shapes where the planners split K over workgroups for 17 <= M <= 64 and (down, M = 256) in the 64-row
    large-M kernel.  The oracle checks a seeded subset of rows."""
    import torch

    case = W4Case(3000 + K + N, 256, K, N, kind="gptq", dtype="f16")
    dev = W4Device(case, gpu)
    rows = np.unique(np.concatenate([[3, 20, 40, 60], np.random.default_rng(6).choice(256, size=8, replace=False)]))
    want = case.oracle(rows=rows)
    for M in (32, 64, 256):
        sel = rows[rows < M]
        got = dev.gemm(act=dev.act[:M].contiguous()).float().cpu().numpy()
        orc.assert_parity(got[sel], want[: len(sel)], f"cfg3 K={K} N={N} M={M}")
    del dev
    torch.cuda.empty_cache()


def test_linearity_at_full_size(gpu):
    """Size-independent property at a full 7B shape: f(a + b) = f(a) + f(b) when a, b and a + b are exactly
    representable and the fp16 results do not round differently (integer activations, unit scales)."""
    K, N, M = 4096, 12288, 16
    rng = np.random.default_rng(7)
    # sparse {-1,0,1} activations keep every |sum| far below 2^11 units, where fp16 is exact
    a = (rng.integers(-1, 2, size=(M, K)) * (rng.random((M, K)) < 0.25)).astype(np.float32)
    b = (rng.integers(-1, 2, size=(M, K)) * (rng.random((M, K)) < 0.25)).astype(np.float32)
    ones = np.full((K // 128, N), 2.0**-6, dtype=np.float32)
    ca = W4Case(7, M, K, N, kind="awq", dtype="f16", act=a, scales=ones)
    dev = W4Device(ca, gpu)
    import torch

    def run(x):
        t = torch.from_numpy(orc.to_bits(x, orc.F16).view(np.int16)).to(gpu).view(torch.float16)
        return dev.gemm(act=t).float().cpu().numpy().astype(np.float64)

    fa, fb, fab = run(a), run(b), run(a + b)
    # every value is an integer multiple of 2^-6 below 2^11 * 2^-6, so all three are exact
    assert np.array_equal(fa + fb, fab)
