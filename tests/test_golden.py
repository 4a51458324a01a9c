"""The oracle against the committed golden vectors of tests/golden (written by tests/golden/make_fixtures.py from an
independent numpy statement of the formats; no GPU needed)."""
import os

import numpy as np
import pytest

from oracle import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
W4_CASES = ["w4a16_gptq_f16_16x256x128", "w4a16_awq_f16_5x256x64_g64", "w4a16_awq_bf16_16x384x128",
            "w4a16_awq_bf16_130x256x272", "w4a16_gptq_f16_7x192x64_g64", "w4a16_awq_bf16_9x256x64_wide"]


def load(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"))


def test_gptq_layout_vectors():
    f = load("gptq_64x64")
    assert np.array_equal(orc.gptq_unpack(f["qweight"]), f["u"])
    assert np.array_equal(orc.gptq_pack(f["u"]), f["qweight"])
    assert np.array_equal(orc.rowmajor_pack(f["u"]).view(np.uint8), f["rowmajor"].view(np.uint8))
    assert np.array_equal(orc.rowmajor_unpack(f["rowmajor"].view(np.uint8)), f["u"])


def test_awq_layout_vectors():
    f = load("awq_128x64")
    assert np.array_equal(orc.awq_unpack(f["qweight"]), f["u"])
    assert np.array_equal(orc.awq_unpack(f["qzeros"]), f["z"])
    assert np.array_equal(orc.awq_pack(f["u"]), f["qweight"])
    assert np.array_equal(orc.rowmajor_unpack(f["rowmajor"].view(np.uint8)), f["u"])


def test_e4m3_table():
    want = load("e4m3_table")["value"]
    got = orc.e4m3_decode(np.arange(256, dtype=np.uint8)).astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok])
    # every finite code is a fixed point of encode(decode(.)) apart from the sign of zero handled explicitly
    codes = np.arange(256, dtype=np.uint8)[ok]
    assert np.array_equal(orc.e4m3_encode(want[ok].astype(np.float32)), codes)


@pytest.mark.parametrize("name", W4_CASES)
def test_w4a16_vectors(name):
    f = load(name)
    dt = orc.BF16 if int(f["bf16"]) else orc.F16
    g = int(f["group"])
    if "qzeros" in f.files:
        u, z = orc.awq_unpack(f["qweight"]), orc.awq_unpack(f["qzeros"])
        assert np.array_equal(z, f["z"])
    else:
        u, z = orc.gptq_unpack(f["qweight"]), None
    assert np.array_equal(u, f["u"])
    got = orc.w4a16_forward(f["act_bits"], dt, u, f["scales_bits"], dt, z, g)
    want = f["out"]
    # fp32 accumulation of the oracle against the float64 truth: far inside the parity bar
    m = orc.error_metrics(got, want)
    assert m["max_rel"] < 2e-5 and m["mean_abs_over_rms"] < 2e-6, m


def test_fp8_vectors():
    f = load("fp8_8x256x64")
    m, k = f["x_bits"].shape
    scale = orc.fp8_compute_scale(f["x_bits"], orc.F16, m, k)
    assert np.array_equal(scale, f["a_scale"])
    assert np.array_equal(orc.fp8_quantize(f["x_bits"], orc.F16, scale, m, k), f["aq"])
    got = orc.fp8_gemm(f["aq"], f["a_scale"], f["wq"], f["w_scale"])
    met = orc.error_metrics(got, f["out"])
    assert met["max_rel"] < 2e-5 and met["mean_abs_over_rms"] < 2e-6, met


def test_next_layout_vectors():
    """The oracle's restatements of the CUTLASS preprocessor, the Marlin repack kernels and permutations and the
    desc_act ordering against vectors written by whole-array numpy reshapes; and the library's host repack reading
    every one of those layouts back to the same fragment order."""
    from ksanallm_amd import capi

    f = load("w4a16_next_f16_12x256x128")
    u, z, sb = f["u"], f["z"], f["scales_bits"]
    K, N = u.shape
    g = int(f["group"])
    rowmajor = orc.rowmajor_pack(u)
    assert np.array_equal(orc.cutlass_preprocess(rowmajor, 80), f["cutlass80"])
    assert np.array_equal(orc.cutlass_preprocess(rowmajor, 90), f["cutlass90"])
    assert np.array_equal(orc.marlin_repack(f["qweight_gptq"], K, N, "gptq"), f["marlin"])
    assert np.array_equal(orc.marlin_repack(f["qweight_awq"], K, N, "awq"), f["marlin"])
    assert np.array_equal(orc.marlin_permute_scales(sb, K, g), f["marlin_scales_bits"])
    assert np.array_equal(orc.marlin_zero_points(z), f["marlin_zp"])
    assert np.array_equal(orc.act_order_perm(f["g_idx"]), f["perm"])
    perm = np.empty(K, dtype=np.int32)
    capi.gptq_act_order_perm(f["g_idx"], K, g, perm)
    assert np.array_equal(perm, f["perm"])

    want_w = np.zeros(K * N // 8, dtype=np.uint32)
    want_sz = np.zeros((K // g) * N, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_AWQ_INT32_NPACK, f["qweight_awq"], capi.ZERO_AWQ_INT32, f["qzeros_awq"], sb, capi.F16,
                           K, N, g, want_w, want_sz)
    for layout, src, zk, zsrc, scales in [
        (capi.W4_CUTLASS_SM80_INTERLEAVED, f["cutlass80"], capi.ZERO_UINT8, z, sb),
        (capi.W4_CUTLASS_SM90_COLMAJOR, f["cutlass90"], capi.ZERO_UINT8, z, sb),
        (capi.W4_MARLIN, f["marlin"], capi.ZERO_MARLIN_INT32, f["marlin_zp"], f["marlin_scales_bits"]),
    ]:
        got_w, got_sz = np.zeros_like(want_w), np.zeros_like(want_sz)
        capi.w4a16_repack_host(layout, np.ascontiguousarray(src), zk, np.ascontiguousarray(zsrc),
                               np.ascontiguousarray(scales), capi.F16, K, N, g, got_w, got_sz)
        assert np.array_equal(got_w, want_w), layout
        assert np.array_equal(got_sz, want_sz), layout


def test_next_output_vectors():
    f = load("w4a16_next_f16_12x256x128")
    g = int(f["group"])
    acc = orc.w4a16_forward(f["act_bits"], orc.F16, f["u"], f["scales_bits"], orc.F16, f["z"], g)
    for got, want in [(acc, f["out"]), (orc.silu_mul(acc), f["out_silu"]),
                      (acc + orc.from_bits(f["bias_bits"], orc.F16)[None, :], f["out_bias"])]:
        m = orc.error_metrics(got, want)
        assert m["max_rel"] < 5e-5 and m["mean_abs_over_rms"] < 5e-6, m
