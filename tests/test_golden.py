"""The oracle against the committed golden vectors of tests/golden (written by tests/golden/make_fixtures.py from an
independent numpy statement of the formats; no GPU needed)."""
import os

import numpy as np
import pytest

from oracle import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
W4_CASES = ["w4a16_gptq_f16_16x256x128", "w4a16_awq_f16_5x256x64_g64", "w4a16_awq_bf16_16x384x128",
            "w4a16_awq_bf16_130x256x272"]


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
