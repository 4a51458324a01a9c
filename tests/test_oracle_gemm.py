"""Pins the oracle's dequantize-then-GEMM: integer cases that are exact in fp32, one-hot activations that
return dequantized rows exactly, an fp64-accumulated product, and numpy's matmul."""
import numpy as np

from oracle import oracle as orc


def test_integer_case_is_exact():
    rng = np.random.default_rng(11)
    M, K, N, g = 5, 256, 32, 128
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    a_int = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
    ones = orc.to_bits(np.ones((K // g, N), dtype=np.float32), orc.F16)
    out = orc.w4a16_forward(orc.to_bits(a_int, orc.F16), orc.F16, u, ones, orc.F16, None, g)
    want = a_int.astype(np.int64) @ (u.astype(np.int64) - 8)
    assert np.array_equal(out.astype(np.int64), want)


def test_one_hot_rows_return_dequantized_rows():
    rng = np.random.default_rng(12)
    K, N, g = 256, 64, 128
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = orc.to_bits(np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3, orc.BF16)
    rows = [0, 1, 127, 128, 255]
    a = np.zeros((len(rows), K), dtype=np.float32)
    for i, k in enumerate(rows):
        a[i, k] = 1.0
    out = orc.w4a16_forward(orc.to_bits(a, orc.BF16), orc.BF16, u, s, orc.BF16, z, g)
    w = orc.dequant(u, s, orc.BF16, z, g)
    assert np.array_equal(out, w[rows])


def test_gemm_against_fp64_and_numpy():
    rng = np.random.default_rng(13)
    M, K, N = 16, 512, 300  # N not a multiple of the oracle's block
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    out = orc.gemm_f32(a, w)
    ref64 = a.astype(np.float64) @ w.astype(np.float64)
    assert np.allclose(orc.gemm_f64acc(a, w), ref64, rtol=1e-12, atol=1e-12)
    m = orc.error_metrics(out, ref64)
    assert m["max_rel"] < 1e-5 and m["mean_abs_over_rms"] < 1e-6


def test_gemm_ragged_m():
    rng = np.random.default_rng(14)
    for M in (1, 3, 17, 33):
        a = rng.standard_normal((M, 128)).astype(np.float32)
        w = rng.standard_normal((128, 16)).astype(np.float32)
        assert np.allclose(orc.gemm_f32(a, w), a @ w, rtol=1e-4, atol=1e-4)


def test_error_metric_definition():
    want = np.array([1.0, -1.0, 0.0, 2.0])
    got = np.array([1.0, -1.0, 0.1, 2.0])
    m = orc.error_metrics(got, want)
    rms = np.sqrt(6.0 / 4.0)
    assert abs(m["max_rel"] - 0.1 / rms) < 1e-12
    assert abs(m["mean_abs_over_rms"] - (0.1 / 4) / rms) < 1e-12
