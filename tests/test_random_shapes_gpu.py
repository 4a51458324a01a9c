"""Seeded random shapes around the launch planners' thresholds (row counts either side of every kernel boundary, narrow
and wide N, short and long K, both group sizes, both element types), through the C ABI against the oracle: parity,
every output element written, two runs bit for bit.  Large cases compare a subset of rows."""
import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import W4Case, W4Device

pytestmark = pytest.mark.gpu

W4_M = [1, 3, 4, 5, 8, 9, 16, 17, 31, 32, 33, 40, 47, 48, 49, 63, 64, 65, 66, 100, 127, 128, 129, 191, 200, 256, 257,
        300, 511, 513, 640, 1000]
W4_N = [16, 48, 256, 272, 1040, 4096, 4112, 8192, 16384, 16400, 22016]
W4_K = [128, 256, 384, 640, 1024, 2048, 4096]
FP8_M = [1, 2, 4, 5, 8, 16, 17, 31, 32, 33, 48, 49, 64, 65, 100, 127, 128, 129, 255, 256, 257, 300, 511, 512, 600, 1030]
FP8_N = [8, 64, 256, 272, 544, 4104, 6144, 8192, 16384, 16392, 24576]
FP8_K = [128, 256, 1024, 1152, 4096, 8192, 9600]


@pytest.mark.parametrize("seed", range(6))
def test_w4a16_random_shapes(gpu, seed):
    rng = np.random.default_rng(9000 + seed)
    done = 0
    while done < 14:
        M, N, K = int(rng.choice(W4_M)), int(rng.choice(W4_N)), int(rng.choice(W4_K))
        if M * K * N > 4e9:
            continue
        g, kind, dtype = int(rng.choice([64, 128])), str(rng.choice(["awq", "gptq"])), str(rng.choice(["f16", "bf16"]))
        what = f"random w4a16 M={M} K={K} N={N} g={g} {kind} {dtype}"
        print(what, flush=True)
        case = W4Case(int(rng.integers(1 << 30)), M, K, N, g=g, kind=kind, dtype=dtype)
        dev = W4Device(case, gpu)
        got, again = dev.gemm_f32(), dev.gemm_f32()
        assert not np.isnan(got).any(), what + ": output not fully written"
        assert np.array_equal(got, again), what + ": two runs differ"
        if M * K * N > 1e9:
            rows = np.unique(rng.choice(M, size=min(M, 24), replace=False))
            orc.assert_parity(got[rows], case.oracle(rows=rows), what)
        else:
            orc.assert_parity(got, case.oracle(), what)
        done += 1


@pytest.mark.parametrize("seed", range(4))
def test_fp8_random_shapes(gpu, seed):
    from tests.test_fp8_gpu import _run_gemm

    rng = np.random.default_rng(9100 + seed)
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    done = 0
    while done < 12:
        M, N, K = int(rng.choice(FP8_M)), int(rng.choice(FP8_N)), int(rng.choice(FP8_K))
        if M * K * N > 6e9:
            continue
        per_channel, dtype = bool(rng.integers(2)), str(rng.choice(["f16", "bf16"]))
        what = f"random fp8 M={M} K={K} N={N} per_channel={per_channel} {dtype}"
        print(what, flush=True)
        # random e4m3 codes with the top exponent bit cleared, so that the sums stay inside fp16
        xq = codes[rng.integers(0, len(codes), size=(M, K))] & np.uint8(0xBF)
        wq = codes[rng.integers(0, len(codes), size=(N, K))] & np.uint8(0xBF)
        xs = ((rng.random(M if per_channel else 1) + 0.5) * 1e-2).astype(np.float32)
        ws = ((rng.random(N if per_channel else 1) + 0.5) * 1e-2).astype(np.float32)
        got, again = _run_gemm(gpu, xq, xs, wq, ws, dtype), _run_gemm(gpu, xq, xs, wq, ws, dtype)
        assert not np.isnan(got).any(), what + ": output not fully written"
        assert np.array_equal(got, again), what + ": two runs differ"
        if M * K * N > 1e9:
            rows = np.unique(rng.choice(M, size=min(M, 16), replace=False))
            orc.assert_parity(got[rows], orc.fp8_gemm(xq[rows], xs[rows] if per_channel else xs, wq, ws), what)
        else:
            orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), what)
        done += 1
