"""Pins the oracle's e4m3 codec and FP8 scale / quantize / rescale / GEMM: the OCP closed form over all 256
codes, torch.float8_e4m3fn CPU casts as an independent library routine, and the closed forms the reference's
own unit test asserts (LU/utils_test.cu:49-56, 93-99, 136-141) on the shapes that test uses."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

REF_SHAPES = [(1, 31), (1, 16383), (16383, 7), (7, 16383), (16383, 1), (31, 1)]  # LU/utils_test.cu:30,64


def _ocp_value(code):
    s = -1.0 if code & 0x80 else 1.0
    e = (code >> 3) & 0xF
    m = code & 7
    if e == 15 and m == 7:
        return float("nan")
    if e == 0:
        return s * m * 2.0**-9
    return s * (1 + m / 8.0) * 2.0 ** (e - 7)


def test_decode_all_codes_closed_form_and_torch():
    codes = np.arange(256, dtype=np.uint8)
    got = orc.e4m3_decode(codes)
    want = np.array([_ocp_value(int(c)) for c in codes], dtype=np.float32)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok])
    t = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(got[ok], t[ok])
    assert np.signbit(got[0x80]) and got[0x80] == 0.0
    assert got[0x7E] == 448.0 and got[0x01] == 2.0**-9 and got[0x08] == 2.0**-6


def test_encode_roundtrip_and_nearest_even():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    vals = orc.e4m3_decode(codes)
    assert np.array_equal(orc.e4m3_encode(vals), codes)
    pos = np.sort(vals[vals >= 0])
    mids = (pos[:-1] + pos[1:]) / 2  # exact in fp32
    enc = orc.e4m3_decode(orc.e4m3_encode(mids))
    for lo, hi, e in zip(pos[:-1], pos[1:], enc):
        c_lo = int(orc.e4m3_encode(np.array([lo]))[0])
        assert e == (lo if c_lo % 2 == 0 else hi)  # tie goes to the even code
    assert orc.e4m3_encode(np.array([np.nan], dtype=np.float32))[0] & 0x7F == 0x7F
    for v in (448.0, 463.9, 464.0, 1e9, np.inf):
        assert orc.e4m3_encode(np.array([v], dtype=np.float32))[0] == 0x7E
        assert orc.e4m3_encode(np.array([-v], dtype=np.float32))[0] == 0xFE


def test_encode_matches_torch_on_dense_sweep():
    rng = np.random.default_rng(21)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 100,
        rng.standard_normal(20000).astype(np.float32),
        rng.standard_normal(20000).astype(np.float32) * 0.01,
        np.linspace(-448, 448, 40001, dtype=np.float32),
        np.linspace(-2.0**-5, 2.0**-5, 4097, dtype=np.float32),
    ])
    x = np.clip(x, -448, 448)  # torch's cast does not saturate; the reference clamps first
    got = orc.e4m3_encode(x)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    same = got == want
    # -0 vs +0 for tiny negatives is the only allowed representation difference
    assert np.all(same | ((got & 0x7F) == 0) & ((want & 0x7F) == 0))


@pytest.mark.parametrize("shape", REF_SHAPES)
def test_scale_and_quantize_closed_forms(shape):
    rng = np.random.default_rng(22)
    C, L = shape
    x = (rng.random((C, L), dtype=np.float32) * 0.2 - 0.1).astype(np.float16)  # the reference test's range
    xb = x.view(np.uint16)
    s = orc.fp8_compute_scale(xb, orc.F16, C, L)
    want = np.maximum(np.abs(x.astype(np.float32)).max(axis=1) / np.float32(448.0), np.float32(1.0 / 448.0 / 512.0))
    assert np.allclose(s, want, rtol=1e-6, atol=0)
    sc = (rng.random(C, dtype=np.float32) * (1 - 1 / 448 / 512) + 1 / 448 / 512).astype(np.float32)
    q = orc.fp8_quantize(xb, orc.F16, sc, C, L)
    v = np.clip(x.astype(np.float32) / sc[:, None], -448, 448).astype(np.float32)
    want_q = torch.from_numpy(v).to(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(orc.e4m3_decode(q), want_q)


def test_min_scale_floor():
    z = np.zeros((2, 8), dtype=np.float16).view(np.uint16)
    assert np.array_equal(orc.fp8_compute_scale(z, orc.F16, 2, 8), np.full(2, np.float32(1.0) / 448 / 512, np.float32))


@pytest.mark.parametrize("n", [1, 7, 31, 16383])
def test_rescale_closed_form(n):
    rng = np.random.default_rng(23)
    q = rng.integers(0, 256, size=n, dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0x10
    s_in, s_out = np.float32(0.37), np.float32(0.11)
    got = orc.e4m3_decode(orc.fp8_rescale(q, s_in, s_out))
    v = np.clip(orc.e4m3_decode(q) * np.float32(s_in / s_out), -448, 448).astype(np.float32)
    want = torch.from_numpy(v).to(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(got, want)


def test_fp8_gemm_exact_products_and_scale_order():
    rng = np.random.default_rng(24)
    M, K, N = 4, 64, 8
    aq = rng.integers(0, 0x78, size=(M, K), dtype=np.uint8)
    wq = (rng.integers(0, 0x50, size=(N, K), dtype=np.uint8) | (rng.integers(0, 2, size=(N, K), dtype=np.uint8) << 7))
    a = orc.e4m3_decode(aq).astype(np.float64)
    w = orc.e4m3_decode(wq).astype(np.float64)
    xs = rng.random(M, dtype=np.float32) + 0.5
    ws = rng.random(N, dtype=np.float32) + 0.5
    got = orc.fp8_gemm(aq, xs, wq, ws)
    want = (a @ w.T) * ws[None, :].astype(np.float64) * xs[:, None].astype(np.float64)
    assert np.allclose(got, want, rtol=2e-6, atol=0)
    got1 = orc.fp8_gemm(aq, xs[:1], wq, ws[:1])
    assert np.allclose(got1, (a @ w.T) * float(ws[0]) * float(xs[0]), rtol=2e-6, atol=0)


def test_fp8_convert_weight_transposes_and_uses_one_scale():
    rng = np.random.default_rng(25)
    K, N = 48, 20
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float16)
    wq, s = orc.fp8_convert_weight(w.view(np.uint16), orc.F16)
    assert wq.shape == (N, K)
    assert np.isclose(s[0], np.abs(w.astype(np.float32)).max() / 448.0, rtol=1e-6)
    back = orc.e4m3_decode(wq) * s[0]
    assert np.max(np.abs(back - w.T.astype(np.float32))) <= np.abs(w.astype(np.float32)).max() / 448.0 * 16 + 1e-9


def test_convert_weight_per_channel_closed_form():
    """Per-channel conversion = the per-row closed form of LU/utils_test.cu:93-99 applied to the transposed tensor."""
    rng = np.random.default_rng(77)
    K, N = 48, 20
    w = (rng.standard_normal((K, N)) * np.exp2(rng.integers(-6, 4, size=N))[None, :]).astype(np.float32)
    w[:, 3] = 0.0  # an all-zero channel takes the minimum scale
    bits = orc.to_bits(w, orc.F16)
    wv = orc.from_bits(bits, orc.F16)
    wq, s = orc.fp8_convert_weight_per_channel(bits, orc.F16)
    want_s = np.maximum(np.abs(wv).max(axis=0) / np.float32(448.0), np.float32(1.0 / (448.0 * 512.0))).astype(np.float32)
    assert np.array_equal(s, want_s)
    ratio = np.clip((wv.T / want_s[:, None]).astype(np.float32), -448.0, 448.0)
    want_q = orc.e4m3_encode(ratio.reshape(-1)).reshape(N, K)
    assert np.array_equal(wq & 0x7F, want_q & 0x7F)
    nz = (want_q & 0x7F) != 0
    assert np.array_equal(wq[nz], want_q[nz])
    # dequantised values are within half an e4m3 step (2^-4 relative) of the source
    back = orc.e4m3_decode(wq.reshape(-1)).reshape(N, K) * s[:, None]
    assert np.all(np.abs(back - wv.T) <= np.abs(wv.T) * 2.0**-4 + s[:, None] * 2.0**-10)


def test_merge_qkv_max_matches_requantisation_of_the_parts():
    """The max merge of KS/models/quant/quant_weight.cpp:816-897 on synthetic parts: the merged scale is the maximum,
    the part that owns it is unchanged, the others are e4m3(value * ratio)."""
    rng = np.random.default_rng(78)
    nq, nk, nv, K = 8, 4, 4, 32
    wq = rng.integers(0, 256, size=(nq + nk + nv, K), dtype=np.uint8)
    wq[(wq & 0x7F) == 0x7F] = 0x11
    sq, sk, sv = np.float32(0.02), np.float32(0.05), np.float32(0.0125)
    merged, s = orc.fp8_merge_qkv_max(wq, sq, sk, sv, nq, nk, nv)
    assert s.shape == (1,) and s[0] == sk
    assert np.array_equal(merged[nq:nq + nk], wq[nq:nq + nk])
    vals = orc.e4m3_decode(wq[:nq].reshape(-1)) * np.float32(sq / sk)
    want = orc.e4m3_encode(vals.astype(np.float32)).reshape(nq, K)
    nz = (want & 0x7F) != 0
    assert np.array_equal(merged[:nq][nz], want[nz])
    # v: ratio 0.25 is a power of two, so every normal value moves exactly
    v_in = orc.e4m3_decode(wq[nq + nk:].reshape(-1))
    v_out = orc.e4m3_decode(merged[nq + nk:].reshape(-1))
    normal = np.abs(v_in) >= 2.0**-4
    assert np.array_equal(v_out[normal], v_in[normal] * 0.25)
