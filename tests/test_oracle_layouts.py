"""Pins the oracle's checkpoint-layout functions without using the oracle's own formulas: brute-force bit
extraction in pure Python on small cases, pack/unpack identities, and the AutoAWQ order composition."""
import numpy as np

from oracle import oracle as orc


def _rng(seed):
    return np.random.default_rng(seed)


def test_gptq_unpack_bruteforce():
    rng = _rng(1)
    K, N = 64, 24
    q = rng.integers(-2**31, 2**31, size=(K // 8, N), dtype=np.int64).astype(np.int32)
    u = orc.gptq_unpack(q)
    for k in range(K):
        for n in range(N):
            word = int(q[k // 8, n]) & 0xFFFFFFFF
            assert u[k, n] == (word >> (4 * (k % 8))) & 15


def test_gptq_matches_reference_byte_view_formulation():
    # the reference transposes, views int32 as bytes, and takes byte % 16 / byte // 16 (quant_weight.cpp:291-300)
    rng = _rng(2)
    K, N = 128, 16
    q = rng.integers(-2**31, 2**31, size=(K // 8, N), dtype=np.int64).astype(np.int32)
    bytes_view = np.ascontiguousarray(q.T).view(np.uint8)  # [N, K/2]
    w = np.zeros((N, K), dtype=np.uint8)
    w[:, 0::2] = bytes_view % 16
    w[:, 1::2] = bytes_view // 16
    assert np.array_equal(orc.gptq_unpack(q), w.T)


def test_gptq_pack_unpack_identity():
    rng = _rng(3)
    u = rng.integers(0, 16, size=(256, 40), dtype=np.uint8)
    assert np.array_equal(orc.gptq_unpack(orc.gptq_pack(u)), u)


def test_awq_order_composition_is_identity():
    order = [0, 2, 4, 6, 1, 3, 5, 7]  # AutoAWQ packing order
    rev = [0, 4, 1, 5, 2, 6, 3, 7]  # reference's reverse order (quant_weight.cpp:276)
    assert [order[rev[i]] for i in range(8)] == list(range(8))


def test_awq_unpack_bruteforce():
    rng = _rng(4)
    R, N = 16, 64
    q = rng.integers(-2**31, 2**31, size=(R, N // 8), dtype=np.int64).astype(np.int32)
    u = orc.awq_unpack(q)
    rev = [0, 4, 1, 5, 2, 6, 3, 7]
    # the reference: shift by 0,4,...,28 -> slots, then gather slots by rev within every 8 columns
    for r in range(R):
        for c in range(N // 8):
            word = int(q[r, c]) & 0xFFFFFFFF
            slots = [(word >> (4 * j)) & 15 for j in range(8)]
            for i in range(8):
                assert u[r, 8 * c + i] == slots[rev[i]]


def test_awq_pack_is_autoawq_order():
    rng = _rng(5)
    u = rng.integers(0, 16, size=(8, 32), dtype=np.uint8)
    q = orc.awq_pack(u)
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    for r in range(8):
        for c in range(4):
            word = 0
            for j in range(8):
                word |= int(u[r, 8 * c + order[j]]) << (4 * j)
            assert (int(q[r, c]) & 0xFFFFFFFF) == word
    assert np.array_equal(orc.awq_unpack(q), u)


def test_rowmajor_pack_bruteforce_and_identity():
    rng = _rng(6)
    u = rng.integers(0, 16, size=(32, 16), dtype=np.uint8)
    p = orc.rowmajor_pack(u)
    for k in range(32):
        for b in range(8):
            q0 = int(u[k, 2 * b]) - 8
            q1 = int(u[k, 2 * b + 1]) - 8
            assert p[k, b] == ((q0 & 0xF) | ((q1 & 0xF) << 4))
    assert np.array_equal(orc.rowmajor_unpack(p), u)


def test_awq_additive_zero_identity():
    # s*(u-8) + s*(8-z) == s*(u-z): the two dequant forms agree to fp16 rounding of the additive zero
    rng = _rng(7)
    K, N, g = 256, 32, 128
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = orc.to_bits(np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3, orc.F16)
    za = orc.awq_additive_zeros(s, orc.F16, z)
    sf = orc.from_bits(s, orc.F16)
    want = np.float16(sf * (8.0 - z.astype(np.float32)))
    assert np.array_equal(za.view(np.float16), want)
    w_int = orc.dequant(u, s, orc.F16, z, g)
    w_add = orc.dequant_additive(u, s, orc.F16, za, g)
    scale_full = np.repeat(sf, g, axis=0)
    assert np.max(np.abs(w_int - w_add) / scale_full) <= 8 * 2.0**-11 + 1e-6


def test_dequant_closed_form_numpy():
    rng = _rng(8)
    K, N, g = 384, 48, 128
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    for dt, npdt in ((orc.F16, np.float16), (orc.BF16, None)):
        sv = (np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3).astype(np.float32)
        s = orc.to_bits(sv, dt)
        sf = orc.from_bits(s, dt)
        if npdt is not None:
            assert np.array_equal(sf, sv.astype(npdt).astype(np.float32))
        else:  # bf16: top 16 bits after round-to-nearest-even
            b = sv.view(np.uint32).astype(np.uint64)
            r = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
            assert np.array_equal(s, r)
        want = np.repeat(sf, g, axis=0) * (u.astype(np.float32) - np.repeat(z, g, axis=0).astype(np.float32))
        assert np.array_equal(orc.dequant(u, s, dt, z, g), want)
        want8 = np.repeat(sf, g, axis=0) * (u.astype(np.float32) - 8.0)
        assert np.array_equal(orc.dequant(u, s, dt, None, g), want8)
