"""CPU-side tests of the C ABI: the library loads, exports every declared symbol, validates arguments with the
documented status codes, and the host repack produces the documented fragment order (checked against an
independent pure-Python statement of the layout).  No compute entry point is called on a device here."""
import ctypes
import os
import re

import numpy as np
import pytest

from ksanallm_amd import capi
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "ksq.h")).read()
    declared = set(re.findall(r"\b(ksq_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    L = capi.lib()
    for name in sorted(declared):
        assert hasattr(L, name), f"libksq.so does not export {name}"
    assert set(capi.EXPORTS) == declared
    assert capi.version() >= 100


def _expected_words(u):
    K, N = u.shape
    words = np.zeros(K * N // 8, dtype=np.uint32)
    for k in range(K):
        for n in range(N):
            nt, kt, c, kk = n // 16, k // 128, n % 16, k % 128
            d, j, e = kk >> 5, (kk >> 3) & 3, kk & 7
            w = ((nt * (K // 128) + kt) * 64 + 16 * j + c) * 4 + d
            nib = 4 + e // 2 if e & 1 else e // 2
            words[w] |= np.uint32(int(u[k, n]) << (4 * nib))
    return words


@pytest.mark.parametrize("g", [64, 128])
def test_host_repack_fragment_order(g):
    rng = np.random.default_rng(31)
    K, N = 256, 48
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = orc.to_bits(np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3, orc.BF16)
    want = _expected_words(u)
    sources = [
        (capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u)),
        (capi.W4_AWQ_INT32_NPACK, orc.awq_pack(u)),
        (capi.W4_ROWMAJOR_INT4_SIGNED, orc.rowmajor_pack(u)),
    ]
    zero_forms = [
        (capi.ZERO_UINT8, z, z),
        (capi.ZERO_AWQ_INT32, orc.awq_pack(z), z),
        (capi.ZERO_ADDITIVE, orc.awq_additive_zeros(s, orc.BF16, z), z),
        (capi.ZERO_NONE, None, np.full_like(z, 8)),
    ]
    for layout, src in sources:
        for zk, zsrc, zwant in zero_forms:
            dw = np.zeros(K * N // 8, dtype=np.uint32)
            dsz = np.zeros((K // g) * N, dtype=np.uint32)
            capi.w4a16_repack_host(layout, src, zk, zsrc, s, capi.BF16, K, N, g, dw, dsz)
            assert np.array_equal(dw, want)
            szw = dsz.reshape(N // 16, K // g, 16).transpose(1, 0, 2).reshape(K // g, N)
            assert np.array_equal((szw & 0xFFFF).astype(np.uint16), s)
            assert np.array_equal(((szw >> 16) & 0xFF).astype(np.uint8), zwant)
            # bits 24..31: with bf16 scales, the largest binary exponent of the column's scales in every word of it
            col_exp = np.floor(np.log2(orc.from_bits(s, orc.BF16))).max(axis=0).astype(np.int64)
            assert np.array_equal((szw >> 24).astype(np.uint8).view(np.int8), np.tile(col_exp.astype(np.int8), (K // g, 1)))


def test_host_repack_column_exponent_of_bf16_scales():
    """Bits 24..31 of a scale/zero word: zero for fp16 scales; for bf16 scales the largest exponent among the column's
    finite non-zero scales (zero for a column of zeros), whatever the magnitudes."""
    rng = np.random.default_rng(32)
    K, N, g = 512, 32, 128
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    sv = np.exp2(rng.integers(-120, 120, size=(K // g, N)).astype(np.float64)) * (1 + rng.random((K // g, N)))
    sv[:, 3] = 0.0
    sv[1, 5] = 0.0
    s = orc.to_bits(sv.astype(np.float32), orc.BF16)
    back = orc.from_bits(s, orc.BF16).astype(np.float64)
    want = np.zeros(N, dtype=np.int64)
    for n in range(N):
        nz = back[:, n][back[:, n] > 0]
        want[n] = int(np.floor(np.log2(nz)).max()) if nz.size else 0
    dw = np.zeros(K * N // 8, dtype=np.uint32)
    dsz = np.zeros((K // g) * N, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u), capi.ZERO_NONE, None, s, capi.BF16, K, N, g, dw, dsz)
    szw = dsz.reshape(N // 16, K // g, 16).transpose(1, 0, 2).reshape(K // g, N)
    assert np.array_equal((szw >> 24).astype(np.uint8).view(np.int8).astype(np.int64), np.tile(want, (K // g, 1)))
    s16 = orc.to_bits(np.clip(sv, 0, 6e4).astype(np.float32), orc.F16)
    capi.w4a16_repack_host(capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u), capi.ZERO_NONE, None, s16, capi.F16, K, N, g, dw, dsz)
    assert np.all(dsz >> 24 == 0)


def test_additive_zero_recovery_fp16_all_values():
    # every z in [0,15] against a spread of scales, including tiny and large ones
    scales = np.array([1e-3, 0.0123, 0.02, 0.5, 1.0, 3.3, 6e-5, 100.0], dtype=np.float32)
    K, g = 128, 128
    N = 16 * len(scales)
    sv = np.repeat(scales, 16)[None, :]
    z = np.tile(np.arange(16, dtype=np.uint8), len(scales))[None, :]
    s = orc.to_bits(sv, orc.F16)
    za = orc.awq_additive_zeros(s, orc.F16, z)
    u = np.zeros((K, N), dtype=np.uint8)
    dw = np.zeros(K * N // 8, dtype=np.uint32)
    dsz = np.zeros(N, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u), capi.ZERO_ADDITIVE, za, s, capi.F16, K, N, g,
                           dw, dsz)
    got = ((dsz.reshape(N // 16, 1, 16) >> 16) & 0xFF).astype(np.uint8).transpose(1, 0, 2).reshape(1, N)
    assert np.array_equal(got, z)


def test_sizes_and_argument_validation():
    assert capi.w4a16_repack_sizes(4096, 4096, 128) == (4096 * 4096 // 2, 32 * 4096 * 4)
    for k, n, g in [(100, 64, 128), (256, 24, 128), (256, 64, 32), (0, 64, 128)]:
        with pytest.raises(capi.KsqError) as ei:
            capi.w4a16_repack_sizes(k, n, g)
        assert ei.value.code in (capi.ERR_UNSUPPORTED, capi.ERR_INVALID_ARGUMENT)
    buf = np.zeros(64, dtype=np.uint8)
    with pytest.raises(capi.KsqError) as ei:  # null tensor
        capi.w4a16_gemm(capi.F16, None, buf, buf, buf, 1, 16, 128, 128)
    assert ei.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError) as ei:  # the reference kernels also refuse other group sizes
        capi.w4a16_gemm(capi.F16, buf, buf, buf, buf, 1, 16, 128, 32)
    assert ei.value.code == capi.ERR_UNSUPPORTED
    for k, g in ((192, 128), (160, 64)):  # k not a whole number of groups
        with pytest.raises(capi.KsqError) as ei:
            capi.w4a16_gemm(capi.F16, buf, buf, buf, buf, 1, 16, k, g)
        assert ei.value.code == capi.ERR_UNSUPPORTED
    with pytest.raises(capi.KsqError) as ei:  # bad dtype
        capi.w4a16_gemm(7, buf, buf, buf, buf, 1, 16, 128, 128)
    assert ei.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError) as ei:  # weight scale missing: the reference layer throws too
        capi.fp8_gemm(capi.BF16, buf, buf, buf, 1, buf, None, 1, 1, 16, 64)
    assert ei.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError) as ei:
        capi.fp8_gemm(capi.BF16, buf, buf, buf, 3, buf, buf, 1, 2, 16, 64)  # act_scale_count not 1 or m
    assert ei.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError) as ei:
        capi.fp8_quantize(capi.F16, buf, 1, 16, 9, buf, buf)
    assert ei.value.code == capi.ERR_INVALID_ARGUMENT
    assert "mode" in str(ei.value)


def test_empty_inputs_are_noops():
    buf = np.zeros(64, dtype=np.uint8)
    capi.w4a16_gemm(capi.F16, buf, buf, buf, buf, 0, 16, 128, 128)  # m = 0
    capi.fp8_gemm(capi.F16, buf, buf, buf, 1, buf, buf, 1, 0, 16, 64)
    capi.fp8_quantize(capi.F16, buf, 0, 16, capi.FP8_PER_TOKEN_DYNAMIC, buf, buf)
    capi.fp8_rescale(buf, buf, 0, buf, buf)


def test_workspace_sizes_are_monotone_and_bounded():
    for n, k in [(4096, 4096), (12288, 4096), (22016, 4096), (4096, 11008), (57344, 8192)]:
        w16 = capi.w4a16_workspace_bytes(16, n, k)
        w64 = capi.w4a16_workspace_bytes(64, n, k)
        w4096 = capi.w4a16_workspace_bytes(4096, n, k)
        assert w16 <= w64 <= w4096
        assert w64 <= k * n // 2  # decode: never more than the weights themselves
        # prefill: an fp16 copy of the activations + row factors, and split-K partial tiles of at most two workgroups
        # per compute unit (64 x 256 fp32 each)
        assert w4096 <= max(w64, 4096 * k * 2 + 4096 * 4 + 512 + 2 * 256 * 64 * 256 * 4)
    assert capi.fp8_workspace_bytes(64, 8192, 8192) <= 8192 * 8192


def test_workspace_sizes_of_padded_k_and_split_last_round():
    """What the planners add to the workspace, computed on the host alone (256 compute units when no device is there):
    the padded copy of the activation rows when K is an odd multiple of 64, and the fp32 partial tiles of a large-M FP8
    GEMM whose last round of 256 x 256 tiles is between a quarter and half full, or that is a single round leaving most
    units empty; the
    self-quantising entry point adds the FP8 rows and scales."""
    assert capi.w4a16_workspace_bytes(16, 64, 192) == capi.w4a16_workspace_bytes(16, 64, 256) + 16 * 256 * 2
    # 8 x 44 = 352 tiles: the last 96 (more than a quarter, at most half of the units) go out with K split in two; a
    # smaller batch needs more (M = 256: 44 tiles in one round, 64 k stages = 5 splits of 12 at least)
    assert capi.fp8_workspace_bytes(2048, 11264, 8192) == 44 * 5 * 256 * 256 * 4
    assert 96 * 2 < 44 * 5
    # 8 x 40 = 320 tiles: the last 64 go out as column quarters and need nothing; what is left is the largest need of
    # a smaller batch (M = 512: 80 tiles in one round, K split in three)
    assert capi.fp8_workspace_bytes(2048, 10240, 8192) == 80 * 3 * 256 * 256 * 4
    # a single round that leaves most units empty is split as a whole: 40 tiles, 64 k stages = 5 splits of 12 at least
    assert capi.fp8_workspace_bytes(256, 10240, 8192) == 40 * 5 * 256 * 256 * 4
    assert capi.fp8_workspace_bytes(64, 10240, 8192) < 40 * 5 * 256 * 256 * 4       # decode kernels only
    front = capi.fp8_gemm_dynamic_workspace_bytes(2048, 10240, 8192) - capi.fp8_workspace_bytes(2048, 10240, 8192)
    assert 2048 * 8192 + 2048 * 4 <= front <= 2048 * 8192 + 2048 * 4 + 1024


def test_host_repack_pads_a_k_that_is_an_odd_multiple_of_64():
    """Group size 64 admits K = 64 * odd (the reference's k % 64 == 0): the destination has whole 128-row tiles, the
    rows past K hold nibble 8 and their group's words a zero scale with z = 8, everything else is the ordinary repack."""
    rng = np.random.default_rng(33)
    K, N, g = 192, 32, 64
    Kp = 256
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = orc.to_bits(np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3, orc.F16)
    assert capi.w4a16_repack_sizes(K, N, g) == (Kp * N // 2, (Kp // g) * N * 4)
    dw = np.zeros(Kp * N // 8, dtype=np.uint32)
    dsz = np.zeros((Kp // g) * N, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_AWQ_INT32_NPACK, orc.awq_pack(u), capi.ZERO_AWQ_INT32, orc.awq_pack(z), s, capi.F16,
                           K, N, g, dw, dsz)
    upad = np.concatenate([u, np.full((Kp - K, N), 8, dtype=np.uint8)])
    assert np.array_equal(dw, _expected_words(upad))
    szw = dsz.reshape(N // 16, Kp // g, 16).transpose(1, 0, 2).reshape(Kp // g, N)
    assert np.array_equal((szw[: K // g] & 0xFFFF).astype(np.uint16), s)
    assert np.array_equal(((szw[: K // g] >> 16) & 0xFF).astype(np.uint8), z)
    assert np.all(szw[K // g:] == (8 << 16))
    with pytest.raises(capi.KsqError):
        capi.w4a16_repack_sizes(192, N, 128)   # group size 128 needs whole groups


def test_workgroup_to_tile_map_is_a_bijection():
    """tile_of / tile_grid (csrc/ksq_internal.h), the map from workgroup ids to output tiles that the large-M kernels
    share: every tile exactly once for 40 x 31 grid sizes, ids past the last tile refused, bands of eight row blocks
    walked column by column.  The checker is a host program built next to the library."""
    import subprocess

    exe = os.path.join(os.path.dirname(capi.LIB_PATH), "tile_map_test")
    if not os.path.exists(exe):
        pytest.skip("tile_map_test has not been built (python -m ksanallm_amd.build)")
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert p.returncode == 0 and p.stdout.startswith("OK"), p.stdout
