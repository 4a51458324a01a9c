"""CPU-side tests of the load-time pieces that widen the path: the CUTLASS-preprocessed weight layouts as repack
input, the desc_act row permutation, the gate/up column interleave.  The oracle's restatement of the reference's
preprocessor is pinned step by step against what the reference documents about each step (its row map and register
picture, the meaning of a column-major tile-interleaved layout), then the library's repack, which reads that layout
through a closed-form inverse, must reproduce the repack of the row-major source bit for bit.  Runs without a GPU
(host entry points only)."""
import numpy as np
import pytest

from ksanallm_amd import capi
from oracle import oracle as orc


def _nibbles(buf):
    b = np.asarray(buf, dtype=np.uint8).reshape(-1)
    out = np.empty(b.size * 2, dtype=np.uint8)
    out[0::2] = b & 15
    out[1::2] = b >> 4
    return out


def _pack_nibbles(n):
    n = np.asarray(n, dtype=np.uint8).reshape(-1)
    return (n[0::2] | (n[1::2] << 4)).astype(np.uint8)


# ---- the four steps of preprocess_weights_for_mixed_gemm, one at a time

def test_cutlass_row_permutation_is_the_documented_map():
    # the reference documents the W4_A16 map for each group of 32 rows (cutlass_preprocessors.cpp:123-124)
    documented = [0, 1, 8, 9, 16, 17, 24, 25, 2, 3, 10, 11, 18, 19, 26, 27,
                  4, 5, 12, 13, 20, 21, 28, 29, 6, 7, 14, 15, 22, 23, 30, 31]
    K, N = 64, 16
    rows = np.repeat(np.arange(K, dtype=np.uint8)[:, None], N // 2, axis=1)  # every byte of row k holds k
    out = orc.cutlass_step("permute_rows", rows, K, N).reshape(K, N // 2)
    assert [int(x) for x in out[:32, 0]] == documented
    assert [int(x) - 32 for x in out[32:, 0]] == documented
    assert np.all(out == out[:, :1])


def test_cutlass_transpose_is_a_nibble_transpose():
    rng = np.random.default_rng(41)
    K, N = 64, 24
    nib = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    out = orc.cutlass_step("transpose", _pack_nibbles(nib), K, N)
    assert np.array_equal(_nibbles(out).reshape(N, K), nib.T)


def test_cutlass_column_interleave_is_tile_interleave_64x4():
    # ColumnMajorTileInterleave<64, 4>: the column-major matrix is read as (4K) x (N/4); inside column n/4 come, for
    # every tile of 64 rows, the 64 rows of column 4q, then of 4q+1, 4q+2, 4q+3.
    rng = np.random.default_rng(42)
    K, N = 192, 16
    nib = rng.integers(0, 16, size=(N, K), dtype=np.uint8)  # column-major input: [n][k]
    out = _nibbles(orc.cutlass_step("interleave_columns", _pack_nibbles(nib), K, N))
    for n in range(N):
        for k in range(K):
            pos = (n // 4) * 4 * K + (k // 64) * 256 + (n % 4) * 64 + (k % 64)
            assert out[pos] == nib[n, k]


def test_cutlass_register_relayout_matches_the_documented_picture():
    # signed nibbles -8..7 become 0..15, and [elt_7 .. elt_0] becomes [elt_7 elt_5 elt_3 elt_1 elt_6 elt_4 elt_2 elt_0]
    # from bit 32 down (cutlass_preprocessors.cpp:376-383)
    signed = np.array([0, 1, 2, 3, 4, 5, 6, 7], dtype=np.int8) - 8  # elt_i = i - 8 -> i after the bias
    reg = _pack_nibbles((signed & 15).astype(np.uint8))
    out = orc.cutlass_step("bias_and_interleave", np.tile(reg, 2), 4, 4)
    assert int(out[:4].view(np.uint32)[0]) == 0x75316420
    signed = np.array([7, -8, -1, 0, 3, -4, 5, -6], dtype=np.int8)
    reg = _pack_nibbles((signed & 15).astype(np.uint8))
    got = _nibbles(orc.cutlass_step("bias_and_interleave", np.tile(reg, 2), 4, 4)[:4])
    assert [int(x) for x in got] == [int(signed[i]) + 8 for i in (0, 2, 4, 6, 1, 3, 5, 7)]


def test_cutlass_pipeline_is_a_bijection_that_keeps_the_values():
    rng = np.random.default_rng(43)
    K, N = 128, 32
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    out = orc.cutlass_preprocess(orc.rowmajor_pack(u), 80)
    assert np.array_equal(np.bincount(_nibbles(out), minlength=16), np.bincount(u.reshape(-1), minlength=16))
    # one marked nibble at a time lands in one place, and different sources in different places
    seen = set()
    for k, n in [(0, 0), (1, 0), (0, 1), (31, 5), (32, 5), (63, 31), (64, 0), (127, 31), (77, 18)]:
        v = np.full((K, N), 8, dtype=np.uint8)  # q = 0 everywhere
        v[k, n] = 15
        o = _nibbles(orc.cutlass_preprocess(orc.rowmajor_pack(v), 80))
        where = np.flatnonzero(o != 8)
        assert where.size == 1 and o[where[0]] == 15
        assert int(where[0]) not in seen
        seen.add(int(where[0]))


# ---- the library's repack reads these layouts

@pytest.mark.parametrize("arch,layout", [(80, capi.W4_CUTLASS_SM80_INTERLEAVED), (90, capi.W4_CUTLASS_SM90_COLMAJOR)])
@pytest.mark.parametrize("K,N", [(128, 16), (256, 48), (384, 64)])
def test_host_repack_from_cutlass_layouts_equals_repack_from_rowmajor(arch, layout, K, N):
    rng = np.random.default_rng(50 + K + N)
    g = 128
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = orc.to_bits(np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3, orc.F16)
    zeros = orc.awq_additive_zeros(s, orc.F16, z)  # what the reference's loader hands to the layer
    rowmajor = orc.rowmajor_pack(u)
    want_w = np.zeros(K * N // 8, dtype=np.uint32)
    want_sz = np.zeros((K // g) * N, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_ROWMAJOR_INT4_SIGNED, rowmajor, capi.ZERO_ADDITIVE, zeros, s, capi.F16, K, N, g,
                           want_w, want_sz)
    pre = orc.cutlass_preprocess(rowmajor, arch)
    got_w = np.zeros_like(want_w)
    got_sz = np.zeros_like(want_sz)
    capi.w4a16_repack_host(layout, pre, capi.ZERO_ADDITIVE, zeros, s, capi.F16, K, N, g, got_w, got_sz)
    assert np.array_equal(got_w, want_w)
    assert np.array_equal(got_sz, want_sz)


# ---- desc_act

def _act_order_g_idx(rng, K, g):
    """g_idx of a GPTQ act-order checkpoint: rows are quantised in a permuted order, g at a time."""
    order = rng.permutation(K)
    g_idx = np.empty(K, dtype=np.int32)
    g_idx[order] = np.arange(K, dtype=np.int32) // g
    return g_idx


def test_act_order_perm_is_the_stable_argsort():
    rng = np.random.default_rng(60)
    K, g = 512, 64
    g_idx = _act_order_g_idx(rng, K, g)
    perm = np.empty(K, dtype=np.int32)
    capi.gptq_act_order_perm(g_idx, K, g, perm)
    assert np.array_equal(perm, np.argsort(g_idx, kind="stable").astype(np.int32))  # library routine
    assert np.array_equal(perm, orc.act_order_perm(g_idx))                           # the oracle's insertion sort
    assert np.array_equal(g_idx[perm], np.arange(K) // g)


def test_act_order_perm_rejects_partial_groups_and_bad_indices():
    K, g = 256, 128
    perm = np.empty(K, dtype=np.int32)
    g_idx = (np.arange(K) // g).astype(np.int32)
    g_idx[0] = 1  # group 0 has 127 rows, group 1 has 129
    with pytest.raises(capi.KsqError) as e:
        capi.gptq_act_order_perm(g_idx, K, g, perm)
    assert e.value.code == capi.ERR_UNSUPPORTED
    g_idx[0] = 2
    with pytest.raises(capi.KsqError) as e:
        capi.gptq_act_order_perm(g_idx, K, g, perm)
    assert e.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError):
        capi.gptq_act_order_perm(g_idx, 100, 128, perm)


@pytest.mark.parametrize("order", [capi.COLS_NATURAL, capi.COLS_HALVES_INTERLEAVED])
def test_host_repack_ex_row_perm_and_column_order(order):
    rng = np.random.default_rng(61)
    K, N, g = 256, 64, 64
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    s = orc.to_bits(np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3, orc.F16)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    perm = rng.permutation(K).astype(np.int32)
    cols = np.arange(N)
    if order == capi.COLS_HALVES_INTERLEAVED:
        cols = np.empty(N, dtype=np.int64)
        cols[0::2] = np.arange(N // 2)
        cols[1::2] = N // 2 + np.arange(N // 2)
    # what the call must produce: the plain repack of the tensor with rows and columns already moved
    want_w = np.zeros(K * N // 8, dtype=np.uint32)
    want_sz = np.zeros((K // g) * N, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(np.ascontiguousarray(u[perm][:, cols])),
                           capi.ZERO_UINT8, np.ascontiguousarray(z[:, cols]), np.ascontiguousarray(s[:, cols]),
                           capi.F16, K, N, g, want_w, want_sz)
    for layout, src, zk, zsrc in [
        (capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u), capi.ZERO_UINT8, z),
        (capi.W4_AWQ_INT32_NPACK, orc.awq_pack(u), capi.ZERO_AWQ_INT32, orc.awq_pack(z)),
        (capi.W4_CUTLASS_SM80_INTERLEAVED, orc.cutlass_preprocess(orc.rowmajor_pack(u), 80), capi.ZERO_UINT8, z),
    ]:
        got_w = np.zeros_like(want_w)
        got_sz = np.zeros_like(want_sz)
        capi.w4a16_repack_ex_host(layout, src, zk, zsrc, s, capi.F16, K, N, g, perm, order, got_w, got_sz)
        assert np.array_equal(got_w, want_w)
        assert np.array_equal(got_sz, want_sz)


def test_host_repack_ex_validates():
    K, N, g = 128, 16, 128
    u = np.zeros((K, N), dtype=np.uint8)
    s = np.zeros((1, N), dtype=np.uint16)
    dw = np.zeros(K * N // 8, dtype=np.uint32)
    dsz = np.zeros(N, dtype=np.uint32)
    bad = np.arange(K, dtype=np.int32)
    bad[5] = K
    with pytest.raises(capi.KsqError) as e:
        capi.w4a16_repack_ex_host(capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u), capi.ZERO_NONE, None, s, capi.F16, K, N,
                                  g, bad, capi.COLS_NATURAL, dw, dsz)
    assert e.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError) as e:
        capi.w4a16_repack_ex_host(capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u), capi.ZERO_NONE, None, s, capi.F16, K, N,
                                  g, None, 7, dw, dsz)
    assert e.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError):
        capi.w4a16_repack_host(9, orc.gptq_pack(u), capi.ZERO_NONE, None, s, capi.F16, K, N, g, dw, dsz)


def test_silu_mul_oracle_against_library_routine():
    import torch

    rng = np.random.default_rng(62)
    acc = (rng.standard_normal((7, 64)) * 4).astype(np.float32)
    acc[0, 0], acc[0, 1], acc[0, 2] = -80.0, 80.0, 0.0
    want = (torch.nn.functional.silu(torch.from_numpy(acc[:, :32]).double()) * torch.from_numpy(acc[:, 32:]).double())
    got = orc.silu_mul(acc)
    assert np.allclose(got, want.numpy(), rtol=1e-6, atol=1e-30)


# ---- Marlin

def _published_marlin_weights(u):
    """The Marlin 4-bit weight format as published with it (vLLM's marlin_permute_weights + get_weight_perm + pack_cols,
    the file the reference cites at quant_weight.cpp:348), in numpy: u [K, N] unsigned nibbles -> int32 [K/16, N*2]."""
    K, N = u.shape
    perm = []
    for i in range(32):
        perm1 = []
        col = i // 4
        for block in (0, 1):
            for row in (2 * (i % 4), 2 * (i % 4) + 1, 2 * (i % 4 + 4), 2 * (i % 4 + 4) + 1):
                perm1.append(16 * row + col + 8 * block)
        for j in range(4):
            perm.extend(p + 256 * j for p in perm1)
    perm = np.array(perm).reshape(-1, 8)[:, [0, 2, 4, 6, 1, 3, 5, 7]].ravel()
    q = u.astype(np.uint32).reshape(K // 16, 16, N // 16, 16).transpose(0, 2, 1, 3).reshape(K // 16, N * 16)
    q = q.reshape(-1, perm.size)[:, perm].reshape(K // 16, N * 16)
    packed = np.zeros((K // 16, N * 2), dtype=np.uint32)
    for i in range(8):
        packed |= q[:, i::8] << np.uint32(4 * i)
    return packed.view(np.int32)


@pytest.mark.parametrize("K,N", [(128, 64), (256, 192)])
def test_marlin_repack_restatements_match_the_published_format(K, N):
    rng = np.random.default_rng(70 + K)
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    want = _published_marlin_weights(u)
    assert np.array_equal(orc.marlin_repack(orc.gptq_pack(u), K, N, "gptq"), want)
    assert np.array_equal(orc.marlin_repack(orc.awq_pack(u), K, N, "awq"), want)


def test_marlin_scale_and_zero_point_restatements():
    # each block of 64 columns is read as an 8 x 8 matrix and transposed; a single group uses blocks of 32 instead
    s = np.arange(2 * 128, dtype=np.uint16).reshape(2, 128)
    got = orc.marlin_permute_scales(s, 256, 128)
    want = s.reshape(2, 2, 8, 8).transpose(0, 1, 3, 2).reshape(2, 128)
    assert np.array_equal(got, want)
    one = np.arange(64, dtype=np.uint16).reshape(1, 64)
    got1 = orc.marlin_permute_scales(one, 128, 128)
    assert [int(x) for x in got1[0, :8]] == [0, 1, 8, 9, 16, 17, 24, 25] and int(got1[0, 8]) == 2
    assert sorted(int(x) for x in got1[0, :32]) == list(range(32))
    z = (np.arange(64, dtype=np.uint8) % 16).reshape(1, 64)
    zp = orc.marlin_zero_points(z).view(np.uint32)
    cols = z.reshape(8, 8).T.reshape(-1)  # after the 8 x 8 transpose
    for wd in range(8):
        for nib, src in enumerate([0, 2, 4, 6, 1, 3, 5, 7]):
            assert (int(zp[0, wd]) >> (4 * nib)) & 15 == int(cols[8 * wd + src])


@pytest.mark.parametrize("kind", ["gptq", "awq"])
@pytest.mark.parametrize("K,N,g", [(128, 64, 128), (256, 192, 128), (256, 128, 64)])
def test_host_repack_from_marlin_equals_repack_from_checkpoint(kind, K, N, g):
    rng = np.random.default_rng(80 + K + N)
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    s = orc.to_bits(np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3, orc.F16)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8) if kind == "awq" else None
    want_w = np.zeros(K * N // 8, dtype=np.uint32)
    want_sz = np.zeros((K // g) * N, dtype=np.uint32)
    if kind == "awq":
        capi.w4a16_repack_host(capi.W4_AWQ_INT32_NPACK, orc.awq_pack(u), capi.ZERO_AWQ_INT32, orc.awq_pack(z), s,
                               capi.F16, K, N, g, want_w, want_sz)
        marlin = orc.marlin_repack(orc.awq_pack(u), K, N, "awq")
        zk, zsrc = capi.ZERO_MARLIN_INT32, orc.marlin_zero_points(z)
    else:
        capi.w4a16_repack_host(capi.W4_GPTQ_INT32_KPACK, orc.gptq_pack(u), capi.ZERO_NONE, None, s, capi.F16, K, N, g,
                               want_w, want_sz)
        marlin = orc.marlin_repack(orc.gptq_pack(u), K, N, "gptq")
        zk, zsrc = capi.ZERO_NONE, None
    got_w = np.zeros_like(want_w)
    got_sz = np.zeros_like(want_sz)
    capi.w4a16_repack_host(capi.W4_MARLIN, marlin, zk, zsrc, orc.marlin_permute_scales(s, K, g), capi.F16, K, N, g,
                           got_w, got_sz)
    assert np.array_equal(got_w, want_w)
    assert np.array_equal(got_sz, want_sz)


def test_marlin_argument_rules():
    K, N, g = 128, 64, 128
    w = np.zeros((K // 16, N * 2), dtype=np.int32)
    s = np.zeros((1, N), dtype=np.uint16)
    z8 = np.zeros((1, N), dtype=np.uint8)
    dw = np.zeros(K * N // 8, dtype=np.uint32)
    dsz = np.zeros(N, dtype=np.uint32)
    with pytest.raises(capi.KsqError) as e:  # Marlin weights with zero points in another form
        capi.w4a16_repack_host(capi.W4_MARLIN, w, capi.ZERO_UINT8, z8, s, capi.F16, K, N, g, dw, dsz)
    assert e.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError) as e:  # Marlin zero points with another weight layout
        capi.w4a16_repack_host(capi.W4_GPTQ_INT32_KPACK, np.zeros((K // 8, N), dtype=np.int32), capi.ZERO_MARLIN_INT32,
                               np.zeros((1, N // 8), dtype=np.int32), s, capi.F16, K, N, g, dw, dsz)
    assert e.value.code == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(capi.KsqError) as e:  # n must be a multiple of 64
        capi.w4a16_repack_host(capi.W4_MARLIN, np.zeros((K // 16, 96), dtype=np.int32), capi.ZERO_NONE, None,
                               np.zeros((1, 48), dtype=np.uint16), capi.F16, K, 48, g, np.zeros(K * 48 // 8, np.uint32),
                               np.zeros(48, np.uint32))
    assert e.value.code == capi.ERR_UNSUPPORTED


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_parts_repacked_side_by_side_equal_the_concatenated_repack(dtype):
    """Column tiles are contiguous in the fragment order and in the scale/zero words, so tensors that share K can be
    repacked one by one into consecutive ranges of the fused buffers (what replaces the loader's q/k/v concat,
    KS/models/quant/quant_weight.cpp:471-513): bit for bit the repack of the concatenated tensor."""
    rng = np.random.default_rng(77)
    K, g = 512, 128
    widths = [96, 32, 48]
    N = sum(widths)
    odt = orc.F16 if dtype == "f16" else orc.BF16
    cdt = capi.F16 if dtype == "f16" else capi.BF16
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = orc.to_bits((np.abs(rng.standard_normal((K // g, N))) * 0.02 + 1e-3).astype(np.float32), odt)
    want_w = np.zeros(K * N // 8, dtype=np.uint32)
    want_sz = np.zeros((K // g) * N, dtype=np.uint32)
    capi.w4a16_repack_host(capi.W4_AWQ_INT32_NPACK, orc.awq_pack(u), capi.ZERO_AWQ_INT32, orc.awq_pack(z), s, cdt, K, N, g,
                           want_w, want_sz)
    got_w, got_sz = np.zeros_like(want_w), np.zeros_like(want_sz)
    n0 = 0
    for w in widths:
        wb, sb = capi.w4a16_repack_sizes(K, n0, g) if n0 else (0, 0)
        capi.w4a16_repack_host(capi.W4_AWQ_INT32_NPACK, orc.awq_pack(np.ascontiguousarray(u[:, n0:n0 + w])),
                               capi.ZERO_AWQ_INT32, orc.awq_pack(np.ascontiguousarray(z[:, n0:n0 + w])),
                               np.ascontiguousarray(s[:, n0:n0 + w]), cdt, K, w, g, got_w[wb // 4:], got_sz[sb // 4:])
        n0 += w
    assert np.array_equal(got_w, want_w)
    assert np.array_equal(got_sz, want_sz)
