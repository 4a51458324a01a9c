#!/usr/bin/env python3
"""Writes the golden vectors of tests/golden/*.npz.

Everything here is computed by an independent statement of the formats -- plain numpy integer arithmetic and
float64 sums, no call into the oracle and none into the GPU library -- so the fixtures pin both.  The formats
follow KsanaLLM's loader and FP8 helpers (KS = src/ksana_llm, LU = 3rdparty/LLM_kernels/csrc/utils/nvidia):

  gptq_64x64      KS/models/quant/quant_weight.cpp:291-300   qweight int32 [K/8,N], element k=8r+j in bits 4j..4j+3
  awq_128x64      KS/models/quant/quant_weight.cpp:262-287   qweight int32 [K,N/8], slot j = column 8c+[0,2,4,6,1,3,5,7][j]
  rowmajor        KS/models/quant/quant_weight.cpp:304-328   int8 [K,N/2], low nibble = even column, signed u-8
  e4m3_table      OCP FP8 E4M3 (bias 7, no infinities, 0x7f/0xff NaN, max 448), as __nv_fp8_e4m3 in LU/cuda_fp8_utils.h
  w4a16_*         out = sum_k a[m,k] * s[k/g,n] * (u[k,n] - z[k/g,n]) in float64 from the exact fp16 / bf16 values,
                  stored rounded once to float32
  fp8_quant_*     LU/cuda_fp8_utils.cu:27-44, 85-127         scale = max(absmax/448, 1/(448*512)), q = e4m3(clamp(x/scale))
  fp8_gemm_*      KS/kernels/nvidia/kernel_wrapper.cpp:1033-1041  out = (sum_k a*w) * w_scale[n] * a_scale[m] in float64
  w4a16_next_*    the same weights as the loader's other back ends leave them, and the steps either side of the GEMM:
                  cutlass80 / cutlass90  LK/asymmetric_gemm/cutlass_preprocessors.cpp:466-508 as whole-array reshapes
                  marlin*                the format as published with vLLM's marlin_utils (cited at quant_weight.cpp:348)
                  g_idx / perm / out_desc  desc_act: row k uses scales[g_idx[k]]; perm = stable argsort (quant_weight.cpp:455-460)
                  out_silu / out_bias    silu(gate) * up of [gate | up] and out + bias, in float64

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
AWQ_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]


def f16_bits(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_value(b):
    return b.view(np.float16).astype(np.float64)


def bf16_bits(x):
    """float32 -> bfloat16 bit pattern, round to nearest even (finite inputs)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_value(b):
    return (b.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def gptq_pack(u):
    K, N = u.shape
    q = np.zeros((K // 8, N), dtype=np.uint32)
    for r in range(K // 8):
        for j in range(8):
            q[r] |= u[8 * r + j].astype(np.uint32) << np.uint32(4 * j)
    return q.view(np.int32)


def awq_pack(u):
    K, N = u.shape
    q = np.zeros((K, N // 8), dtype=np.uint32)
    for c in range(N // 8):
        for j in range(8):
            q[:, c] |= u[:, 8 * c + AWQ_ORDER[j]].astype(np.uint32) << np.uint32(4 * j)
    return q.view(np.int32)


def rowmajor_pack(u):
    s = (u.astype(np.int16) - 8) & 0xF
    return (s[:, 0::2] | (s[:, 1::2] << 4)).astype(np.uint8).view(np.int8)


def e4m3_table():
    t = np.zeros(256, dtype=np.float64)
    for c in range(256):
        sign = -1.0 if c & 0x80 else 1.0
        e, m = (c >> 3) & 0xF, c & 7
        if e == 15 and m == 7:
            t[c] = np.nan
        elif e == 0:
            t[c] = sign * m * 2.0 ** -9
        else:
            t[c] = sign * (1 + m / 8.0) * 2.0 ** (e - 7)
    return t


def e4m3_encode(x, table):
    """Nearest representable value, ties to the even code, saturating at 448; x is float64 and already clamped."""
    pos = table[:127]  # 0 .. 448, increasing
    ax = np.abs(x)
    hi = np.searchsorted(pos, ax, side="left").clip(1, 126)
    lo = hi - 1
    dlo, dhi = ax - pos[lo], pos[hi] - ax
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    return code | np.where(np.signbit(x), 0x80, 0).astype(np.uint8)


def w4a16_case(seed, M, K, N, g, awq, bf16, column_exponents=0):
    """column_exponents = e > 0 multiplies every column's scales by 2^j, j drawn per column from [-e, e]: bf16 scales
    that no fp16 holds, with the spread inside a column (about 2^6) left as it is."""
    rng = np.random.default_rng(seed)
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8) if awq else np.full((K // g, N), 8, dtype=np.uint8)
    s = np.abs(rng.standard_normal((K // g, N))).astype(np.float32) * 0.02 + 1e-3
    if column_exponents:
        s = s * np.exp2(rng.integers(-column_exponents, column_exponents + 1, size=N)).astype(np.float32)[None, :]
    a = rng.standard_normal((M, K)).astype(np.float32)
    to_bits, to_val = (bf16_bits, bf16_value) if bf16 else (f16_bits, f16_value)
    sb, ab = to_bits(s), to_bits(a)
    w = (u.astype(np.float64) - np.repeat(z, g, axis=0)) * np.repeat(to_val(sb), g, axis=0)
    out = to_val(ab) @ w
    d = dict(u=u, scales_bits=sb, act_bits=ab, out=out.astype(np.float32), group=np.int64(g), bf16=np.int64(bf16))
    if awq:
        d.update(qweight=awq_pack(u), qzeros=awq_pack(z), z=z)
    else:
        d.update(qweight=gptq_pack(u))
    return d


CUTLASS_ROW_MAP = [0, 1, 8, 9, 16, 17, 24, 25, 2, 3, 10, 11, 18, 19, 26, 27,
                   4, 5, 12, 13, 20, 21, 28, 29, 6, 7, 14, 15, 22, 23, 30, 31]


def pack_nibbles(n):
    n = n.reshape(-1).astype(np.uint8)
    return (n[0::2] | (n[1::2] << 4)).astype(np.uint8)


def cutlass_sm80(u):
    """u [K, N] unsigned -> bytes: rows permuted in groups of 32, column major, tiles of 64 rows with four columns
    interleaved, elements [0,2,4,6,1,3,5,7] inside every group of eight, unsigned."""
    K, N = u.shape
    p1 = u.reshape(K // 32, 32, N)[:, CUTLASS_ROW_MAP, :].reshape(K, N)
    regs = p1.T.reshape(N // 4, 4, K // 64, 8, 8)            # [column group, column, row tile, register, element]
    regs = regs.transpose(0, 2, 1, 3, 4)                     # row tile outside the four columns
    regs = regs[..., AWQ_ORDER]                              # the register relayout is the same order
    return pack_nibbles(regs)


def cutlass_sm90(u):
    return pack_nibbles(((u.astype(np.int16) - 8) & 0xF).T)  # transpose only, nibbles stay signed


def marlin_weights(u):
    K, N = u.shape
    perm = []
    for i in range(32):
        perm1 = []
        for block in (0, 1):
            for row in (2 * (i % 4), 2 * (i % 4) + 1, 2 * (i % 4 + 4), 2 * (i % 4 + 4) + 1):
                perm1.append(16 * row + i // 4 + 8 * block)
        for j in range(4):
            perm.extend(p + 256 * j for p in perm1)
    perm = np.array(perm).reshape(-1, 8)[:, AWQ_ORDER].ravel()
    q = u.astype(np.uint32).reshape(K // 16, 16, N // 16, 16).transpose(0, 2, 1, 3).reshape(-1, perm.size)[:, perm]
    q = q.reshape(K // 16, N * 16)
    packed = np.zeros((K // 16, N * 2), dtype=np.uint32)
    for i in range(8):
        packed |= q[:, i::8] << np.uint32(4 * i)
    return packed.view(np.int32)


def marlin_scales(s):
    G, N = s.shape
    return np.ascontiguousarray(s.reshape(G, N // 64, 8, 8).transpose(0, 1, 3, 2).reshape(G, N))


def marlin_zero_points(z):
    G, N = z.shape
    zp = marlin_scales(z).reshape(-1, 8)[:, AWQ_ORDER].reshape(G, N).astype(np.uint32)
    packed = np.zeros((G, N // 8), dtype=np.uint32)
    for i in range(8):
        packed |= zp[:, i::8] << np.uint32(4 * i)
    return packed.view(np.int32)


def next_case(seed, M, K, N, g):
    rng = np.random.default_rng(seed)
    u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    sb = f16_bits(np.abs(rng.standard_normal((K // g, N))).astype(np.float32) * 0.02 + 1e-3)
    ab = f16_bits(rng.standard_normal((M, K)).astype(np.float32))
    bias = f16_bits(rng.standard_normal(N).astype(np.float32))
    sv, av = f16_value(sb), f16_value(ab)
    out = av @ ((u.astype(np.float64) - np.repeat(z, g, axis=0)) * np.repeat(sv, g, axis=0))
    order = rng.permutation(K)
    g_idx = np.empty(K, dtype=np.int32)
    g_idx[order] = np.arange(K, dtype=np.int32) // g
    out_desc = av @ ((u.astype(np.float64) - 8.0) * sv[g_idx])
    gate, up = out[:, : N // 2], out[:, N // 2:]
    return dict(u=u, z=z, scales_bits=sb, act_bits=ab, bias_bits=bias, group=np.int64(g),
                qweight_gptq=gptq_pack(u), qweight_awq=awq_pack(u), qzeros_awq=awq_pack(z),
                cutlass80=cutlass_sm80(u), cutlass90=cutlass_sm90(u), marlin=marlin_weights(u),
                marlin_scales_bits=marlin_scales(sb), marlin_zp=marlin_zero_points(z),
                g_idx=g_idx, perm=np.argsort(g_idx, kind="stable").astype(np.int32),
                out=out.astype(np.float32), out_desc=out_desc.astype(np.float32),
                out_silu=(gate / (1.0 + np.exp(-gate)) * up).astype(np.float32),
                out_bias=(out + f16_value(bias)[None, :]).astype(np.float32))


def main():
    rng = np.random.default_rng(20240607)
    table = e4m3_table()

    u = rng.integers(0, 16, size=(64, 64), dtype=np.uint8)
    np.savez_compressed(os.path.join(HERE, "gptq_64x64.npz"), u=u, qweight=gptq_pack(u), rowmajor=rowmajor_pack(u))
    u = rng.integers(0, 16, size=(128, 64), dtype=np.uint8)
    z = rng.integers(0, 16, size=(1, 64), dtype=np.uint8)
    np.savez_compressed(os.path.join(HERE, "awq_128x64.npz"), u=u, qweight=awq_pack(u), z=z, qzeros=awq_pack(z),
                        rowmajor=rowmajor_pack(u))
    np.savez_compressed(os.path.join(HERE, "e4m3_table.npz"), value=table)

    np.savez_compressed(os.path.join(HERE, "w4a16_gptq_f16_16x256x128.npz"), **w4a16_case(1, 16, 256, 128, 128, False, False))
    np.savez_compressed(os.path.join(HERE, "w4a16_awq_f16_5x256x64_g64.npz"), **w4a16_case(2, 5, 256, 64, 64, True, False))
    np.savez_compressed(os.path.join(HERE, "w4a16_awq_bf16_16x384x128.npz"), **w4a16_case(3, 16, 384, 128, 128, True, True))
    np.savez_compressed(os.path.join(HERE, "w4a16_awq_bf16_130x256x272.npz"), **w4a16_case(4, 130, 256, 272, 128, True, True))

    # K an odd multiple of 64 (group size 64), and bf16 scales spread over 2^-40 .. 2^40 from column to column
    np.savez_compressed(os.path.join(HERE, "w4a16_gptq_f16_7x192x64_g64.npz"), **w4a16_case(6, 7, 192, 64, 64, False, False))
    np.savez_compressed(os.path.join(HERE, "w4a16_awq_bf16_9x256x64_wide.npz"),
                        **w4a16_case(7, 9, 256, 64, 128, True, True, column_exponents=40))

    np.savez_compressed(os.path.join(HERE, "w4a16_next_f16_12x256x128.npz"), **next_case(5, 12, 256, 128, 128))

    # FP8 activation quantisation, per token, fp16 input 8 x 256
    x = (rng.standard_normal((8, 256)) * 0.7).astype(np.float32)
    xb = f16_bits(x)
    xv = f16_value(xb).astype(np.float32)
    scale = np.maximum(np.abs(xv).max(axis=1) / np.float32(448.0), np.float32(1.0 / (448.0 * 512.0))).astype(np.float32)
    ratio = np.clip((xv / scale[:, None]).astype(np.float32), -448.0, 448.0)
    aq = e4m3_encode(ratio.astype(np.float64), table)
    # FP8 weight 64 x 256 with per-channel scales, and the GEMM 8 x 256 x 64
    wq = rng.integers(0, 256, size=(64, 256), dtype=np.uint8)
    wq[(wq & 0x7F) == 0x7F] = 0x30
    w_scale = (rng.random(64).astype(np.float32) * 0.01 + 1e-3).astype(np.float32)
    out = (table[aq] @ table[wq].T) * w_scale.astype(np.float64)[None, :] * scale.astype(np.float64)[:, None]
    np.savez_compressed(os.path.join(HERE, "fp8_8x256x64.npz"), x_bits=xb, a_scale=scale, aq=aq, wq=wq, w_scale=w_scale,
                        out=out.astype(np.float32))


if __name__ == "__main__":
    main()
