"""numpy front end of the CPU oracle (``ksq_oracle.c``).

Test infrastructure only.  The shipped package never imports this module; the parity tests, the smoke
test and the bench's host-core baseline leg do.  Each wrapper keeps the name of the C function it calls;
the C file cites the reference code every function restates.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libksq_oracle.so")

F16, BF16, F32 = 0, 1, 2


def build(force=False):
    """Compile ksq_oracle.c with gcc (only when missing unless ``force``)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.orc_e4m3_decode.restype = ctypes.c_float
        _lib.orc_e4m3_decode.argtypes = [ctypes.c_uint8]
        _lib.orc_e4m3_encode.restype = ctypes.c_uint8
        _lib.orc_e4m3_encode.argtypes = [ctypes.c_float]
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _sz(x):
    return ctypes.c_size_t(int(x))


def _c(a, dtype=None):
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != dtype:
        raise TypeError(f"expected {dtype}, got {a.dtype}")
    return a


# ---------------------------------------------------------------- 16-bit float helpers
def to_bits(x, dtype):
    """fp32 array -> uint16 bit patterns of fp16 / bf16 (round to nearest even)."""
    x = _c(np.asarray(x, dtype=np.float32))
    if dtype == F32:
        return x.copy()
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_from_f32(_p(x), dtype, _sz(x.size), _p(out))
    return out


def from_bits(b, dtype):
    """uint16 bit patterns (or fp32) -> fp32 values."""
    b = _c(b)
    if dtype == F32:
        return b.astype(np.float32)
    out = np.empty(b.shape, dtype=np.float32)
    lib().orc_to_f32(_p(_c(b, np.uint16)), dtype, _sz(b.size), _p(out))
    return out


# ---------------------------------------------------------------- layouts
def gptq_unpack(qweight):
    qweight = _c(qweight, np.int32)
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    u = np.empty((K, N), dtype=np.uint8)
    lib().orc_gptq_unpack(_p(qweight), _sz(K), _sz(N), _p(u))
    return u


def gptq_pack(u):
    u = _c(u, np.uint8)
    K, N = u.shape
    q = np.empty((K // 8, N), dtype=np.int32)
    lib().orc_gptq_pack(_p(u), _sz(K), _sz(N), _p(q))
    return q


def awq_unpack(q):
    q = _c(q, np.int32)
    R, N = q.shape[0], q.shape[1] * 8
    u = np.empty((R, N), dtype=np.uint8)
    lib().orc_awq_unpack(_p(q), _sz(R), _sz(N), _p(u))
    return u


def awq_pack(u):
    u = _c(u, np.uint8)
    R, N = u.shape
    q = np.empty((R, N // 8), dtype=np.int32)
    lib().orc_awq_pack(_p(u), _sz(R), _sz(N), _p(q))
    return q


def rowmajor_pack(u):
    u = _c(u, np.uint8)
    K, N = u.shape
    p = np.empty((K, N // 2), dtype=np.uint8)
    lib().orc_rowmajor_pack(_p(u), _sz(K), _sz(N), _p(p))
    return p


def rowmajor_unpack(p):
    p = _c(p, np.uint8)
    K, N = p.shape[0], p.shape[1] * 2
    u = np.empty((K, N), dtype=np.uint8)
    lib().orc_rowmajor_unpack(_p(p), _sz(K), _sz(N), _p(u))
    return u


def awq_additive_zeros(scales_bits, dtype, z):
    scales_bits = _c(scales_bits, np.uint16)
    z = _c(z, np.uint8)
    G, N = z.shape
    out = np.empty((G, N), dtype=np.uint16)
    lib().orc_awq_additive_zeros(_p(scales_bits), dtype, _p(z), _sz(G), _sz(N), _p(out))
    return out


# ---------------------------------------------------------------- dequantize-then-GEMM
def dequant(u, scales_bits, sdtype, z, g, out=None):
    """fp32 [K,N] = s * (u - z); ``out`` = a C-contiguous float32 [K,N] buffer to fill instead of a new array."""
    u = _c(u, np.uint8)
    scales_bits = _c(scales_bits)
    z = _c(z, np.uint8) if z is not None else None
    K, N = u.shape
    w = np.empty((K, N), dtype=np.float32) if out is None else out
    assert w.shape == (K, N) and w.dtype == np.float32 and w.flags.c_contiguous
    lib().orc_dequant(_p(u), _p(scales_bits), sdtype, _p(z), _sz(K), _sz(N), _sz(g), _p(w))
    return w


def dequant_additive(u, scales_bits, sdtype, zeros_additive_bits, g):
    u = _c(u, np.uint8)
    scales_bits = _c(scales_bits)
    za = _c(zeros_additive_bits) if zeros_additive_bits is not None else None
    K, N = u.shape
    w = np.empty((K, N), dtype=np.float32)
    lib().orc_dequant_additive(_p(u), _p(scales_bits), sdtype, _p(za), _sz(K), _sz(N), _sz(g), _p(w))
    return w


def gemm_f32(a, w):
    a = _c(a, np.float32)
    w = _c(w, np.float32)
    M, K = a.shape
    N = w.shape[1]
    out = np.empty((M, N), dtype=np.float32)
    lib().orc_gemm_f32(_p(a), _p(w), _sz(M), _sz(N), _sz(K), _p(out))
    return out


def gemm_f64acc(a, w):
    a = _c(a, np.float32)
    w = _c(w, np.float32)
    M, K = a.shape
    N = w.shape[1]
    out = np.empty((M, N), dtype=np.float64)
    lib().orc_gemm_f64acc(_p(a), _p(w), _sz(M), _sz(N), _sz(K), _p(out))
    return out


def w4a16_forward(act_bits, adtype, u, scales_bits, sdtype, z, g, scratch=None):
    """Dequantize to fp32 + blocked GEMM; returns fp32 [M,N].  ``scratch`` = (w[K,N], a[M,K]) float32
    buffers to reuse between calls (the bench's host-core baseline passes them so only compute is timed)."""
    act_bits = _c(act_bits)
    u = _c(u, np.uint8)
    scales_bits = _c(scales_bits)
    z = _c(z, np.uint8) if z is not None else None
    M, K = act_bits.shape
    N = u.shape[1]
    if scratch is None:
        scratch = (np.empty((K, N), dtype=np.float32), np.empty((M, K), dtype=np.float32))
    out = np.empty((M, N), dtype=np.float32)
    lib().orc_w4a16_forward(_p(act_bits), adtype, _p(u), _p(scales_bits), sdtype, _p(z), _sz(M), _sz(N), _sz(K),
                            _sz(g), _p(scratch[0]), _p(scratch[1]), _p(out))
    return out


# ---------------------------------------------------------------- FP8
def e4m3_decode(codes):
    codes = _c(codes, np.uint8)
    table = np.array([lib().orc_e4m3_decode(i) for i in range(256)], dtype=np.float32)
    return table[codes]


def e4m3_encode(x):
    x = _c(np.asarray(x, dtype=np.float32))
    f = lib().orc_e4m3_encode
    return np.array([f(float(v)) for v in x.ravel()], dtype=np.uint8).reshape(x.shape)


def fp8_compute_scale(x_bits, dtype, num_channels, channel_size):
    x_bits = _c(x_bits)
    s = np.empty((num_channels,), dtype=np.float32)
    lib().orc_fp8_compute_scale(_p(x_bits), dtype, _sz(num_channels), _sz(channel_size), _p(s))
    return s


def fp8_quantize(x_bits, dtype, scale, num_channels, channel_size):
    x_bits = _c(x_bits)
    scale = _c(scale, np.float32)
    q = np.empty((num_channels, channel_size), dtype=np.uint8)
    lib().orc_fp8_quantize(_p(x_bits), dtype, _p(scale), _sz(num_channels), _sz(channel_size), _p(q))
    return q


def fp8_rescale(q, s_in, s_out):
    q = _c(q, np.uint8)
    out = np.empty_like(q)
    lib().orc_fp8_rescale(_p(q), _sz(q.size), ctypes.c_float(s_in), ctypes.c_float(s_out), _p(out))
    return out


def fp8_gemm(aq, a_scale, wq, w_scale):
    aq = _c(aq, np.uint8)
    wq = _c(wq, np.uint8)
    a_scale = _c(np.atleast_1d(a_scale), np.float32)
    w_scale = _c(np.atleast_1d(w_scale), np.float32)
    M, K = aq.shape
    N = wq.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    lib().orc_fp8_gemm(_p(aq), _p(a_scale), _sz(a_scale.size), _p(wq), _p(w_scale), _sz(w_scale.size), _sz(M),
                       _sz(N), _sz(K), _p(out))
    return out


def fp8_convert_weight(w_kn_bits, dtype):
    w_kn_bits = _c(w_kn_bits)
    K, N = w_kn_bits.shape
    wq = np.empty((N, K), dtype=np.uint8)
    s = np.empty((1,), dtype=np.float32)
    lib().orc_fp8_convert_weight(_p(w_kn_bits), dtype, _sz(K), _sz(N), _p(wq), _p(s))
    return wq, s


def fp8_convert_weight_per_channel(w_kn_bits, dtype):
    w_kn_bits = _c(w_kn_bits)
    K, N = w_kn_bits.shape
    wq = np.empty((N, K), dtype=np.uint8)
    s = np.empty((N,), dtype=np.float32)
    lib().orc_fp8_convert_weight_per_channel(_p(w_kn_bits), dtype, _sz(K), _sz(N), _p(wq), _p(s))
    return wq, s


def fp8_merge_qkv_max(wq, q_scale, k_scale, v_scale, nq, nk, nv):
    """KS/models/quant/quant_weight.cpp:816-897: one scale = max of the three, every row range requantised as
    e4m3(float(w) * (part_scale / max_scale)).  Returns (merged weight, scale[1])."""
    merged = np.array([max(float(q_scale), float(k_scale), float(v_scale))], dtype=np.float32)
    out = np.array(wq, copy=True)
    row = 0
    for rows, s in ((nq, q_scale), (nk, k_scale), (nv, v_scale)):
        part = out[row:row + rows].reshape(-1)
        out[row:row + rows] = fp8_rescale(part, np.float32(s), merged[0]).reshape(rows, -1)
        row += rows
    return out, merged


# ---------------------------------------------------------------- layouts the loader's back ends leave behind
def cutlass_preprocess(rowmajor, arch=80):
    """Output bytes of preprocess_weights_for_mixed_gemm (W4_A16) for a row-major signed int4 tensor [K, N/2]."""
    rowmajor = _c(rowmajor, np.uint8)
    K, N = rowmajor.shape[0], rowmajor.shape[1] * 2
    out = np.empty(K * N // 2, dtype=np.uint8)
    lib().orc_cutlass_preprocess(_p(rowmajor), _sz(K), _sz(N), int(arch), _p(out))
    return out


def cutlass_step(step, data, K, N):
    """One step of the preprocessor on a whole buffer of K*N/2 bytes: 'permute_rows', 'transpose',
    'interleave_columns' or 'bias_and_interleave'."""
    data = _c(data, np.uint8).reshape(-1)
    assert data.size == K * N // 2
    if step == "bias_and_interleave":
        out = data.copy()
        lib().orc_cutlass_bias_and_interleave(_p(out), _sz(out.size // 4))
        return out
    out = np.zeros_like(data)
    getattr(lib(), "orc_cutlass_" + step)(_p(data), _sz(K), _sz(N), _p(out))
    return out


def marlin_repack(qweight, K, N, kind):
    """kind 'gptq': int32 [K/8, N]; 'awq': int32 [K, N/8].  Returns the Marlin weight, int32 [K/16, N*2]."""
    q = _c(qweight).view(np.uint32)
    out = np.zeros((K // 16, N * 2), dtype=np.uint32)
    getattr(lib(), "orc_marlin_repack_" + kind)(_p(q), _sz(K), _sz(N), _p(out))
    return out.view(np.int32)


def marlin_permute_scales(s, K, group_size):
    """MarlinPermuteScales (KS/models/quant/quant_weight.cpp:350-375) on a [G, N] array of any 16-bit dtype."""
    s = np.ascontiguousarray(s)
    N = s.shape[1]
    if group_size < K and group_size != -1:
        perm = [i + 8 * j for i in range(8) for j in range(8)]
    else:
        perm = [2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)]
    return np.ascontiguousarray(s.reshape(-1, len(perm))[:, perm].reshape(-1, N))


def marlin_zero_points(z):
    """MarlinZeroPoints (quant_weight.cpp:397-426) for 4 bits: z uint8 [G, N] -> int32 [G, N/8]."""
    z = _c(z, np.uint8)
    G, N = z.shape
    perm = [i + 8 * j for i in range(8) for j in range(8)]
    zp = z.reshape(-1, 64)[:, perm]
    zp = zp.reshape(-1, 8)[:, [0, 2, 4, 6, 1, 3, 5, 7]].reshape(G, N).astype(np.uint32)
    packed = np.zeros((G, N // 8), dtype=np.uint32)
    for i in range(8):  # MarlinPackCols (:385-395)
        packed |= zp[:, i::8] << np.uint32(4 * i)
    return packed.view(np.int32)


def act_order_perm(g_idx):
    g_idx = _c(g_idx, np.int32)
    perm = np.empty(g_idx.shape[0], dtype=np.int32)
    lib().orc_act_order_perm(_p(g_idx), _sz(g_idx.shape[0]), _p(perm))
    return perm


def silu_mul(acc):
    """acc [M, 2H] fp32 = [gate | up] -> silu(gate) * up, [M, H] fp32."""
    acc = _c(acc, np.float32)
    M, H = acc.shape[0], acc.shape[1] // 2
    out = np.empty((M, H), dtype=np.float32)
    lib().orc_silu_mul(_p(acc), _sz(M), _sz(H), _p(out))
    return out


def num_threads():
    return int(lib().orc_num_threads())


# ---------------------------------------------------------------- error metrics of the parity bar
def error_metrics(got, want):
    """max relative error with the denominator floored at RMS(want), and mean absolute error / RMS(want).

    max_rel = max_i |got_i - want_i| / max(|want_i|, RMS(want));   mean_abs_over_rms = mean_i |got_i - want_i| / RMS(want)
    """
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    rms = float(np.sqrt(np.mean(want * want))) if want.size else 0.0
    if rms == 0.0:
        rms = 1.0
    diff = np.abs(got - want)
    max_rel = float(np.max(diff / np.maximum(np.abs(want), rms))) if want.size else 0.0
    return {"max_rel": max_rel, "mean_abs_over_rms": float(np.mean(diff) / rms) if want.size else 0.0, "rms": rms}


MAX_REL_TOL = 1e-2
MEAN_ABS_TOL = 2e-3


def assert_parity(got, want, what=""):
    m = error_metrics(got, want)
    assert np.all(np.isfinite(np.asarray(got, dtype=np.float64))), f"{what}: non-finite output"
    assert m["max_rel"] <= MAX_REL_TOL, f"{what}: max_rel {m['max_rel']:.3e} > {MAX_REL_TOL}"
    assert m["mean_abs_over_rms"] <= MEAN_ABS_TOL, f"{what}: mean_abs/rms {m['mean_abs_over_rms']:.3e} > {MEAN_ABS_TOL}"
    return m
