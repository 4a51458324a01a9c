"""ctypes binding of libksq.so (the C ABI declared in include/ksq.h).

Every wrapper takes raw device (or host) addresses as Python ints, or objects with ``data_ptr()`` (torch tensors)
/ ``ctypes.data`` (numpy arrays), and raises :class:`KsqError` on a non-zero status.  Nothing here computes: a
missing or unloadable library is an ImportError-like failure, never a fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libksq.so")

# enums of include/ksq.h
F16, BF16, F32 = 0, 1, 2  # F32: the FP8 entry points only
W4_GPTQ_INT32_KPACK, W4_AWQ_INT32_NPACK, W4_ROWMAJOR_INT4_SIGNED = 0, 1, 2
W4_CUTLASS_SM80_INTERLEAVED, W4_CUTLASS_SM90_COLMAJOR, W4_MARLIN = 3, 4, 5
COLS_NATURAL, COLS_HALVES_INTERLEAVED = 0, 1
EPILOGUE_NONE, EPILOGUE_BIAS, EPILOGUE_SILU_MUL = 0, 1, 2
ZERO_NONE, ZERO_AWQ_INT32, ZERO_UINT8, ZERO_ADDITIVE, ZERO_MARLIN_INT32 = 0, 1, 2, 3, 4
FP8_PER_TENSOR_DYNAMIC, FP8_PER_TENSOR_STATIC, FP8_PER_TOKEN_DYNAMIC = 0, 1, 2
FP8_MERGE_MAX, FP8_MERGE_PER_CHANNEL = 0, 1
OK, ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_HIP = 0, -1, -2, -3, -4

EXPORTS = [
    "ksq_version", "ksq_last_error_string", "ksq_device_compute_units",
    "ksq_w4a16_repack_sizes", "ksq_w4a16_repack", "ksq_w4a16_repack_host",
    "ksq_w4a16_workspace_bytes", "ksq_w4a16_gemm",
    "ksq_fp8_quantize", "ksq_fp8_rescale", "ksq_fp8_convert_weight",
    "ksq_fp8_convert_weight_per_channel", "ksq_fp8_merge_qkv_scales", "ksq_fp8_workspace_bytes", "ksq_fp8_gemm",
    "ksq_w4a16_repack_ex", "ksq_w4a16_repack_ex_host", "ksq_gptq_act_order_perm", "ksq_permute_columns",
    "ksq_w4a16_workspace_bytes_ex", "ksq_w4a16_gemm_ex", "ksq_fp8_gemm_ex", "ksq_interleave_halves",
    "ksq_w4a16_gemm_static_scratch", "ksq_fp8_gemm_dynamic_workspace_bytes", "ksq_fp8_gemm_dynamic",
    "ksq_set_launch_log", "ksq_last_launch_string", "ksq_bind_splitk_counters",
    "ksq_fill_zero_f32", "ksq_w4a16_gemm_rowmax", "ksq_fp8_gemm_rowmax", "ksq_fp8_quantize_rows_from_absmax",
]
SPLITK_COUNTER_BYTES = 65536
STATIC_SCRATCH_BYTES = 64 << 20


class KsqError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"ksq error {code}: {message}")
        self.code = code


_lib = None


def _bind(L):
    """Declare the argument and result types of every entry point of include/ksq.h on a loaded library."""
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    psz = ctypes.POINTER(ctypes.c_size_t)
    L.ksq_version.restype = ci
    L.ksq_last_error_string.restype = ctypes.c_char_p
    L.ksq_device_compute_units.restype = ci
    L.ksq_w4a16_repack_sizes.argtypes = [sz, sz, sz, psz, psz]
    L.ksq_w4a16_repack.argtypes = [ci, vp, ci, vp, vp, ci, sz, sz, sz, vp, vp, vp]
    L.ksq_w4a16_repack_host.argtypes = [ci, vp, ci, vp, vp, ci, sz, sz, sz, vp, vp]
    L.ksq_w4a16_workspace_bytes.argtypes = [sz, sz, sz, psz]
    L.ksq_w4a16_gemm.argtypes = [ci, vp, vp, vp, vp, sz, sz, sz, sz, vp, sz, vp]
    L.ksq_fp8_quantize.argtypes = [ci, vp, sz, sz, ci, vp, vp, vp]
    L.ksq_fp8_rescale.argtypes = [vp, vp, sz, vp, vp, vp]
    L.ksq_fp8_convert_weight.argtypes = [ci, vp, sz, sz, vp, vp, vp]
    L.ksq_fp8_convert_weight_per_channel.argtypes = [ci, vp, sz, sz, vp, vp, vp]
    L.ksq_fp8_merge_qkv_scales.argtypes = [ci, vp, vp, vp, sz, sz, sz, vp, sz, vp, vp]
    L.ksq_fp8_workspace_bytes.argtypes = [sz, sz, sz, psz]
    L.ksq_fp8_gemm.argtypes = [ci, vp, vp, vp, sz, vp, vp, sz, sz, sz, sz, vp, sz, vp]
    L.ksq_w4a16_repack_ex.argtypes = [ci, vp, ci, vp, vp, ci, sz, sz, sz, vp, ci, vp, vp, vp]
    L.ksq_w4a16_repack_ex_host.argtypes = [ci, vp, ci, vp, vp, ci, sz, sz, sz, vp, ci, vp, vp]
    L.ksq_gptq_act_order_perm.argtypes = [vp, sz, sz, vp]
    L.ksq_permute_columns.argtypes = [vp, vp, vp, sz, sz, vp]
    L.ksq_w4a16_workspace_bytes_ex.argtypes = [sz, sz, sz, ci, psz]
    L.ksq_w4a16_gemm_ex.argtypes = [ci, vp, vp, vp, vp, sz, sz, sz, sz, vp, ci, vp, vp, sz, vp]
    L.ksq_fp8_gemm_ex.argtypes = [ci, vp, vp, vp, sz, vp, vp, sz, sz, sz, sz, ci, vp, vp, sz, vp]
    L.ksq_interleave_halves.argtypes = [vp, vp, sz, sz, vp]
    L.ksq_w4a16_gemm_static_scratch.argtypes = [ci, vp, vp, vp, vp, sz, sz, sz, sz, vp]
    L.ksq_fp8_gemm_dynamic_workspace_bytes.argtypes = [sz, sz, sz, psz]
    L.ksq_fp8_gemm_dynamic.argtypes = [ci, vp, vp, vp, vp, sz, sz, sz, sz, ci, vp, vp, sz, vp]
    L.ksq_set_launch_log.argtypes = [ci]
    L.ksq_set_launch_log.restype = None
    L.ksq_last_launch_string.restype = ctypes.c_char_p
    L.ksq_bind_splitk_counters.argtypes = [vp, vp, sz]
    L.ksq_fill_zero_f32.argtypes = [vp, sz, vp]
    L.ksq_w4a16_gemm_rowmax.argtypes = [ci, vp, vp, vp, vp, sz, sz, sz, sz, ci, vp, vp, vp, sz, vp]
    L.ksq_fp8_gemm_rowmax.argtypes = [ci, vp, vp, vp, sz, vp, vp, sz, sz, sz, sz, ci, vp, vp, vp, sz, vp]
    L.ksq_fp8_quantize_rows_from_absmax.argtypes = [ci, vp, sz, sz, vp, vp, vp, vp]
    for name in EXPORTS:
        if name not in ("ksq_last_error_string", "ksq_set_launch_log", "ksq_last_launch_string"):
            getattr(L, name).restype = ci
    return L


def lib():
    """Load libksq.so; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise KsqError(ERR_HIP, f"{LIB_PATH} is missing: build it with `python -m ksanallm_amd.build`")
        _lib = _bind(ctypes.CDLL(LIB_PATH))
    return _lib


def _addr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    if hasattr(x, "ctypes"):
        return x.ctypes.data
    raise TypeError(f"cannot take the address of {type(x)}")


def _check(code):
    if code != OK:
        raise KsqError(code, lib().ksq_last_error_string().decode())


def version():
    return lib().ksq_version()


def set_launch_log(enabled=True):
    lib().ksq_set_launch_log(1 if enabled else 0)


def last_launch():
    """What the calling thread's last GEMM call launched (needs set_launch_log first)."""
    return lib().ksq_last_launch_string().decode()


def bind_splitk_counters(stream, counters, nbytes=None):
    """Bind caller-owned, zero-filled device memory as the split-K arrival counters of `stream` (None unbinds)."""
    n = 0 if counters is None else (nbytes if nbytes is not None else counters.numel() * counters.element_size())
    _check(lib().ksq_bind_splitk_counters(stream, _addr(counters), n))


def device_compute_units():
    return lib().ksq_device_compute_units()


def w4a16_repack_sizes(k, n, group_size):
    wb, sb = ctypes.c_size_t(0), ctypes.c_size_t(0)
    _check(lib().ksq_w4a16_repack_sizes(k, n, group_size, ctypes.byref(wb), ctypes.byref(sb)))
    return wb.value, sb.value


def w4a16_repack(src_layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, group_size, dst_weight, dst_sz,
                 stream=None):
    _check(lib().ksq_w4a16_repack(src_layout, _addr(qweight), zero_kind, _addr(zeros), _addr(scales), scale_dtype, k,
                                  n, group_size, _addr(dst_weight), _addr(dst_sz), stream))


def w4a16_repack_host(src_layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, group_size, dst_weight,
                      dst_sz):
    _check(lib().ksq_w4a16_repack_host(src_layout, _addr(qweight), zero_kind, _addr(zeros), _addr(scales),
                                       scale_dtype, k, n, group_size, _addr(dst_weight), _addr(dst_sz)))


def w4a16_repack_ex(src_layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, group_size, row_perm,
                    column_order, dst_weight, dst_sz, stream=None):
    _check(lib().ksq_w4a16_repack_ex(src_layout, _addr(qweight), zero_kind, _addr(zeros), _addr(scales), scale_dtype,
                                     k, n, group_size, _addr(row_perm), column_order, _addr(dst_weight),
                                     _addr(dst_sz), stream))


def w4a16_repack_ex_host(src_layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, group_size, row_perm,
                         column_order, dst_weight, dst_sz):
    _check(lib().ksq_w4a16_repack_ex_host(src_layout, _addr(qweight), zero_kind, _addr(zeros), _addr(scales),
                                          scale_dtype, k, n, group_size, _addr(row_perm), column_order,
                                          _addr(dst_weight), _addr(dst_sz)))


def gptq_act_order_perm(g_idx, k, group_size, perm):
    """Host arrays (numpy int32) in, host array out."""
    _check(lib().ksq_gptq_act_order_perm(_addr(g_idx), k, group_size, _addr(perm)))


def permute_columns(out, src, perm, m, k, stream=None):
    _check(lib().ksq_permute_columns(_addr(out), _addr(src), _addr(perm), m, k, stream))


def interleave_halves(out, src, rows, row_bytes, stream=None):
    _check(lib().ksq_interleave_halves(_addr(out), _addr(src), rows, row_bytes, stream))


def w4a16_workspace_bytes_ex(max_m, n, k, act_order):
    b = ctypes.c_size_t(0)
    _check(lib().ksq_w4a16_workspace_bytes_ex(max_m, n, k, int(bool(act_order)), ctypes.byref(b)))
    return b.value


def w4a16_gemm_ex(dtype, out, act, weight, sz, m, n, k, group_size, act_perm=None, epilogue=EPILOGUE_NONE, bias=None,
                  workspace=None, workspace_bytes=0, stream=None):
    _check(lib().ksq_w4a16_gemm_ex(dtype, _addr(out), _addr(act), _addr(weight), _addr(sz), m, n, k, group_size,
                                   _addr(act_perm), epilogue, _addr(bias), _addr(workspace), workspace_bytes, stream))


def w4a16_workspace_bytes(max_m, n, k):
    b = ctypes.c_size_t(0)
    _check(lib().ksq_w4a16_workspace_bytes(max_m, n, k, ctypes.byref(b)))
    return b.value


def w4a16_gemm(dtype, out, act, weight, sz, m, n, k, group_size, workspace=None, workspace_bytes=0, stream=None):
    _check(lib().ksq_w4a16_gemm(dtype, _addr(out), _addr(act), _addr(weight), _addr(sz), m, n, k, group_size,
                                _addr(workspace), workspace_bytes, stream))


def w4a16_gemm_static_scratch(dtype, out, act, weight, sz, m, n, k, group_size, stream=None):
    _check(lib().ksq_w4a16_gemm_static_scratch(dtype, _addr(out), _addr(act), _addr(weight), _addr(sz), m, n, k,
                                               group_size, stream))


def fp8_gemm_dynamic_workspace_bytes(max_m, n, k):
    b = ctypes.c_size_t(0)
    _check(lib().ksq_fp8_gemm_dynamic_workspace_bytes(max_m, n, k, ctypes.byref(b)))
    return b.value


def fp8_gemm_dynamic(dtype, out, act, w_q, w_scale, w_scale_count, m, n, k, epilogue=EPILOGUE_NONE, bias=None,
                     workspace=None, workspace_bytes=0, stream=None):
    _check(lib().ksq_fp8_gemm_dynamic(dtype, _addr(out), _addr(act), _addr(w_q), _addr(w_scale), w_scale_count, m, n, k,
                                      epilogue, _addr(bias), _addr(workspace), workspace_bytes, stream))


def fill_zero_f32(p, count, stream=None):
    _check(lib().ksq_fill_zero_f32(_addr(p), count, stream))


def w4a16_gemm_rowmax(dtype, out, act, weight, sz, m, n, k, group_size, row_absmax, epilogue=EPILOGUE_NONE, bias=None,
                      workspace=None, workspace_bytes=0, stream=None):
    _check(lib().ksq_w4a16_gemm_rowmax(dtype, _addr(out), _addr(act), _addr(weight), _addr(sz), m, n, k, group_size,
                                       epilogue, _addr(bias), _addr(row_absmax), _addr(workspace), workspace_bytes, stream))


def fp8_gemm_rowmax(out_dtype, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m, n, k, row_absmax,
                    epilogue=EPILOGUE_NONE, bias=None, workspace=None, workspace_bytes=0, stream=None):
    _check(lib().ksq_fp8_gemm_rowmax(out_dtype, _addr(out), _addr(act_q), _addr(act_scale), act_scale_count, _addr(w_q),
                                     _addr(w_scale), w_scale_count, m, n, k, epilogue, _addr(bias), _addr(row_absmax),
                                     _addr(workspace), workspace_bytes, stream))


def fp8_quantize_rows_from_absmax(dtype, act, m, k, row_absmax, act_q, act_scale, stream=None):
    _check(lib().ksq_fp8_quantize_rows_from_absmax(dtype, _addr(act), m, k, _addr(row_absmax), _addr(act_q),
                                                   _addr(act_scale), stream))


def fp8_quantize(dtype, act, m, k, mode, act_q, act_scale, stream=None):
    _check(lib().ksq_fp8_quantize(dtype, _addr(act), m, k, mode, _addr(act_q), _addr(act_scale), stream))


def fp8_rescale(src, dst, count, scale_in, scale_out, stream=None):
    _check(lib().ksq_fp8_rescale(_addr(src), _addr(dst), count, _addr(scale_in), _addr(scale_out), stream))


def fp8_convert_weight(dtype, w, k, n, w_q, w_scale, stream=None):
    _check(lib().ksq_fp8_convert_weight(dtype, _addr(w), k, n, _addr(w_q), _addr(w_scale), stream))


def fp8_convert_weight_per_channel(dtype, w, k, n, w_q, w_scale, stream=None):
    _check(lib().ksq_fp8_convert_weight_per_channel(dtype, _addr(w), k, n, _addr(w_q), _addr(w_scale), stream))


def fp8_merge_qkv_scales(mode, q_scale, k_scale, v_scale, nq, nk, nv, w_q, k, w_scale, stream=None):
    _check(lib().ksq_fp8_merge_qkv_scales(mode, _addr(q_scale), _addr(k_scale), _addr(v_scale), nq, nk, nv, _addr(w_q), k,
                                          _addr(w_scale), stream))


def fp8_workspace_bytes(max_m, n, k):
    b = ctypes.c_size_t(0)
    _check(lib().ksq_fp8_workspace_bytes(max_m, n, k, ctypes.byref(b)))
    return b.value


def fp8_gemm(out_dtype, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m, n, k, workspace=None,
             workspace_bytes=0, stream=None):
    _check(lib().ksq_fp8_gemm(out_dtype, _addr(out), _addr(act_q), _addr(act_scale), act_scale_count, _addr(w_q),
                              _addr(w_scale), w_scale_count, m, n, k, _addr(workspace), workspace_bytes, stream))


def fp8_gemm_ex(out_dtype, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m, n, k,
                epilogue=EPILOGUE_NONE, bias=None, workspace=None, workspace_bytes=0, stream=None):
    _check(lib().ksq_fp8_gemm_ex(out_dtype, _addr(out), _addr(act_q), _addr(act_scale), act_scale_count, _addr(w_q),
                                 _addr(w_scale), w_scale_count, m, n, k, epilogue, _addr(bias), _addr(workspace),
                                 workspace_bytes, stream))
