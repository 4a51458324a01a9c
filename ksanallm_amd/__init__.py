"""MI355X-native quantized linear-layer path (W4A16 group GEMM + FP8 e4m3 GEMM) behind a C ABI.

``ksanallm_amd.capi`` binds ``libksq.so`` (hand-written gfx950 HIP kernels) with ctypes; the C++ shims under
``ksanallm_amd/csrc/layers`` mirror the ``Init / Forward(input_tensors, output_tensors)`` interface of ksana_llm's
quantized MatMul layers on top of the same C ABI.  There is no CPU or PyTorch fallback: if the library is missing, loading raises.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
