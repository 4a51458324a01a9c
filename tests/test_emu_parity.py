"""The GPU parity tests, run on the CPU: the same test functions as tests/test_*_gpu.py, with the C ABI bound to the
emulated library (tests/emu: the library's kernel sources compiled for the host and executed one fiber per lane) and
CPU tensors standing in for device memory.  Every case is checked against the oracle exactly as on the GPU, and in
addition the emulator's bounds checks must stay silent: a buffer load that the hardware's range check would let
through but that leaves its tensor fails the case.  Cases at the full sizes of the benchmark configurations are left
to the GPU; the shapes here are the small ones that walk every kernel, planner branch and forced override.

The emulated library is test infrastructure: nothing under ksanallm_amd/ loads it, and the GPU tests never do."""
import numpy as np
import pytest
import torch

from tests import emu
from tests import test_fp8_gpu as f8
from tests import test_golden_gpu as gold
from tests import test_next_rows_gpu as nxt
from tests import test_w4a16_gpu as w4
from tests import test_zz_no_alloc as noalloc


@pytest.fixture
def gpu(monkeypatch):
    """Stands in for the `gpu` fixture of the GPU tests: CPU tensors, the emulated library behind the C ABI."""
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    monkeypatch.setattr(torch.cuda, "empty_cache", lambda *a, **k: None)
    # device allocations are at least 256-byte aligned, which the library asks of a workspace; torch's CPU allocator
    # gives 64: byte buffers (what the tests use as workspaces) are carved out of a larger one at a 256-byte boundary
    real_empty = torch.empty

    def empty(*size, **kw):
        if kw.get("dtype") is torch.uint8 and len(size) == 1 and isinstance(size[0], int):
            buf = real_empty(size[0] + 256, **kw)
            off = (-buf.data_ptr()) % 256
            return buf[off:off + size[0]]
        return real_empty(*size, **kw)

    monkeypatch.setattr(torch, "empty", empty)
    with emu.session():
        yield torch.device("cpu")
        emu.assert_clean("emulated run")


# ---- W4A16 ---------------------------------------------------------------------------------------------------------------
test_device_repack_matches_host_repack = w4.test_device_repack_matches_host_repack
test_one_hot_rows_return_dequantized_rows_exactly = w4.test_one_hot_rows_return_dequantized_rows_exactly
test_integer_case_is_exact = w4.test_integer_case_is_exact
test_m_sweep_small_shape = w4.test_m_sweep_small_shape
test_m_sweep_both_decode_routes = w4.test_m_sweep_both_decode_routes
test_group_sizes_and_kinds = w4.test_group_sizes_and_kinds
test_forced_split_k_and_tile_widths = w4.test_forced_split_k_and_tile_widths
test_prefill_kernel_widths = w4.test_prefill_kernel_widths
test_prefill_row_tiles = w4.test_prefill_row_tiles
test_prefill_128_rows_k_groups = w4.test_prefill_128_rows_k_groups
test_prefill_split_k = w4.test_prefill_split_k
test_prefill_128_rows_split_k = w4.test_prefill_128_rows_split_k
test_accumulator_stationary_route = w4.test_accumulator_stationary_route
test_accumulator_stationary_split_k = w4.test_accumulator_stationary_split_k
test_planner_choices_without_overrides = w4.test_planner_choices_without_overrides
test_prefill_bf16_row_magnitudes = w4.test_prefill_bf16_row_magnitudes
test_bf16_scales_far_outside_the_fp16_range = w4.test_bf16_scales_far_outside_the_fp16_range
test_k_odd_multiple_of_64 = w4.test_k_odd_multiple_of_64
test_random_shapes = w4.test_random_shapes
test_no_workspace_still_correct = w4.test_no_workspace_still_correct
test_caller_bound_split_k_counters_and_launch_log = w4.test_caller_bound_split_k_counters_and_launch_log
test_k_tiles_per_wave = w4.test_k_tiles_per_wave
test_k_phases_inside_the_workgroup = w4.test_k_phases_inside_the_workgroup

# ---- FP8 -------------------------------------------------------------------------------------------------------------------
test_per_channel_quantize_reference_shapes = f8.test_per_channel_quantize_reference_shapes
test_per_tensor_dynamic_and_static = f8.test_per_tensor_dynamic_and_static
test_quantize_special_values = f8.test_quantize_special_values
test_rescale = f8.test_rescale
test_convert_weight = f8.test_convert_weight
test_gemm_rowwise_scales = f8.test_gemm_rowwise_scales
test_gemm_per_tensor_scales_and_ragged_shapes = f8.test_gemm_per_tensor_scales_and_ragged_shapes
test_gemm_large_m_ragged = f8.test_gemm_large_m_ragged
test_gemm_large_m_both_tiles = f8.test_gemm_large_m_both_tiles
test_gemm_k_phases_inside_the_workgroup = f8.test_gemm_k_phases_inside_the_workgroup
test_gemm_random_shapes = f8.test_gemm_random_shapes
test_gemm_fp32_results_every_route = f8.test_gemm_fp32_results_every_route
test_gemm_dynamic_fp32 = f8.test_gemm_dynamic_fp32
test_gemm_large_m_small_integers_exact = f8.test_gemm_large_m_small_integers_exact
test_gemm_small_integers_exact = f8.test_gemm_small_integers_exact
test_convert_weight_per_channel = f8.test_convert_weight_per_channel
test_merge_qkv_scales = f8.test_merge_qkv_scales
test_gemm_dynamic_quantiser_is_the_quantise_kernels = f8.test_gemm_dynamic_quantiser_is_the_quantise_kernels
test_gemm_dynamic_epilogues_and_errors = f8.test_gemm_dynamic_epilogues_and_errors

# ---- golden fixtures, widened rows, the entry point that allocates nothing ---------------------------------------------------
test_w4a16_golden = gold.test_w4a16_golden
test_fp8_golden = gold.test_fp8_golden
test_w4a16_next_golden = gold.test_w4a16_next_golden
test_device_repack_ex_matches_host = nxt.test_device_repack_ex_matches_host
test_gemm_from_preprocessed_weights = nxt.test_gemm_from_preprocessed_weights
test_gemm_from_marlin_weights = nxt.test_gemm_from_marlin_weights
test_desc_act_marlin_weights = nxt.test_desc_act_marlin_weights
test_one_hot_rows_through_cutlass_layout_are_exact = nxt.test_one_hot_rows_through_cutlass_layout_are_exact
test_permute_columns_and_interleave_halves = nxt.test_permute_columns_and_interleave_halves
test_desc_act_checkpoint = nxt.test_desc_act_checkpoint
test_act_perm_without_workspace_is_refused = nxt.test_act_perm_without_workspace_is_refused
test_silu_mul_epilogue = nxt.test_silu_mul_epilogue
test_bias_epilogue = nxt.test_bias_epilogue
test_fp8_epilogues = nxt.test_fp8_epilogues
test_w4a16_gemm_row_maxima_feed_the_quantiser = nxt.test_w4a16_gemm_row_maxima_feed_the_quantiser
test_fp8_gemm_row_maxima = nxt.test_fp8_gemm_row_maxima
test_static_scratch_matches_workspace_entry_point = noalloc.test_static_scratch_matches_workspace_entry_point
