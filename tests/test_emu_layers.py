"""The C++ layer shims (GroupMatMulLayer / Fp8MatMulLayer) on the CPU: the cases of tests/test_layers_gpu.py run
through the same test driver linked against the emulated library (tests/emu), against the oracle.  The emulator's
bounds checks are on: an out-of-range buffer load in any kernel the layers launch fails the case."""
import os
import subprocess

import pytest

import tests.test_layers_gpu as cases
from tests import emu

EMU_DRIVER = os.path.join(os.path.dirname(os.path.abspath(emu.__file__)), "layer_driver_emu")


def _run(args):
    if not os.path.exists(EMU_DRIVER):
        from tests.emu import build_emu

        emu.library()
        build_emu.build_layer_driver()
    env = dict(os.environ, KSQ_EMU_EXIT_CODE_ON_ERROR="97")
    p = subprocess.run([EMU_DRIVER, *map(str, args)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=600, env=env)
    return p.returncode, p.stdout.strip()


@pytest.fixture
def on_cpu(monkeypatch):
    monkeypatch.setattr(cases, "_run", _run)


@pytest.mark.parametrize("dtype,method,layout,zeros,M", [
    ("f16", "gptq", "gptq", "none", 16),
    ("bf16", "awq", "awq", "awq", 5),
    ("f16", "awq", "rowmajor", "additive", 33),
    ("bf16", "awq", "rowmajor", "uint8", 130),
])
def test_group_matmul_layer_forward(on_cpu, tmp_path, dtype, method, layout, zeros, M):
    cases.test_group_matmul_layer_forward(None, tmp_path, dtype, method, layout, zeros, M)


@pytest.mark.parametrize("dtype,extra,layout,M", [
    ("f16", "none", "cutlass80", 16),
    ("f16", "desc", "gptq", 24),
    ("bf16", "silu", "awq", 70),
    ("f16", "bias", "awq", 40),
])
def test_group_matmul_layer_widened(on_cpu, tmp_path, dtype, extra, layout, M):
    cases.test_group_matmul_layer_widened(None, tmp_path, dtype, extra, layout, M)


def test_group_matmul_layer_fused(on_cpu, tmp_path):
    cases.test_group_matmul_layer_fused_from_separate_projections(None, tmp_path, "f16", 16)


@pytest.mark.parametrize("dtype,M,parts", [("f16", 16, None), ("bf16", 70, None), ("f16", 5, [64, 32, 32]),
                                           ("bf16", 130, [64, 64])])
def test_group_matmul_layer_k_not_a_multiple_of_128(on_cpu, tmp_path, dtype, M, parts):
    cases._odd_k_case(_run, tmp_path, dtype, M, parts)


@pytest.mark.parametrize("dtype,layout,kind,M", [("f16", "cutlass80", "awq", 16), ("bf16", "cutlass80", "gptq", 70),
                                                 ("f16", "cutlass90", "awq", 5)])
def test_group_matmul_layer_takes_the_reference_loaders_tensors_at_forward(on_cpu, tmp_path, dtype, layout, kind, M):
    cases._adopt_case(_run, tmp_path, dtype, layout, kind, M)


@pytest.mark.parametrize("dtype,wscales,static,M", [("f16", "1", 0, 16), ("bf16", "n", 0, 70), ("f16", "1", 1, 5),
                                                    ("f32", "n", 0, 9), ("f32", "1", 0, 70), ("f32", "1", 1, 5)])
def test_fp8_matmul_layer_forward(on_cpu, tmp_path, dtype, wscales, static, M):
    cases.test_fp8_matmul_layer_forward(None, tmp_path, dtype, wscales, static, M)


@pytest.mark.parametrize("per_channel", [0, 1])
def test_fp8_load_time_pipeline(on_cpu, tmp_path, per_channel):
    cases.test_fp8_load_time_pipeline(None, tmp_path, "bf16", per_channel)


def test_error_conventions(on_cpu):
    cases.test_error_conventions(None)
