"""bench.py on the CPU: the algorithmic byte counts its figures are built on, and the one-GPU contract."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402

LLAMA_7B = [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]  # K x N of qkv, o, gate_up, down


def test_step_bytes_of_the_headline_workload():
    # one step = the four GEMMs of a Llama-2-7B layer at M = 16, AWQ-style (uint4 zeros), group size 128:
    # int4 weights + fp16 scales + uint4 zeros + fp16 activations in + fp16 out
    total = 0
    for k, n in LLAMA_7B:
        g = k // 128
        want = k * n // 2 + 2 * g * n + g * n // 2 + 16 * k * 2 + 16 * n * 2
        assert bench.w4a16_bytes(16, k, n) == want
        total += want
    assert total == 107_245_568


def test_fp8_bytes():
    # e4m3 weights + fp32 per-channel scales + e4m3 activations + fp32 per-token scales + 16-bit output
    assert bench.fp8_bytes(1, 8192, 8192) == 8192 * 8192 + 4 * 8192 + 8192 + 4 + 2 * 8192


def test_weight_copies_cover_the_last_level_cache():
    # distinct weight bytes between two uses of one copy: at least 600 MB, whatever the shape
    for k, n in LLAMA_7B + [(8192, 57344), (28672, 8192)]:
        wb = k * n // 2
        assert bench.ncopies_for(wb) * wb >= 600 << 20
        assert (bench.ncopies_for(wb) - 1) * wb < 600 << 20


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
