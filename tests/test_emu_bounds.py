"""Every buffer-resource access of every kernel, over a lattice of shapes around the planners' thresholds, must stay
inside the tensor it belongs to: run on the CPU through the emulated library (tests/emu/bounds_sweep.py).

This is the check that found an out-of-bounds prefetch in the k-stationary decode kernel: with K = 128 and 17..32 rows
the kernel ran an instantiation with two k tiles per wave, the wave's buffer resource was sized for both, and the
prefetch of the column tile after the workgroup's last one passed the hardware's range check -- the last workgroup read
1 KiB past the end of the weights and 64 bytes per group past the scale/zero words.  `test_found_bug_shape` keeps that
shape; the sweeps cover the rest."""
import pytest

from tests.emu import bounds_sweep as bs


def test_found_bug_shape():
    for dt in ("f16", "bf16"):
        for M in (17, 20, 32):
            for N in (16, 48, 272):
                for g in (64, 128):
                    assert bs.run_w4((M, N, 128, g, dt, True), 0) is None


def test_w4a16_lattice():
    n, bad = bs.sweep("w4")
    assert n > 5000 and not bad, bad[:5]


def test_fp8_lattice():
    n, bad = bs.sweep("fp8")
    assert n > 2000 and not bad, bad[:5]
