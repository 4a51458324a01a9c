"""A slice of the emulated parity tests under AddressSanitizer: the kernels' raw-pointer accesses (partial tiles in the
workspace, arrival counters, epilogue stores, LDS arrays) are ordinary host accesses in the emulated build, so the
sanitizer sees every one of them.  Runs in a subprocess that preloads the sanitizer's runtime; the whole of
tests/test_emu_parity.py passes the same way (about twenty minutes, `KSQ_EMU_ASAN_ALL=1`)."""
import glob
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SLICE = "golden or one_hot or no_workspace or static_scratch or integer_case or test_gemm_rowwise_scales"


def _runtime():
    hits = glob.glob("/opt/rocm/lib/llvm/lib/clang/*/lib/linux/libclang_rt.asan-x86_64.so")
    return hits[0] if hits else None


def test_parity_slice_under_address_sanitizer():
    rt = _runtime()
    if rt is None:
        pytest.skip("the sanitizer runtime of the ROCm clang is not installed")
    from tests.emu import build_emu

    if not os.path.exists(build_emu.LIB_ASAN):
        build_emu.build(asan=True)
    env = dict(os.environ, KSQ_EMU_ASAN="1", KSQ_EMU_THREADS="1",
               LD_PRELOAD=rt + (":" + os.environ["LD_PRELOAD"] if os.environ.get("LD_PRELOAD") else ""),
               ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0:detect_stack_use_after_return=0:abort_on_error=0")
    cmd = [sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_emu_parity.py"), "-x", "-q", "-p",
           "no:cacheprovider"]
    if os.environ.get("KSQ_EMU_ASAN_ALL") != "1":
        cmd += ["-k", SLICE]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, cwd=ROOT, timeout=3000)
    assert p.returncode == 0 and "AddressSanitizer" not in p.stdout, p.stdout[-4000:]
