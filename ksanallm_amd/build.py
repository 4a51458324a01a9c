"""Builds libksq.so (the HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libksq.so")

SOURCES = ["ksq_api.hip", "ksq_repack.hip", "ksq_w4a16_stream.hip", "ksq_w4a16_kstat.hip", "ksq_w4a16_astream.hip", "ksq_w4a16_prefill.hip", "ksq_fp8.hip", "ksq_fp8_kstat.hip", "ksq_fp8_prefill.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Rpass-analysis=kernel-resource-usage",  # read back by check_scratch below; not printed
    "-I" + os.path.join(ROOT, "include"),
    "-I" + CSRC,
]


# Private (scratch) memory per lane that a kernel may use.  The kernels keep their accumulators in lambdas' captures; if
# the compiler ever stops inlining one of those lambdas the captures move to memory (seen once: 1136 bytes per lane and
# a tenth of the speed, with every test still passing).  Real register spills of the fallback kernels stay below this.
MAX_SCRATCH_BYTES = 512


def check_scratch(src, remarks):
    """remarks: the compiler's kernel-resource-usage lines for one source file; raises on a kernel over the limit."""
    name = None
    for line in remarks:
        text = line.split("remark:", 1)[1].strip()
        if text.startswith("Function Name:"):
            name = text.split(":", 1)[1].split("[")[0].strip()
        elif text.startswith("ScratchSize"):
            size = int(text.split(":", 1)[1].split("[")[0].strip())
            if size > MAX_SCRATCH_BYTES:
                raise RuntimeError(f"{src}: kernel {name} uses {size} bytes of scratch memory per lane "
                                   f"(limit {MAX_SCRATCH_BYTES}): a lambda of the kernel is probably no longer inlined")


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libksq.so cannot be built")
    return exe


def build_library(verbose=False, jobs=5):
    """Compile every HIP source to an object (in parallel) and link libksq.so next to this file."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    cc = hipcc()
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [cc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    link = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    subprocess.check_call(link)
    return LIB


def build_layer_driver():
    """Compile the C++ layer shims (host code over the C ABI) and their test driver next to libksq.so."""
    cc = hipcc()
    layers = os.path.join(CSRC, "layers")
    out = os.path.join(HERE, "layer_driver")
    cmd = [cc, "-std=c++17", "-O2", "-Wall", "-Wno-unused-parameter", "-I" + os.path.join(ROOT, "include"),
           "-I" + layers, os.path.join(ROOT, "tests", "cpp", "layer_driver.cpp"), os.path.join(layers, "layers.cpp"),
           "-L" + HERE, "-lksq", "-Wl,-rpath,$ORIGIN", "-o", out]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("layer driver build failed:\n" + p.stdout)
    # host-only check of the workgroup -> tile map shared by the tile kernels (run by tests/test_capi_host.py)
    tm = os.path.join(HERE, "tile_map_test")
    cmd = [cc, "--offload-arch=gfx950", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
           os.path.join(ROOT, "tests", "cpp", "tile_map_test.hip"), "-o", tm]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("tile map test build failed:\n" + p.stdout)
    return out


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        remarks, lines, skip = [], [], 0
        for ln in out.splitlines():
            if "-Rpass-analysis=kernel-resource-usage" in ln:
                remarks.append(ln)
                skip = 2  # the source line and the caret that follow a remark
            elif skip and ln.lstrip()[:1] in "0123456789|":
                skip -= 1
            elif "packed-fp32-ops" not in ln and "remarks generated" not in ln:
                skip = 0
                lines.append(ln)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n" + "\n".join(lines))
        check_scratch(src, remarks)
        if lines:
            print("\n".join(lines), file=sys.stderr)


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_layer_driver())
