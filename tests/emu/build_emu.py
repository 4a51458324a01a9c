"""Builds tests/emu/libksq_emu.so: the library's own HIP sources compiled as plain C++ for the host against the
stand-in header in tests/emu/include, plus the fiber runtime.  Test infrastructure; the product never loads it."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from ksanallm_amd.build import CSRC, SOURCES  # noqa: E402

LIB = os.path.join(HERE, "libksq_emu.so")
LIB_ASAN = os.path.join(HERE, "libksq_emu_asan.so")


def clangxx():
    for exe in ("/opt/rocm/lib/llvm/bin/clang++", "/opt/rocm/llvm/bin/clang++"):
        if os.path.exists(exe):
            return exe
    raise RuntimeError("the ROCm clang++ is needed for the host build of the kernels (ext_vector_type, _Float16, __bf16)")


def flags(asan):
    f = ["-x", "c++", "-std=c++17", "-O1", "-g1", "-fPIC", "-march=x86-64-v3", "-pthread",
         "-I" + os.path.join(HERE, "include"), "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
         "-Wno-unknown-attributes", "-Wno-ignored-attributes", "-Wno-unused-function", "-Wno-pass-failed",
         "-Wno-unknown-pragmas"]
    if asan:
        f += ["-fsanitize=address", "-fno-omit-frame-pointer"]
    return f


def build(asan=False, jobs=8, verbose=False):
    cc = clangxx()
    objdir = os.path.join(HERE, "build_asan" if asan else "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES] + [os.path.join(HERE, "emu_runtime.cpp")]
    objs, procs = [], []

    def drain():
        while procs:
            name, p = procs.pop(0)
            out, _ = p.communicate()
            if p.returncode != 0:
                raise RuntimeError(f"host build of {name} failed:\n{out[-6000:]}")
            if verbose and out.strip():
                print(out, file=sys.stderr)

    for src in srcs:
        obj = os.path.join(objdir, os.path.basename(src).rsplit(".", 1)[0] + ".o")
        objs.append(obj)
        cmd = [cc, *flags(asan), "-c", src, "-o", obj]
        procs.append((os.path.basename(src), subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            drain()
    drain()
    out = LIB_ASAN if asan else LIB
    link = [cc, "-shared", "-pthread", "-o", out, *objs]
    if asan:
        link += ["-fsanitize=address", "-shared-libasan"]
    subprocess.check_call(link)
    return out


def build_layer_driver():
    """The C++ layer shims and their test driver (tests/cpp/layer_driver.cpp) against the emulated library."""
    cc = clangxx()
    layers = os.path.join(CSRC, "layers")
    out = os.path.join(HERE, "layer_driver_emu")
    cmd = [cc, "-std=c++17", "-O1", "-g1", "-march=x86-64-v3", "-pthread", "-Wno-unknown-attributes",
           "-I" + os.path.join(HERE, "include"), "-I" + os.path.join(ROOT, "include"), "-I" + layers,
           "-I" + os.path.join(ROOT, "tests", "cpp"), os.path.join(ROOT, "tests", "cpp", "layer_driver.cpp"),
           os.path.join(layers, "layers.cpp"), "-L" + HERE, "-lksq_emu", "-Wl,-rpath,$ORIGIN", "-o", out]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("emulated layer driver build failed:\n" + p.stdout[-6000:])
    return out


if __name__ == "__main__":
    print(build(asan="--asan" in sys.argv, verbose=True))
    if "--asan" not in sys.argv:
        print(build_layer_driver())
