"""Bounds sweep on the CPU: every shape of a lattice around the launch planners' thresholds goes through the C ABI of
the emulated library with tensors of exactly the documented sizes; the real planners pick the kernels, and the
emulator checks every buffer-resource access of the first, the last and a few more workgroups of every launch (all K
splits of those positions) against the tensor it belongs to.  Data is zeros: only addresses matter here (the parity
tests cover values).  `python -m tests.emu.bounds_sweep [w4|fp8] [--full]` runs it standalone on all cores."""
import itertools
import os
import sys

import numpy as np

W4_M = [1, 3, 4, 5, 8, 9, 16, 17, 31, 32, 33, 40, 47, 48, 49, 63, 64, 65, 66, 100, 127, 128, 129, 191, 200, 256, 257,
        300, 511, 513, 640, 1000]
W4_N = [16, 48, 256, 272, 1040, 4096, 4112, 8192, 16384, 16400, 22016]
W4_K = [128, 256, 384, 640, 1024, 2048, 4096, 192, 1088]
FP8_M = [1, 2, 4, 5, 8, 16, 17, 31, 32, 33, 48, 49, 64, 65, 100, 127, 128, 129, 255, 256, 257, 300, 511, 512, 600, 1030]
FP8_N = [8, 64, 256, 272, 544, 4104, 6144, 8192, 16384, 16392, 24576]
FP8_K = [64, 128, 192, 256, 1024, 1088, 1152, 4096, 8192, 9600]


def w4_cases(full):
    """(M, N, K, g, dtype, workspace?): the whole lattice, or every shape once with group size, element type and
    workspace alternating."""
    out = []
    for i, (K, M, N) in enumerate(itertools.product(W4_K, W4_M, W4_N)):
        combos = list(itertools.product([64, 128], ["f16", "bf16"], [True, False]))
        for g, dt, ws in (combos if full else [combos[i % 8], combos[(i + 3) % 8]]):
            if K % g == 0 and (K % 128 == 0 or g == 64):
                out.append((M, N, K, g, dt, ws))
    # K long enough that the decode kernels walk it in phases (up to eight rows), split it over workgroups, or hand it
    # to the streaming kernel with a four-way split (nine to sixteen rows)
    for i, (K, M, N) in enumerate(itertools.product([6272, 8320, 25088], [1, 4, 5, 8, 9, 16, 17, 33], [16, 272, 4112, 8192])):
        combos = list(itertools.product([64, 128], ["f16", "bf16"], [True, False]))
        for g, dt, ws in (combos if full else [combos[i % 8], combos[(i + 5) % 8]]):
            out.append((M, N, K, g, dt, ws))
    # K long and output tiles few at 65 rows and more: the 64-row and the 128-row kernel with K split over workgroups
    # (partial tiles of every split in the workspace, the reduction kernel behind them)
    for i, (K, M, N) in enumerate(itertools.product([8192, 11008], [65, 128, 129, 256, 300, 513], [272, 4096, 4112, 8192])):
        combos = list(itertools.product([64, 128], ["f16", "bf16"], [True, False]))
        for g, dt, ws in (combos if full else [combos[i % 8], combos[(i + 5) % 8]]):
            out.append((M, N, K, g, dt, ws))
    return out


def fp8_cases(full):
    out = []
    for i, (K, M, N) in enumerate(itertools.product(FP8_K, FP8_M, FP8_N)):
        if not full and K >= 8192 and M > 64 and (i % 4):
            continue  # long k loops of the tile kernels are slow to emulate: every fourth of those
        combos = list(itertools.product([False, True], ["f16", "bf16"], [True, False]))
        for pc, dt, ws in (combos if full else [combos[i % 8]]):
            out.append((M, N, K, pc, dt, ws))
    return out


def _aligned(nbytes):
    buf = np.zeros(max(nbytes, 1) + 256, np.uint8)
    off = (-buf.ctypes.data) % 256
    return buf[off:off + max(nbytes, 1)]


def run_w4(case, sample):
    from ksanallm_amd import capi
    from tests import emu

    M, N, K, g, dt, use_ws = case
    with emu.session(sample_blocks=sample) as L:
        wb, sb = capi.w4a16_repack_sizes(K, N, g)
        wsb = capi.w4a16_workspace_bytes(M, N, K) if use_ws else 0
        act, w, sz = np.zeros(M * K, np.uint16), _aligned(wb), np.zeros(sb // 4, np.uint32)
        out, ws = np.zeros(M * N, np.uint16), _aligned(wsb)
        try:
            capi.w4a16_gemm(capi.F16 if dt == "f16" else capi.BF16, out, act, w, sz, M, N, K, g, ws if wsb else None, wsb)
        except capi.KsqError as e:
            if not (K % 128 and not use_ws and e.code == capi.ERR_WORKSPACE):  # k % 128 == 64 needs the padded copy
                return f"w4a16 {case}: {e}"
        n, msgs = emu.errors()
        L.ksq_emu_clear_errors()
        return f"w4a16 {case}: {n} accesses out of bounds, first: {msgs[0]}" if n else None


def run_fp8(case, sample):
    from ksanallm_amd import capi
    from tests import emu

    M, N, K, pc, dt, use_ws = case
    with emu.session(sample_blocks=sample) as L:
        wsb = capi.fp8_workspace_bytes(M, N, K) if use_ws else 0
        xq, wq = np.zeros(M * K, np.uint8), np.zeros(N * K, np.uint8)
        xs, wsc = np.ones(M if pc else 1, np.float32), np.ones(N if pc else 1, np.float32)
        out, ws = np.zeros(M * N, np.uint16), _aligned(wsb)
        try:
            capi.fp8_gemm(capi.F16 if dt == "f16" else capi.BF16, out, xq, xs, len(xs), wq, wsc, len(wsc), M, N, K,
                          ws if wsb else None, wsb)
        except capi.KsqError as e:
            return f"fp8 {case}: {e}"
        n, msgs = emu.errors()
        L.ksq_emu_clear_errors()
        return f"fp8 {case}: {n} accesses out of bounds, first: {msgs[0]}" if n else None


def run_shard(args):
    kind, full, shard, nshards, sample = args
    os.environ["KSQ_EMU_THREADS"] = "1"  # one process per core instead
    cases = (w4_cases if kind == "w4" else fp8_cases)(full)[shard::nshards]
    fn = run_w4 if kind == "w4" else run_fp8
    bad = [r for r in (fn(c, sample) for c in cases) if r]
    return len(cases), bad


def sweep(kind, full=False, sample=3, procs=None):
    """Returns (cases run, list of failures)."""
    import multiprocessing as mp

    procs = procs or min(8, os.cpu_count() or 1)
    with mp.get_context("spawn").Pool(procs) as pool:
        res = pool.map(run_shard, [(kind, full, s, procs, sample) for s in range(procs)])
    return sum(r[0] for r in res), [b for r in res for b in r[1]]


if __name__ == "__main__":
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
    kinds = [a for a in sys.argv[1:] if a in ("w4", "fp8")] or ["w4", "fp8"]
    for kind in kinds:
        n, bad = sweep(kind, full="--full" in sys.argv)
        print(f"{kind}: {n} cases, {len(bad)} failures")
        for b in bad[:20]:
            print("  ", b)
