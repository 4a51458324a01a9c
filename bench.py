#!/usr/bin/env python3
"""Roofline bench of the quantized linear-layer path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: the four W4A16 GEMMs of a Llama-2-7B
decoder layer (qkv 4096x12288, o 4096x4096, gate_up 4096x22016, down 11008x4096; AWQ asymmetric int4, g = 128,
fp16 activations N(0,1)) at M = 16 tokens.  Consecutive steps use different layers (8 distinct weight sets,
~830 MB) so that no launch re-reads weights that are still resident in the 256 MB last-level cache.  All inputs
are resident in HBM before the timed region; the K timed steps are one HIP graph on one stream, bracketed by
events on that stream.

Prints ONE JSON line: value = whole-job algorithmic GB/s of that step, `roofline` for the dominant kernel (the W4A16
k-stationary decode kernel, HBM-bound) with a `mfma` object for the other half of the metric (the same four shapes
at M = 4096, bf16, against the dense MFMA peak), and `cpu_baseline` (the CPU oracle -- dequantize to fp32 + blocked
OpenMP GEMM -- timed on the same step on this machine's host cores).  `extra` carries the other regimes of the path;
every leg there rotates over enough weight copies (600 MB worth) that no launch finds its weights in the last-level
cache.

`--only LEG` runs one leg by itself (for profiling one kernel with rocprofv3) and prints a JSON line for it.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0         # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA, published
MFMA_FP8_PEAK_TFLOPS = 5000.0  # MI355X dense fp8 MFMA, published
ROTATE_BYTES = 600 << 20       # distinct weight bytes between two uses of the same copy (last-level cache: 256 MB)
METRIC = "W4A16 GEMM GB/s (M≤16) & TFLOP/s (M=4096), Llama-7B shapes, 1×MI355X"
SHAPES_7B = [("qkv", 4096, 12288), ("o", 4096, 4096), ("gate_up", 4096, 22016), ("down", 11008, 4096)]
SHAPES_70B = [("qkv", 8192, 10240), ("o", 8192, 8192), ("gate_up", 8192, 57344), ("down", 28672, 8192)]
SHAPES_72B = [("qkv", 8192, 10240), ("o", 8192, 8192), ("gate_up", 8192, 59136), ("down", 29568, 8192)]
GROUP = 128
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "w4a16_kstat_cfg1_m16_pmc.txt")


def w4a16_bytes(m, k, n, awq=True):
    """Algorithmic bytes of one GEMM: int4 weights + scales + (AWQ) uint4 zeros + activations + output."""
    g = k // GROUP
    return k * n // 2 + g * n * 2 + (g * n // 2 if awq else 0) + m * k * 2 + m * n * 2


def fp8_bytes(m, k, n):
    return k * n + 4 * n + m * k + 4 * m + 2 * m * n


def ncopies_for(weight_bytes):
    return max(1, -(-ROTATE_BYTES // weight_bytes))


class Layer:
    """One decoder layer's four AWQ weights, generated on the GPU and repacked through the C ABI."""

    def __init__(self, torch, capi, device, seed, dtype, keep_source=False):
        self.dtype = dtype
        self.weights = []
        self.source = []
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        tdt = torch.float16 if dtype == capi.F16 else torch.bfloat16
        for name, k, n in SHAPES_7B:
            g = k // GROUP
            qweight = torch.randint(-2**31, 2**31 - 1, (k, n // 8), dtype=torch.int32, device=device, generator=gen)
            qzeros = torch.randint(-2**31, 2**31 - 1, (g, n // 8), dtype=torch.int32, device=device, generator=gen)
            scales = (torch.randn((g, n), device=device, generator=gen).abs() * 0.02 + 1e-3).to(tdt)
            wb, sb = capi.w4a16_repack_sizes(k, n, GROUP)
            w = torch.empty(wb, dtype=torch.uint8, device=device)
            sz = torch.empty(sb // 4, dtype=torch.int32, device=device)
            capi.w4a16_repack(capi.W4_AWQ_INT32_NPACK, qweight, capi.ZERO_AWQ_INT32, qzeros, scales, dtype, k, n,
                              GROUP, w, sz)
            self.weights.append((name, k, n, w, sz))
            if keep_source:
                self.source.append((qweight.cpu().numpy(), qzeros.cpu().numpy(), scales))
        torch.cuda.synchronize()


def rotated(torch, w, sz):
    """Enough copies of one repacked weight that a launch never finds its weights in the last-level cache."""
    n = ncopies_for(w.numel())
    return [(w, sz)] + [(w.clone(), sz.clone()) for _ in range(n - 1)]


def gptq_weight(torch, capi, dev, gen, k, n, tdt=None):
    tdt = tdt or torch.float16
    g = k // GROUP
    qweight = torch.randint(-2**31, 2**31 - 1, (k // 8, n), dtype=torch.int32, device=dev, generator=gen)
    scales = (torch.randn((g, n), device=dev, generator=gen).abs() * 0.02 + 1e-3).to(tdt)
    wb, sb = capi.w4a16_repack_sizes(k, n, GROUP)
    w = torch.empty(wb, dtype=torch.uint8, device=dev)
    sz = torch.empty(sb // 4, dtype=torch.int32, device=dev)
    capi.w4a16_repack(capi.W4_GPTQ_INT32_KPACK, qweight, capi.ZERO_NONE, None, scales,
                      capi.F16 if tdt == torch.float16 else capi.BF16, k, n, GROUP, w, sz)
    torch.cuda.synchronize()
    return w, sz


def time_graph(torch, stream, launch, count):
    """Average device time per launch (us) of `count` back-to-back launches replayed as one graph."""
    with torch.cuda.stream(stream):
        for i in range(min(count, 4)):
            launch(i)
        stream.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(count):
                launch(i)
        g.replay()
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        g.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / count


def observed_clocks():
    """What the machine reports about itself: the host CPU model and the GPU's current / peak shader clock."""
    info = {"cpu_model": None, "gpu_sclk": None}
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                info["cpu_model"] = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        out = subprocess.run(["rocm-smi", "--showclocks"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True,
                             timeout=20).stdout
        for line in out.splitlines():
            if "sclk" in line:
                info["gpu_sclk"] = line.split(":", 1)[-1].strip() if ":" in line else line.strip()
                break
    except (OSError, subprocess.SubprocessError):
        pass
    return info


# ------------------------------------------------------------------------------------------------ legs
def w4_decode_shape(torch, capi, stream, name, k, n, w, sz, M, dtype, gen, count=None):
    """One 7B/70B shape at a decode batch: rotated weight copies, GB/s against the HBM peak."""
    dev = w.device
    tdt = torch.float16 if dtype == capi.F16 else torch.bfloat16
    copies = rotated(torch, w, sz)
    act = torch.randn((M, k), device=dev, generator=gen).to(tdt)
    out = torch.empty((M, n), dtype=tdt, device=dev)
    wsb = capi.w4a16_workspace_bytes(M, n, k)
    wk = torch.empty(max(wsb, 256), dtype=torch.uint8, device=dev)

    def launch(i):
        cw, csz = copies[i % len(copies)]
        capi.w4a16_gemm(dtype, out, act, cw, csz, M, n, k, GROUP, wk, wsb, stream.cuda_stream)

    us = time_graph(torch, stream, launch, count or max(32, len(copies)))
    del copies
    return us


def per_shape(torch, capi, layer, stream, M, dtype, gen):
    table = {}
    for name, k, n, w, sz in layer.weights:
        us = w4_decode_shape(torch, capi, stream, name, k, n, w, sz, M, dtype, gen)
        b = w4a16_bytes(M, k, n)
        table[name] = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1), "frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 3),
                       "copies": ncopies_for(w.numel())}
        torch.cuda.empty_cache()
    return table


def fused(torch, capi, layer, stream, M, dtype, dev, gen):
    """The steps either side of the GEMM folded into it, at the decode batch of the headline: gate_up with the
    SiLU-mul epilogue (one launch instead of GEMM + activation kernel; the output is half as wide), qkv with a bias
    row, and qkv of a desc_act checkpoint (column gather of the activations + GEMM, two launches)."""
    table = {}
    tdt = torch.float16 if dtype == capi.F16 else torch.bfloat16
    cases = [("gate_up_silu_mul", 2, capi.EPILOGUE_SILU_MUL, False), ("qkv_bias", 0, capi.EPILOGUE_BIAS, False),
             ("qkv_act_order", 0, capi.EPILOGUE_NONE, True)]
    for label, idx, epi, act_order in cases:
        name, k, n, w, sz = layer.weights[idx]
        copies = rotated(torch, w, sz)
        act = torch.randn((M, k), device=dev, generator=gen).to(tdt)
        out = torch.empty((M, n // 2 if epi == capi.EPILOGUE_SILU_MUL else n), dtype=tdt, device=dev)
        bias = torch.randn((n,), device=dev, generator=gen).to(tdt) if epi == capi.EPILOGUE_BIAS else None
        perm = torch.randperm(k, device=dev, generator=gen).to(torch.int32) if act_order else None
        wsb = capi.w4a16_workspace_bytes_ex(M, n, k, act_order)
        wk = torch.empty(max(wsb, 256), dtype=torch.uint8, device=dev)

        def launch(i):
            cw, csz = copies[i % len(copies)]
            capi.w4a16_gemm_ex(dtype, out, act, cw, csz, M, n, k, GROUP, perm, epi, bias, wk, wsb, stream.cuda_stream)

        us = time_graph(torch, stream, launch, max(32, len(copies)))
        b = w4a16_bytes(M, k, n) - (M * n if epi == capi.EPILOGUE_SILU_MUL else 0)
        table[label] = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1)}
        del copies
        torch.cuda.empty_cache()
    return table


def prefill_shape(torch, capi, stream, k, n, w, sz, M, dtype_name, gen):
    dev = w.device
    tdt = torch.bfloat16 if dtype_name == "bf16" else torch.float16
    cdt = capi.BF16 if dtype_name == "bf16" else capi.F16
    copies = rotated(torch, w, sz)
    act = torch.randn((M, k), device=dev, generator=gen).to(tdt)
    out = torch.empty((M, n), dtype=tdt, device=dev)
    wsb = capi.w4a16_workspace_bytes(M, n, k)
    ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device=dev)

    def launch(i):
        cw, csz = copies[i % len(copies)]
        capi.w4a16_gemm(cdt, out, act, cw, csz, M, n, k, GROUP, ws, wsb, stream.cuda_stream)

    us = time_graph(torch, stream, launch, max(4, min(len(copies), 16)))
    del copies
    return us


def prefill(torch, capi, layer, stream, gen, dtype_name="bf16", M=4096):
    """configs[2] (bf16 activations, M = 512 / 2048 / 4096): TFLOP/s per shape against the dense MFMA peak, bf16
    conversion kernel included.  `layer` has to be repacked for the element type of the leg (bf16 scales carry a
    column exponent that the fp16-scaled set does not); weight copies rotate, activations and outputs do not."""
    assert layer.dtype == (capi.BF16 if dtype_name == "bf16" else capi.F16), "weights repacked for the other element type"
    table = {}
    for name, k, n, w, sz in layer.weights:
        us = prefill_shape(torch, capi, stream, k, n, w, sz, M, dtype_name, gen)
        tf = 2.0 * M * k * n / us / 1e6
        table[name] = {"us": round(us, 1), "TFLOPs": round(tf, 1), "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        torch.cuda.empty_cache()
    return table


def mfma_half(table):
    """The M = 4096 half of the metric as one roofline object: the four shapes in sequence."""
    flops = sum(2.0 * 4096 * k * n for _, k, n in SHAPES_7B)
    us = sum(table[name]["us"] for name, _, _ in SHAPES_7B)
    tf = flops / us / 1e6
    return {"bound": "mfma", "kernel": "w4a16_prefill_kernel (+ bf16_rows_to_f16_kernel)",
            "workload": "configs[2]: the four Llama-2-7B shapes at M=4096, bf16 activations, in sequence",
            "achieved": round(tf, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4), "avg_launch_us": round(us / len(SHAPES_7B), 1),
            "per_shape": {name: table[name]["TFLOPs"] for name, _, _ in SHAPES_7B}}


def fp8_weights(torch, capi, dev, gen, k, n):
    """configs[4]: weights N(0,1) * 0.02 in bf16, [k, n], converted by the library's own load-time step
    (ksq_fp8_convert_weight_per_channel: transpose to [n, k] e4m3 with one fp32 scale per output channel); enough
    distinct copies that no launch finds its weights in the last-level cache."""
    ncopies = ncopies_for(k * n)
    ws, wscale = [], None
    for _ in range(ncopies):
        src = (torch.randn((k, n), device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        wq = torch.empty((n, k), dtype=torch.uint8, device=dev)
        sc = torch.empty(n, dtype=torch.float32, device=dev)
        capi.fp8_convert_weight_per_channel(capi.BF16, src, k, n, wq, sc)
        torch.cuda.synchronize()
        del src
        ws.append(wq)
        wscale = sc  # the copies differ in bytes, not in distribution: one scale vector serves the timing
    return ws, wscale


def fp8_case(torch, capi, dev, stream, gen, ws, wscale, k, n, M, reps):
    act = torch.randn((M, k), device=dev, generator=gen).to(torch.bfloat16)
    aq = torch.empty((M, k), dtype=torch.uint8, device=dev)
    ascale = torch.empty(M, dtype=torch.float32, device=dev)
    out = torch.empty((M, n), dtype=torch.bfloat16, device=dev)
    wsb = capi.fp8_workspace_bytes(M, n, k)
    wk = torch.empty(max(wsb, 256), dtype=torch.uint8, device=dev)

    def launch_q(i):
        capi.fp8_quantize(capi.BF16, act, M, k, capi.FP8_PER_TOKEN_DYNAMIC, aq, ascale, stream.cuda_stream)

    def launch_g(i):
        capi.fp8_gemm(capi.BF16, out, aq, ascale, M, ws[i % len(ws)], wscale, n, M, n, k, wk, wsb, stream.cuda_stream)

    launch_q(0)
    torch.cuda.synchronize()
    uq = time_graph(torch, stream, launch_q, reps)
    ug = time_graph(torch, stream, launch_g, max(reps, len(ws)))
    ud = None
    if M <= 8:  # quantisation folded into the GEMM: one launch
        dwsb = capi.fp8_gemm_dynamic_workspace_bytes(M, n, k)
        dwk = torch.empty(max(dwsb, 256), dtype=torch.uint8, device=dev)

        def launch_d(i):
            capi.fp8_gemm_dynamic(capi.BF16, out, act, ws[i % len(ws)], wscale, n, M, n, k, capi.EPILOGUE_NONE, None, dwk,
                                  dwsb, stream.cuda_stream)

        ud = time_graph(torch, stream, launch_d, max(reps, len(ws)))
    return uq, ug, ud


def fp8_sweep(torch, capi, dev, stream):
    """configs[4]: FP8 e4m3 GEMM at the Qwen-72B shapes, per-channel weight scales x per-token activation scales,
    bf16 in / out.  M = 1 and 64 against the HBM peak (algorithmic bytes K*N + 4N + M*K + 4M + 2*M*N), M = 2048 against
    the dense FP8 MFMA peak (and M = 256, a batch between the configs' own, where the tile grid leaves most compute
    units without a tile of their own); the activation quantisation is timed on its own."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    table = {}
    for name, k, n in SHAPES_72B:
        ws, wscale = fp8_weights(torch, capi, dev, gen, k, n)
        row = {"copies": len(ws)}
        for M in (1, 64, 256, 2048):
            uq, ug, ud = fp8_case(torch, capi, dev, stream, gen, ws, wscale, k, n, M, 32 if M <= 64 else (16 if M < 2048 else 4))
            if M <= 64:
                b = fp8_bytes(M, k, n)
                row[f"m{M}"] = {"quant_us": round(uq, 1), "gemm_us": round(ug, 1), "GBps": round(b / ug / 1e3, 1),
                                "frac": round(b / ug / 1e3 / HBM_PEAK_GBPS, 3)}
                if ud is not None:  # bf16 activations in (2 bytes each), no e4m3 copy written or read
                    row[f"m{M}"]["quant_and_gemm_one_launch_us"] = round(ud, 1)
            else:
                tf = 2.0 * M * k * n / ug / 1e6
                row[f"m{M}"] = {"quant_us": round(uq, 1), "gemm_us": round(ug, 1), "TFLOPs": round(tf, 1),
                                "frac": round(tf / MFMA_FP8_PEAK_TFLOPS, 4)}
        table[name] = row
        del ws
        torch.cuda.empty_cache()
    return table


def fp8_rowmax_chain(torch, capi, dev, stream):
    """The per-token quantisation's max pass moved into the GEMM that produces the tensor: the Qwen-72B o projection
    (K = N = 8192, FP8) with and without the row maxima in its epilogue, and the quantiser of its output (bf16
    [M, 8192]) with its own max pass and without (one read)."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(9)
    k = n = 8192
    ws, wscale = fp8_weights(torch, capi, dev, gen, k, n)
    table = {}
    for M in (8, 64, 2048):
        act = torch.randn((M, k), device=dev, generator=gen).to(torch.bfloat16)
        aq = torch.empty((M, k), dtype=torch.uint8, device=dev)
        ascale = torch.empty(M, dtype=torch.float32, device=dev)
        capi.fp8_quantize(capi.BF16, act, M, k, capi.FP8_PER_TOKEN_DYNAMIC, aq, ascale, stream.cuda_stream)
        out = torch.empty((M, n), dtype=torch.bfloat16, device=dev)
        rowmax = torch.zeros(M, dtype=torch.float32, device=dev)
        oq = torch.empty((M, n), dtype=torch.uint8, device=dev)
        oscale = torch.empty(M, dtype=torch.float32, device=dev)
        wsb = capi.fp8_workspace_bytes(M, n, k)
        wk = torch.empty(max(wsb, 256), dtype=torch.uint8, device=dev)
        sp = stream.cuda_stream
        reps = max(16 if M <= 64 else 4, len(ws))

        def gemm(i):
            capi.fp8_gemm(capi.BF16, out, aq, ascale, M, ws[i % len(ws)], wscale, n, M, n, k, wk, wsb, sp)

        def gemm_rowmax(i):
            capi.fill_zero_f32(rowmax, M, sp)
            capi.fp8_gemm_rowmax(capi.BF16, out, aq, ascale, M, ws[i % len(ws)], wscale, n, M, n, k, rowmax,
                                 capi.EPILOGUE_NONE, None, wk, wsb, sp)

        def quant2(i):
            capi.fp8_quantize(capi.BF16, out, M, n, capi.FP8_PER_TOKEN_DYNAMIC, oq, oscale, sp)

        def quant1(i):
            capi.fp8_quantize_rows_from_absmax(capi.BF16, out, M, n, rowmax, oq, oscale, sp)

        table[f"m{M}"] = {"gemm_us": round(time_graph(torch, stream, gemm, reps), 1),
                          "zero_fill_and_gemm_with_row_maxima_us": round(time_graph(torch, stream, gemm_rowmax, reps), 1),
                          "quantize_two_pass_us": round(time_graph(torch, stream, quant2, 16), 1),
                          "quantize_from_row_maxima_us": round(time_graph(torch, stream, quant1, 16), 1)}
    del ws
    torch.cuda.empty_cache()
    return table


def gptq_70b_sweep(torch, capi, dev, stream):
    """configs[3]: symmetric GPTQ int4 g=128, fp16, the Llama-3-70B shapes at M = 1, 32 (HBM-bound: GB/s against the
    HBM peak) and 256 (TFLOP/s against the dense MFMA peak), and 128 as a batch between the two."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    table = {}
    for name, k, n in SHAPES_70B:
        w, sz = gptq_weight(torch, capi, dev, gen, k, n)
        row = {"copies": ncopies_for(w.numel())}
        for M in (1, 32, 128, 256):
            us = w4_decode_shape(torch, capi, stream, name, k, n, w, sz, M, capi.F16, gen, count=max(16, ncopies_for(w.numel())))
            if M <= 32:
                b = w4a16_bytes(M, k, n, awq=False)
                row[f"m{M}"] = {"us": round(us, 1), "GBps": round(b / us / 1e3, 1), "frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 3)}
            else:
                tf = 2.0 * M * k * n / us / 1e6
                row[f"m{M}"] = {"us": round(us, 1), "TFLOPs": round(tf, 1), "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
            torch.cuda.empty_cache()
        table[name] = row
        del w, sz
        torch.cuda.empty_cache()
    return table


def cpu_baseline(np, torch, capi, layer, acts, outs, workspace, ws_bytes, M, dtype, step_bytes, stream, gen):
    """The CPU oracle on the same workload (one full step = the four GEMMs of layer 0), timed on this machine's
    host cores: dequantize to fp32 and the blocked OpenMP GEMM separately, and the two together (`value`).  Its
    output doubles as a parity check of the GPU result for that layer; a seeded subset of rows of one M = 4096 GEMM
    (gate_up, bf16) is checked the same way."""
    from oracle import oracle as orc

    cases = []
    for (name, k, n, w, sz), (qw, qz, scales) in zip(layer.weights, layer.source):
        u = orc.awq_unpack(qw)
        z = orc.awq_unpack(qz)
        s_bits = scales.view(torch.int16).cpu().numpy().view(np.uint16)
        a_bits = acts[k].view(torch.int16).cpu().numpy().view(np.uint16)
        scratch = (np.empty((k, n), dtype=np.float32), np.empty((M, k), dtype=np.float32))
        cases.append((name, k, n, u, z, s_bits, a_bits, scratch, w, sz))

    def one_step():
        return [orc.w4a16_forward(a, orc.F16, u, s, orc.F16, z, GROUP, scratch)
                for (_, _, _, u, z, s, a, scratch, _, _) in cases]

    def timed(fn):
        fn()  # warm-up (page-faults the buffers)
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            res = fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[1], res

    t, cpu_out = timed(one_step)
    # the two halves on their own, into the same scratch buffers
    t_deq, _ = timed(lambda: [orc.dequant(u, s, orc.F16, z, GROUP, out=scratch[0])
                              for (_, _, _, u, z, s, a, scratch, _, _) in cases])
    a32 = [orc.from_bits(c[6], orc.F16) for c in cases]
    t_gemm, _ = timed(lambda: [orc.gemm_f32(a, c[7][0]) for a, c in zip(a32, cases)])
    worst = {"max_rel": 0.0, "mean_abs_over_rms": 0.0}
    for (name, k, n, u, z, s, a, scratch, w, sz), want in zip(cases, cpu_out):
        capi.w4a16_gemm(dtype, outs[n], acts[k], w, sz, M, n, k, GROUP, workspace, ws_bytes, None)
        torch.cuda.synchronize()
        m = orc.error_metrics(outs[n].float().cpu().numpy(), want)
        worst = {key: max(worst[key], m[key]) for key in worst}
    clocks = observed_clocks()
    base = {
        "value": round(step_bytes / t / 1e9, 3),
        "unit": "GB/s",
        "cores": orc.num_threads(),
        "kind": "port",
        "sample": f"one full step (4 GEMMs, M={M}), median of 3 runs, {t:.3f} s per step; dequantize to fp32 + blocked "
                  f"OpenMP GEMM",
        "seconds": {"dequantize": round(t_deq, 4), "gemm": round(t_gemm, 4), "together": round(t, 4)},
        "cpu_model": clocks["cpu_model"],
    }
    parity = {k: float(f"{v:.3e}") for k, v in worst.items()}

    # M = 4096, gate_up, bf16: a seeded subset of rows against the oracle (weights of layer 0)
    name, k, n, w, sz = layer.weights[2]
    qw, qz, scales = layer.source[2]
    M2 = 4096
    act = torch.randn((M2, k), device=w.device, generator=gen).to(torch.bfloat16)
    out = torch.empty((M2, n), dtype=torch.bfloat16, device=w.device)
    # the same nibbles with bf16 scales (a cast of the fp16 values), repacked for the bf16 route
    sc16 = scales.to(torch.bfloat16)
    wb, sb = capi.w4a16_repack_sizes(k, n, GROUP)
    w2 = torch.empty(wb, dtype=torch.uint8, device=w.device)
    sz2 = torch.empty(sb // 4, dtype=torch.int32, device=w.device)
    capi.w4a16_repack(capi.W4_AWQ_INT32_NPACK, torch.from_numpy(qw).to(w.device), capi.ZERO_AWQ_INT32,
                      torch.from_numpy(qz).to(w.device), sc16, capi.BF16, k, n, GROUP, w2, sz2)
    wsb = capi.w4a16_workspace_bytes(M2, n, k)
    wk = torch.empty(max(wsb, 256), dtype=torch.uint8, device=w.device)
    capi.w4a16_gemm(capi.BF16, out, act, w2, sz2, M2, n, k, GROUP, wk, wsb, None)
    torch.cuda.synchronize()
    rows = np.sort(np.random.default_rng(4096).choice(M2, size=16, replace=False))
    trows = torch.from_numpy(rows).to(w.device)
    a_bits = act[trows].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    s_bits = sc16.view(torch.int16).cpu().numpy().view(np.uint16)
    want = orc.w4a16_forward(a_bits, orc.BF16, cases[2][3], s_bits, orc.BF16, cases[2][4], GROUP)
    m = orc.error_metrics(out[trows].float().cpu().numpy(), want)
    parity_m4096 = {"shape": "gate_up 4096x22016, M=4096, bf16", "rows_checked": int(len(rows)),
                    "max_rel": float(f"{m['max_rel']:.3e}"), "mean_abs_over_rms": float(f"{m['mean_abs_over_rms']:.3e}")}
    return base, parity, parity_m4096, clocks


# ------------------------------------------------------------------------------------------------ --only legs
def run_only(torch, capi, dev, stream, leg):
    """One kernel configuration by itself, a few dozen launches: what a rocprofv3 run profiles."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(21)
    if leg.startswith("w4a16_prefill_") or leg.startswith("w4a16_decode_"):
        # w4a16_prefill_<shape>_m<M>_<f16|bf16> / w4a16_decode_<7b|70b>_<shape>_m<M>
        parts = leg.split("_")
        if parts[1] == "prefill":
            shape, M, dt = parts[2] if parts[2] != "gate" else "gate_up", int(parts[-2][1:]), parts[-1]
            name, k, n = next(s for s in SHAPES_7B if s[0] == shape)
            layer = Layer(torch, capi, dev, 1000, capi.BF16 if dt == "bf16" else capi.F16)
            _, _, _, w, sz = next(x for x in layer.weights if x[0] == shape)
            us = prefill_shape(torch, capi, stream, k, n, w, sz, M, dt, gen)
            tf = 2.0 * M * k * n / us / 1e6
            return {"leg": leg, "us": round(us, 1), "TFLOPs": round(tf, 1), "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        family = parts[2]
        shape = "gate_up" if parts[3] == "gate" else parts[3]
        M = int(parts[-1][1:])
        name, k, n = next(s for s in (SHAPES_7B if family == "7b" else SHAPES_70B) if s[0] == shape)
        if family == "7b":
            layer = Layer(torch, capi, dev, 1000, capi.F16)
            _, _, _, w, sz = next(x for x in layer.weights if x[0] == shape)
        else:
            w, sz = gptq_weight(torch, capi, dev, gen, k, n)
        us = w4_decode_shape(torch, capi, stream, name, k, n, w, sz, M, capi.F16, gen)
        b = w4a16_bytes(M, k, n, awq=family == "7b")
        return {"leg": leg, "us": round(us, 2), "GBps": round(b / us / 1e3, 1), "frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 3)}
    if leg.startswith("fp8_"):
        # fp8_<shape>_m<M>
        parts = leg.split("_")
        shape = "gate_up" if parts[1] == "gate" else parts[1]
        M = int(parts[-1][1:])
        name, k, n = next(s for s in SHAPES_72B if s[0] == shape)
        ws, wscale = fp8_weights(torch, capi, dev, gen, k, n)
        uq, ug, ud = fp8_case(torch, capi, dev, stream, gen, ws, wscale, k, n, M, 32 if M <= 64 else 4)
        if M <= 64:
            b = fp8_bytes(M, k, n)
            return {"leg": leg, "quant_us": round(uq, 1), "gemm_us": round(ug, 1), "GBps": round(b / ug / 1e3, 1),
                    "frac": round(b / ug / 1e3 / HBM_PEAK_GBPS, 3),
                    "quant_and_gemm_one_launch_us": None if ud is None else round(ud, 1)}
        tf = 2.0 * M * k * n / ug / 1e6
        return {"leg": leg, "quant_us": round(uq, 1), "gemm_us": round(ug, 1), "TFLOPs": round(tf, 1),
                "frac": round(tf / MFMA_FP8_PEAK_TFLOPS, 4)}
    sys.exit(f"bench.py: unknown leg {leg!r} (w4a16_prefill_<shape>_m<M>_<f16|bf16>, w4a16_decode_<7b|70b>_<shape>_m<M>, "
             f"fp8_<shape>_m<M>)")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=16, help="tokens per step in the headline workload")
    ap.add_argument("--layers", type=int, default=8, help="distinct weight sets rotated over")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-core baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary measurements")
    ap.add_argument("--only", default=None, help="run one leg by itself, e.g. w4a16_prefill_gate_up_m4096_f16, "
                    "w4a16_decode_70b_gate_up_m64, fp8_gate_up_m2048, headline")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); multi-GPU runs are not part of it")

    import numpy as np
    import torch

    from ksanallm_amd import capi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream(device=dev)
    if args.only and args.only != "headline":
        print(json.dumps(run_only(torch, capi, dev, stream, args.only)), flush=True)
        return
    if args.only == "headline":
        args.no_cpu = args.no_extra = True

    M = args.m
    dtype = capi.F16
    layers = [Layer(torch, capi, dev, 1000 + i, dtype, keep_source=(i == 0)) for i in range(args.layers)]
    gen = torch.Generator(device=dev)
    gen.manual_seed(7)
    acts = {k: torch.randn((M, k), device=dev, generator=gen).to(torch.float16) for k in (4096, 11008)}
    outs = {n: torch.empty((M, n), dtype=torch.float16, device=dev) for n in (12288, 4096, 22016)}
    ws_bytes = max(capi.w4a16_workspace_bytes(M, n, k) for _, k, n in SHAPES_7B)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    sp = stream.cuda_stream

    def step(i):
        for _, k, n, w, sz in layers[i % len(layers)].weights:
            capi.w4a16_gemm(dtype, outs[n], acts[k], w, sz, M, n, k, GROUP, workspace, ws_bytes, sp)

    # which kernel instantiation serves each GEMM of the step (the library's launch log, read back per call)
    capi.set_launch_log(True)
    launched = {}
    for name, k, n, w, sz in layers[0].weights:
        capi.w4a16_gemm(dtype, outs[n], acts[k], w, sz, M, n, k, GROUP, workspace, ws_bytes, sp)
        launched[name] = capi.last_launch()
    capi.set_launch_log(False)

    with torch.cuda.stream(stream):
        for i in range(args.warmup):
            step(i)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(args.steps):
                step(i)
        graph.replay()  # untimed: first replay uploads the graph
        stream.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record(stream)
        graph.replay()
        ev1.record(stream)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        gpu_ms = ev0.elapsed_time(ev1)

    # a plain device copy of known size (256 MiB read + 256 MiB written): the yardstick that the HBM traffic
    # counters of a profiled run are scaled by
    calib = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    calib2 = torch.empty_like(calib)
    calib2.copy_(calib)
    torch.cuda.synchronize()
    del calib, calib2

    step_bytes = sum(w4a16_bytes(M, k, n) for _, k, n in SHAPES_7B)
    ms_per_step = wall_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    launches = args.steps * len(SHAPES_7B)
    avg_launch_us = gpu_ms * 1e3 / launches
    achieved = (step_bytes / len(SHAPES_7B)) / (avg_launch_us * 1e-6) / 1e9
    # HBM traffic per launch comes from a rocprofv3 --pmc run of this same command (profiles/): it is attached only if
    # that run launched the very kernel instantiations that this run did
    traffic, traffic_note, profiled = None, None, {}
    if os.path.exists(TRAFFIC_FILE):
        for line in open(TRAFFIC_FILE):
            if line.startswith("traffic_bytes_per_launch:"):
                traffic = float(line.split(":")[1])
            if line.startswith("launched "):
                name, what = line[len("launched "):].split(":", 1)
                profiled[name.strip()] = what.strip()
        if profiled != launched:
            traffic = None
            traffic_note = "profiles/ was taken with other kernel instantiations than this run launched: not attached"

    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": f"configs[1]: Llama-2-7B decode, AWQ int4 g=128, fp16 act, M={M}; step = qkv+o+gate_up+down "
                        f"GEMMs of one layer, {args.layers} layers rotated",
            "bytes_per_step": step_bytes,
            "peaks_divided_by": {"hbm_GBps": HBM_PEAK_GBPS, "mfma_f16_TFLOPs": MFMA_F16_PEAK_TFLOPS,
                                 "mfma_fp8_TFLOPs": MFMA_FP8_PEAK_TFLOPS},
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "w4a16_kstat_kernel",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "avg_launch_us": round(avg_launch_us, 3),
            "launches": launches,
            "launched": launched,
        },
    }
    if traffic_note:
        result["roofline"]["traffic_note"] = traffic_note
    if args.only == "headline":
        print(json.dumps(result), flush=True)
        return

    # the TFLOP/s half of the metric: always measured, carried inside `roofline`; configs[2] has bf16 activations, so
    # its weights are repacked with bf16 scales (the same values cast)
    layer_bf16 = Layer(torch, capi, dev, 1000, capi.BF16)
    m4096 = prefill(torch, capi, layer_bf16, stream, gen)
    result["roofline"]["mfma"] = mfma_half(m4096)

    extra = {}
    if not args.no_extra:
        extra["prefill_m4096"] = m4096
        extra["per_shape"] = per_shape(torch, capi, layers[0], stream, M, dtype, gen)
        for m2 in (1, 4, 64):  # the other batch sizes of configs[1]
            if m2 != M:
                extra[f"decode_m{m2}"] = per_shape(torch, capi, layers[0], stream, m2, dtype, gen)
        extra["fused_m16"] = fused(torch, capi, layers[0], stream, M, dtype, dev, gen)
        extra["prefill_m4096_f16"] = prefill(torch, capi, layers[0], stream, gen, "f16")
        extra["prefill_m2048"] = prefill(torch, capi, layer_bf16, stream, gen, M=2048)
        extra["prefill_m512"] = prefill(torch, capi, layer_bf16, stream, gen, M=512)
        extra["prefill_m128"] = prefill(torch, capi, layer_bf16, stream, gen, M=128)  # between configs[1] and [2]
        extra["prefill_m512_f16"] = prefill(torch, capi, layers[0], stream, gen, "f16", M=512)
        del layer_bf16
        del layers[1:]
        torch.cuda.empty_cache()
        extra["fp8_cfg4"] = fp8_sweep(torch, capi, dev, stream)
        extra["fp8_row_maxima_from_producer"] = fp8_rowmax_chain(torch, capi, dev, stream)
        extra["gptq_70b_cfg3"] = gptq_70b_sweep(torch, capi, dev, stream)
    if not args.no_cpu:
        del layers[1:]
        torch.cuda.empty_cache()
        base, parity, parity_m4096, clocks = cpu_baseline(np, torch, capi, layers[0], acts, outs, workspace, ws_bytes,
                                                          M, dtype, step_bytes, stream, gen)
        result["cpu_baseline"] = base
        extra["parity_vs_cpu"] = parity
        extra["parity_vs_cpu_m4096"] = parity_m4096
        result["config"]["gpu_sclk_observed"] = clocks["gpu_sclk"]
    if extra:
        result["extra"] = extra
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
