"""The launch contract of the C ABI on the GPU: every entry point only enqueues on the stream it is given, so a
sequence of calls can be captured into a HIP graph and replayed, and independent calls may overlap on several streams
(each with a workspace of its own; the split-K arrival counters rotate over 16 library-owned sets).  Results are
deterministic, so replays and concurrent runs are compared bit for bit with a plain serial run."""
import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import W4Case, W4Device, capi_dtype, torch_dtype

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def _fp8_inputs(gpu, M, K, N, seed):
    import torch

    rng = np.random.default_rng(seed)
    x = orc.to_bits(rng.standard_normal((M, K)).astype(np.float32), orc.BF16)
    w = (rng.standard_normal((N, K)) * 0.03).astype(np.float32)
    ws = orc.fp8_compute_scale(w, orc.F32, N, K)
    wq = orc.fp8_quantize(w, orc.F32, ws, N, K)
    return (torch.from_numpy(x.view(np.int16)).to(gpu).view(torch.bfloat16), torch.from_numpy(wq).to(gpu),
            torch.from_numpy(ws).to(gpu), x, wq, ws)


def test_graph_capture_and_replay(gpu):
    """One graph holding every kind of launch the library makes: split-K decode (arrival counters), the
    accumulator-stationary kernel, the two-kernel bf16 large-M route, a desc_act gather + GEMM with an epilogue, and FP8
    quantise + GEMM.  Replayed three times with eager work in between; every replay must equal the eager result."""
    import torch

    from ksanallm_amd import capi

    stream = torch.cuda.Stream(device=gpu)
    cases = [W4Case(3000, 16, 11008, 256, kind="awq", dtype="f16"),    # K beyond one workgroup: split over grid.y
             W4Case(3001, 40, 2048, 1024, kind="gptq", dtype="f16"),
             W4Case(3002, 200, 1024, 512, kind="awq", dtype="bf16"),
             W4Case(3003, 24, 1024, 512, kind="gptq", dtype="bf16"),
             W4Case(3004, 100, 12288, 272, kind="awq", dtype="f16")]   # 64-row large-M kernel, K split in two
    devs = [W4Device(c, gpu) for c in cases]
    perm = torch.from_numpy(np.random.default_rng(3004).permutation(1024).astype(np.int32)).to(gpu)
    bias = torch.from_numpy(orc.to_bits(np.random.default_rng(3005).standard_normal(512).astype(np.float32),
                                        orc.BF16).view(np.int16)).to(gpu)
    ex_bytes = capi.w4a16_workspace_bytes_ex(24, 512, 1024, True)
    ex_ws = torch.empty(max(ex_bytes, 256), dtype=torch.uint8, device=gpu)
    xa, wq, ws, *_ = _fp8_inputs(gpu, 48, 2048, 768, 3006)
    aq = torch.empty((48, 2048), dtype=torch.uint8, device=gpu)
    a_s = torch.empty(48, dtype=torch.float32, device=gpu)
    f8_bytes = capi.fp8_workspace_bytes(48, 768, 2048)
    f8_ws = torch.empty(max(f8_bytes, 256), dtype=torch.uint8, device=gpu)
    outs = [torch.empty((c.M, c.N), dtype=torch_dtype(c.dtype), device=gpu) for c in cases]
    out_ex = torch.empty((24, 512), dtype=torch.bfloat16, device=gpu)
    out_f8 = torch.empty((48, 768), dtype=torch.bfloat16, device=gpu)

    def enqueue(s):
        for c, d, o in zip(cases, devs, outs):
            capi.w4a16_gemm(capi_dtype(c.dtype), o, d.act, d.weight, d.sz, c.M, c.N, c.K, c.g, d.workspace,
                            d.workspace_bytes, s)
        c, d = cases[3], devs[3]
        capi.w4a16_gemm_ex(capi.BF16, out_ex, d.act, d.weight, d.sz, c.M, c.N, c.K, c.g, perm, capi.EPILOGUE_BIAS, bias,
                           ex_ws, ex_bytes, s)
        capi.fp8_quantize(capi.BF16, xa, 48, 2048, capi.FP8_PER_TOKEN_DYNAMIC, aq, a_s, s)
        capi.fp8_gemm(capi.BF16, out_f8, aq, a_s, 48, wq, ws, 768, 48, 768, 2048, f8_ws, f8_bytes, s)

    def snapshot():
        torch.cuda.synchronize()
        return [o.clone() for o in outs + [out_ex, out_f8]]

    def clear():
        for o in outs + [out_ex, out_f8]:
            o.zero_()
        aq.zero_()
        a_s.zero_()

    with torch.cuda.stream(stream):
        enqueue(stream.cuda_stream)
    want = snapshot()
    orc.assert_parity(want[0].float().cpu().numpy(), cases[0].oracle(), "eager split-K")
    orc.assert_parity(want[2].float().cpu().numpy(), cases[2].oracle(), "eager bf16 large M")

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            enqueue(stream.cuda_stream)
    for replay in range(3):
        clear()
        # eager work of the program between replays, on the same buffers' allocator and another stream
        scratch = torch.randn(1 << 20, device=gpu).sum().item()
        assert scratch == scratch
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            graph.replay()
        got = snapshot()
        for i, (g_, w_) in enumerate(zip(got, want)):
            assert torch.equal(g_, w_), f"replay {replay}: output {i} differs from the eager run"


def test_concurrent_streams_with_split_k(gpu):
    """Four streams, each with its own workspace, run split-K GEMMs at the same time for several rounds: the arrival
    counters of concurrent launches must not interfere."""
    import torch

    from ksanallm_amd import capi

    cases = [W4Case(3100 + i, 16 if i % 2 else 7, 11008, 512, kind="awq", dtype="f16") for i in range(4)]
    devs = [W4Device(c, gpu) for c in cases]
    serial = [d.gemm() for d in devs]
    streams = [torch.cuda.Stream(device=gpu) for _ in cases]
    outs = [torch.empty_like(s) for s in serial]
    torch.cuda.synchronize()
    for rnd in range(6):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        for c, d, o, s in zip(cases, devs, outs, streams):
            for _ in range(3):  # back-to-back launches on one stream share its workspace in order
                capi.w4a16_gemm(capi_dtype(c.dtype), o, d.act, d.weight, d.sz, c.M, c.N, c.K, c.g, d.workspace,
                                d.workspace_bytes, s.cuda_stream)
        torch.cuda.synchronize()
        for i, (o, w) in enumerate(zip(outs, serial)):
            assert torch.equal(o, w), f"round {rnd}: stream {i} differs from the serial result"


def test_fp8_concurrent_streams(gpu):
    import torch

    from ksanallm_amd import capi

    M, K, N = 8, 29568 // 2, 512  # K beyond 64 stages: split over grid.y
    sets = []
    for i in range(3):
        xa, wq, ws, x, wq_h, ws_h = _fp8_inputs(gpu, M, K, N, 3200 + i)
        aq = torch.empty((M, K), dtype=torch.uint8, device=gpu)
        a_s = torch.empty(M, dtype=torch.float32, device=gpu)
        nbytes = capi.fp8_workspace_bytes(M, N, K)
        sets.append(dict(xa=xa, wq=wq, ws=ws, aq=aq, a_s=a_s, wk=torch.empty(max(nbytes, 256), dtype=torch.uint8, device=gpu),
                         nbytes=nbytes, out=torch.empty((M, N), dtype=torch.bfloat16, device=gpu), x=x, wq_h=wq_h, ws_h=ws_h))

    def run(d, s):
        capi.fp8_quantize(capi.BF16, d["xa"], M, K, capi.FP8_PER_TOKEN_DYNAMIC, d["aq"], d["a_s"], s)
        capi.fp8_gemm(capi.BF16, d["out"], d["aq"], d["a_s"], M, d["wq"], d["ws"], N, M, N, K, d["wk"], d["nbytes"], s)

    for d in sets:
        run(d, None)
    torch.cuda.synchronize()
    serial = [d["out"].clone() for d in sets]
    d0 = sets[0]
    xs = orc.fp8_compute_scale(d0["x"], orc.BF16, M, K)
    xq = orc.fp8_quantize(d0["x"], orc.BF16, xs, M, K)
    orc.assert_parity(serial[0].float().cpu().numpy(), orc.fp8_gemm(xq, xs, d0["wq_h"], d0["ws_h"]), "fp8 split-K")
    streams = [torch.cuda.Stream(device=gpu) for _ in sets]
    for rnd in range(4):
        for d in sets:
            d["out"].zero_()
        torch.cuda.synchronize()
        for d, s in zip(sets, streams):
            run(d, s.cuda_stream)
            run(d, s.cuda_stream)
        torch.cuda.synchronize()
        for i, (d, w) in enumerate(zip(sets, serial)):
            assert torch.equal(d["out"], w), f"round {rnd}: stream {i}"
