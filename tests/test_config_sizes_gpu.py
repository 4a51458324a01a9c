"""Config-size parity: every shape of the benchmark configurations through the kernels the launch planners pick
on their own (no overrides), against the CPU oracle on a seeded subset of output rows and, for the widest weights,
of output columns.

The weights are far too large to build with numpy in reasonable time on a test box, so they are generated on the GPU
as plain nibbles, packed there into the checkpoint layout (GPTQ int32 [K/8, N] or AWQ int32 [K, N/8]) by a few tensor
operations, and handed to the library's repack as any checkpoint would be.  The packers are first pinned against the
oracle's own packers on a small case.  The oracle then gets exactly the nibbles, zero points, scale bits and
activation bits of the chosen rows and columns.

Bar as everywhere: max relative error <= 1e-2 (denominator floored at the RMS of the oracle output), mean absolute
error <= 2e-3 x RMS."""
import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import ORC_DT, capi_dtype, torch_dtype

pytestmark = pytest.mark.gpu

AWQ_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]  # slot j of an AWQ word holds column 8c + AWQ_ORDER[j]


@pytest.fixture(autouse=True)
def _announce(request):
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


def _pack8(torch, parts):
    """Eight uint8 nibble tensors -> one int32 tensor, part j in bits 4j .. 4j + 3."""
    v = torch.zeros(parts[0].shape, dtype=torch.int64, device=parts[0].device)
    for j, p in enumerate(parts):
        v |= p.to(torch.int64) << (4 * j)
    v = torch.where(v >= 2**31, v - 2**32, v)
    return v.to(torch.int32)


def gptq_pack_device(torch, u):
    K, N = u.shape
    r = u.view(K // 8, 8, N)
    return _pack8(torch, [r[:, j, :] for j in range(8)]).contiguous()


def awq_pack_device(torch, u):
    R, N = u.shape
    r = u.view(R, N // 8, 8)
    return _pack8(torch, [r[:, :, AWQ_ORDER[j]] for j in range(8)]).contiguous()


def test_device_packers_match_oracle_packers(gpu):
    import torch

    rng = np.random.default_rng(9000)
    u = rng.integers(0, 16, size=(256, 64), dtype=np.uint8)
    du = torch.from_numpy(u).to(gpu)
    assert np.array_equal(gptq_pack_device(torch, du).cpu().numpy(), orc.gptq_pack(u))
    assert np.array_equal(awq_pack_device(torch, du).cpu().numpy(), orc.awq_pack(u))


class BigW4:
    """A W4A16 weight of a benchmark shape, built on the GPU and repacked through the C ABI."""

    def __init__(self, torch, gpu, seed, K, N, kind, dtype, g=128):
        from ksanallm_amd import capi

        self.torch, self.gpu, self.K, self.N, self.kind, self.dtype, self.g = torch, gpu, K, N, kind, dtype, g
        gen = torch.Generator(device=gpu)
        gen.manual_seed(seed)
        self.gen = gen
        G = K // g
        self.u = torch.randint(0, 16, (K, N), dtype=torch.uint8, device=gpu, generator=gen)
        self.z = torch.randint(0, 16, (G, N), dtype=torch.uint8, device=gpu, generator=gen) if kind == "awq" else None
        self.scales = (torch.randn((G, N), device=gpu, generator=gen).abs() * 0.02 + 1e-3).to(torch_dtype(dtype))
        wb, sb = capi.w4a16_repack_sizes(K, N, g)
        self.weight = torch.empty(wb, dtype=torch.uint8, device=gpu)
        self.sz = torch.empty(sb // 4, dtype=torch.int32, device=gpu)
        if kind == "awq":
            capi.w4a16_repack(capi.W4_AWQ_INT32_NPACK, awq_pack_device(torch, self.u), capi.ZERO_AWQ_INT32,
                              awq_pack_device(torch, self.z), self.scales, capi_dtype(dtype), K, N, g, self.weight,
                              self.sz)
        else:
            capi.w4a16_repack(capi.W4_GPTQ_INT32_KPACK, gptq_pack_device(torch, self.u), capi.ZERO_NONE, None,
                              self.scales, capi_dtype(dtype), K, N, g, self.weight, self.sz)
        torch.cuda.synchronize()

    def check(self, M, nrows=20, max_cols=4096, what=""):
        """One GEMM at M rows through the product path; the oracle on a subset of rows (and columns)."""
        from ksanallm_amd import capi

        torch, gpu, K, N = self.torch, self.gpu, self.K, self.N
        act = torch.randn((M, K), device=gpu, generator=self.gen).to(torch_dtype(self.dtype))
        out = torch.full((M, N), float("nan"), dtype=torch_dtype(self.dtype), device=gpu)
        wsb = capi.w4a16_workspace_bytes(M, N, K)
        ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device=gpu)
        cdt = capi_dtype(self.dtype)
        capi.w4a16_gemm(cdt, out, act, self.weight, self.sz, M, N, K, self.g, ws, wsb)
        torch.cuda.synchronize()
        out2 = torch.full_like(out, float("nan"))
        capi.w4a16_gemm(cdt, out2, act, self.weight, self.sz, M, N, K, self.g, ws, wsb)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), out2.view(torch.int16)), f"{what}: two runs differ"
        assert not torch.isnan(out.float()).any(), f"{what}: output not fully written"
        rng = np.random.default_rng(M * 31 + N)
        rows = np.unique(np.concatenate([[0, M - 1], rng.choice(M, size=min(M, nrows), replace=False)]))
        if N > max_cols:  # whole 16-column tiles from all over the width, first and last included
            tiles = np.unique(np.concatenate([[0, N // 16 - 1], rng.choice(N // 16, size=max_cols // 16, replace=False)]))
            cols = (tiles[:, None] * 16 + np.arange(16)[None, :]).reshape(-1)
        else:
            cols = np.arange(N)
        tcols = torch.from_numpy(cols).to(gpu)
        trows = torch.from_numpy(rows).to(gpu)
        dt = ORC_DT[self.dtype]
        u = self.u[:, tcols].cpu().numpy()
        z = self.z[:, tcols].cpu().numpy() if self.z is not None else None
        s = self.scales[:, tcols].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        a = act[trows].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        want = orc.w4a16_forward(a, dt, u, s, dt, z, self.g)
        got = out[trows][:, tcols].float().cpu().numpy()
        m = orc.assert_parity(got, want, what)
        print(f"{what}: rows={len(rows)} cols={len(cols)} max_rel={m['max_rel']:.2e} "
              f"mean_abs/rms={m['mean_abs_over_rms']:.2e}", flush=True)


SHAPES_7B = [("qkv", 4096, 12288), ("o", 4096, 4096), ("gate_up", 4096, 22016), ("down", 11008, 4096)]
SHAPES_70B = [("qkv", 8192, 10240), ("o", 8192, 8192), ("gate_up", 8192, 57344), ("down", 28672, 8192)]
SHAPES_72B = [("qkv", 8192, 10240), ("o", 8192, 8192), ("gate_up", 8192, 59136), ("down", 29568, 8192)]


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("name,K,N", SHAPES_7B)
def test_config2_prefill_all_shapes(gpu, name, K, N, dtype):
    """configs[2] (and its fp16 twin): M = 512, 2048 and 4096 at the four Llama-2-7B shapes."""
    import torch

    w = BigW4(torch, gpu, 2100 + K + N, K, N, "awq", dtype)
    for M in (512, 2048, 4096):
        w.check(M, what=f"cfg2 {name} {dtype} M={M}")
    del w
    torch.cuda.empty_cache()


def test_64_row_kernel_more_than_eight_row_blocks(gpu):
    """A shape the planner gives to the 64-row kernel with more than eight row blocks, so that the workgroup order
    walks several super-tile rows."""
    import torch

    w = BigW4(torch, gpu, 2200, 2048, 1024, "awq", "f16")
    for M in (576, 1000):
        w.check(M, what=f"64-row M={M}")


@pytest.mark.parametrize("kind,dtype,K,N", [("awq", "bf16", 4096, 22016), ("awq", "f16", 4096, 22016),
                                            ("gptq", "f16", 28672, 8192)])
def test_wide_shapes_33_to_64_rows(gpu, kind, dtype, K, N):
    """33 to 64 rows on shapes whose columns fill the device several times over (or fill it, with a K long enough to
    split) go through the 64-row kernel of the large-M path, 32 rows and fewer through the decode kernels: both sides
    of that boundary, ragged row counts, bf16 (re-encoded activations) and fp16, and the K split."""
    import torch

    w = BigW4(torch, gpu, 2300 + K + N, K, N, kind, dtype)
    for M in (32, 33, 49, 57, 64):
        w.check(M, what=f"wide {kind} {dtype} K={K} N={N} M={M}")
    del w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("name,K,N", SHAPES_70B)
def test_config3_gptq_70b_all_shapes(gpu, name, K, N):
    """configs[3]: GPTQ symmetric int4, fp16, M = 1, 32 and 256 at the four Llama-3-70B shapes."""
    import torch

    w = BigW4(torch, gpu, 3100 + K + N, K, N, "gptq", "f16")
    for M in (1, 32, 256):
        w.check(M, what=f"cfg3 {name} M={M}")
    del w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("name,K,N", SHAPES_7B)
def test_config1_awq_decode_device_built(gpu, name, K, N):
    """configs[1] once more with device-built weights (M = 1, 4, 16, 64), so that both ways of building a case are
    tied to each other at full size."""
    import torch

    w = BigW4(torch, gpu, 1100 + K + N, K, N, "awq", "f16")
    for M in (1, 4, 16, 64):
        w.check(M, what=f"cfg1 {name} M={M}")
    del w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("name,K,N", SHAPES_72B)
def test_config4_fp8_all_shapes(gpu, name, K, N):
    """configs[4]: e4m3 weights [N, K] with per-channel scales (N(0,1) x 0.02 quantised per output channel by the
    library's own load-time conversion, which has its own bit-exact test), bf16 activations N(0,1) quantised per token,
    M = 1, 64 and 2048, bf16 out; and M = 40 and 100, which the wide shapes (40) and all shapes (100) give to the
    256-row tile kernel with K split over a grid that one round does not fill.  The activation quantisation of the chosen rows is checked bit for bit against the
    oracle, the GEMM to the parity bar."""
    import torch

    from ksanallm_amd import capi

    gen = torch.Generator(device=gpu)
    gen.manual_seed(4100 + K + N)
    wq = torch.empty((N, K), dtype=torch.uint8, device=gpu)
    wscale = torch.empty(N, dtype=torch.float32, device=gpu)
    step = 8192  # output channels converted at a time: bounds the bf16 source held on the device
    for n0 in range(0, N, step):
        n1 = min(N, n0 + step)
        src = (torch.randn((K, n1 - n0), device=gpu, generator=gen) * 0.02).to(torch.bfloat16)
        capi.fp8_convert_weight_per_channel(capi.BF16, src, K, n1 - n0, wq[n0:n1], wscale[n0:n1])
        torch.cuda.synchronize()
        del src
    for M in (1, 40, 64, 100, 2048):
        what = f"cfg4 {name} M={M}"
        act = torch.randn((M, K), device=gpu, generator=gen).to(torch.bfloat16)
        aq = torch.empty((M, K), dtype=torch.uint8, device=gpu)
        ascale = torch.empty(M, dtype=torch.float32, device=gpu)
        capi.fp8_quantize(capi.BF16, act, M, K, capi.FP8_PER_TOKEN_DYNAMIC, aq, ascale)
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=gpu)
        wsb = capi.fp8_workspace_bytes(M, N, K)
        ws = torch.empty(max(wsb, 256), dtype=torch.uint8, device=gpu)
        capi.fp8_gemm(capi.BF16, out, aq, ascale, M, wq, wscale, N, M, N, K, ws, wsb)
        torch.cuda.synchronize()
        out2 = torch.full_like(out, float("nan"))
        capi.fp8_gemm(capi.BF16, out2, aq, ascale, M, wq, wscale, N, M, N, K, ws, wsb)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), out2.view(torch.int16)), f"{what}: two runs differ"
        assert not torch.isnan(out.float()).any(), f"{what}: output not fully written"
        rng = np.random.default_rng(M * 37 + N)
        rows = np.unique(np.concatenate([[0, M - 1], rng.choice(M, size=min(M, 16), replace=False)]))
        cols = np.unique(np.concatenate([[0, N - 1], rng.choice(N, size=min(N, 2048), replace=False)]))
        trows, tcols = torch.from_numpy(rows).to(gpu), torch.from_numpy(cols).to(gpu)
        x_bits = act[trows].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        xs = orc.fp8_compute_scale(x_bits, orc.BF16, len(rows), K)
        xq = orc.fp8_quantize(x_bits, orc.BF16, xs, len(rows), K)
        assert np.array_equal(ascale[trows].cpu().numpy(), xs), f"{what}: activation scales"
        assert np.array_equal(aq[trows].cpu().numpy(), xq), f"{what}: activation bytes"
        want = orc.fp8_gemm(xq, xs, wq[tcols].cpu().numpy(), wscale[tcols].cpu().numpy())
        got = out[trows][:, tcols].float().cpu().numpy()
        m = orc.assert_parity(got, want, what)
        print(f"{what}: rows={len(rows)} cols={len(cols)} max_rel={m['max_rel']:.2e} "
              f"mean_abs/rms={m['mean_abs_over_rms']:.2e}", flush=True)
        del act, aq, out, out2, ws
    del wq
    torch.cuda.empty_cache()
