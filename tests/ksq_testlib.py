"""Shared helpers of the GPU parity tests: seeded synthetic cases in the reference's checkpoint layouts, upload,
repack and GEMM through the C ABI, and the oracle result for the same bytes."""
import numpy as np

from oracle import oracle as orc

ORC_DT = {"f16": orc.F16, "bf16": orc.BF16, "f32": orc.F32}


def torch_dtype(name):
    import torch

    return {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[name]


def capi_dtype(name):
    from ksanallm_amd import capi

    return {"f16": capi.F16, "bf16": capi.BF16, "f32": capi.F32}[name]


class W4Case:
    """One synthetic W4A16 problem: unsigned nibbles u[K,N], zero points z[G,N] (None = symmetric 8), scales and
    activations as 16-bit patterns of ``dtype``."""

    def __init__(self, seed, M, K, N, g=128, kind="awq", dtype="f16", act=None, scales=None):
        rng = np.random.default_rng(seed)
        self.M, self.K, self.N, self.g, self.kind, self.dtype = M, K, N, g, kind, dtype
        G = K // g
        self.u = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
        self.z = rng.integers(0, 16, size=(G, N), dtype=np.uint8) if kind == "awq" else None
        sv = np.abs(rng.standard_normal((G, N))).astype(np.float32) * 0.02 + 1e-3 if scales is None else scales
        self.scales = orc.to_bits(sv, ORC_DT[dtype])
        av = rng.standard_normal((M, K)).astype(np.float32) if act is None else act
        self.act = orc.to_bits(av, ORC_DT[dtype])

    # ---- reference-layout views of the same weights
    def gptq_qweight(self):
        return orc.gptq_pack(self.u)

    def awq_qweight(self):
        return orc.awq_pack(self.u)

    def awq_qzeros(self):
        return orc.awq_pack(self.z)

    def rowmajor(self):
        return orc.rowmajor_pack(self.u)

    def oracle(self, rows=None, cols=None):
        """fp32 dequantize-then-GEMM result (optionally only some activation rows / weight columns)."""
        dt = ORC_DT[self.dtype]
        act = self.act if rows is None else self.act[rows]
        if cols is None:
            return orc.w4a16_forward(act, dt, self.u, self.scales, dt, self.z, self.g)
        u = np.ascontiguousarray(self.u[:, cols])
        s = np.ascontiguousarray(self.scales[:, cols])
        z = np.ascontiguousarray(self.z[:, cols]) if self.z is not None else None
        return orc.w4a16_forward(act, dt, u, s, dt, z, self.g)

    def dequantized(self):
        return orc.dequant(self.u, self.scales, ORC_DT[self.dtype], self.z, self.g)


def _sync(device):
    import torch

    if torch.device(device).type == "cuda":
        torch.cuda.synchronize()


class W4Device:
    """The case on the GPU: repacked through ksq_w4a16_repack from the layout native to its kind."""

    def __init__(self, case, device, layout=None):
        import torch

        from ksanallm_amd import capi

        self.case = case
        self.device = device
        c = case
        wb, sb = capi.w4a16_repack_sizes(c.K, c.N, c.g)
        self.weight = torch.empty(wb, dtype=torch.uint8, device=device)
        self.sz = torch.empty(sb // 4, dtype=torch.int32, device=device)
        if layout is None:
            layout = "gptq" if c.kind == "gptq" else "awq"
        scales = torch.from_numpy(c.scales.view(np.int16)).to(device)
        if layout == "gptq":
            src, lay = torch.from_numpy(c.gptq_qweight()).to(device), capi.W4_GPTQ_INT32_KPACK
        elif layout == "awq":
            src, lay = torch.from_numpy(c.awq_qweight()).to(device), capi.W4_AWQ_INT32_NPACK
        else:
            src, lay = torch.from_numpy(c.rowmajor()).to(device), capi.W4_ROWMAJOR_INT4_SIGNED
        if c.z is None:
            zk, zeros = capi.ZERO_NONE, None
        elif layout == "awq":
            zk, zeros = capi.ZERO_AWQ_INT32, torch.from_numpy(c.awq_qzeros()).to(device)
        else:
            zk, zeros = capi.ZERO_UINT8, torch.from_numpy(c.z).to(device)
        capi.w4a16_repack(lay, src, zk, zeros, scales, capi_dtype(c.dtype), c.K, c.N, c.g, self.weight, self.sz)
        _sync(device)
        self.act = torch.from_numpy(c.act.view(np.int16)).to(device).view(torch_dtype(c.dtype))
        ws = capi.w4a16_workspace_bytes(max(c.M, 1), c.N, c.K)
        self.workspace = torch.empty(max(ws, 16), dtype=torch.uint8, device=device)
        self.workspace_bytes = ws

    def gemm(self, act=None, use_workspace=True):
        import torch

        from ksanallm_amd import capi

        c = self.case
        act = self.act if act is None else act
        m = act.shape[0]
        out = torch.full((m, c.N), float("nan"), dtype=torch_dtype(c.dtype), device=self.device)
        capi.w4a16_gemm(capi_dtype(c.dtype), out, act, self.weight, self.sz, m, c.N, c.K, c.g,
                        self.workspace if use_workspace else None, self.workspace_bytes if use_workspace else 0)
        _sync(self.device)
        return out

    def gemm_f32(self, **kw):
        return self.gemm(**kw).float().cpu().numpy()


def bits_of(t):
    """torch fp16/bf16 tensor -> numpy uint16 bit patterns."""
    import torch

    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
