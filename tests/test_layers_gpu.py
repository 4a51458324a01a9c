"""The C++ layer shims (GroupMatMulLayer / Fp8MatMulLayer built by weight name through the test harness that stands in for KsanaLLM's layer factory, with
the reference's Init / Forward(input_tensors, output_tensors) interface) against the CPU oracle, through the test
driver tests/cpp/layer_driver.cpp.  Also their error conventions (misuse throws std::runtime_error)."""
import os
import subprocess

import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import ORC_DT, W4Case

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "ksanallm_amd", "layer_driver")
DTYPE_ENUM = {"f16": 11, "bf16": 10, "f32": 12}  # TYPE_FP16 / TYPE_BF16 / TYPE_FP32 of the reference's DataType


def _run(args):
    assert os.path.exists(DRIVER), "ksanallm_amd/layer_driver is not built (python -m ksanallm_amd.build)"
    print("[driver]", " ".join(map(str, args)), flush=True)
    p = subprocess.run([DRIVER, *map(str, args)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=120)
    return p.returncode, p.stdout.strip()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("method,layout,zeros,M", [
    ("gptq", "gptq", "none", 16),
    ("awq", "awq", "awq", 5),
    ("awq", "rowmajor", "additive", 33),   # ksana's canonical int4 + additive fp16 zeros, as its loader produces
    ("awq", "rowmajor", "uint8", 130),
])
def test_group_matmul_layer_forward(gpu, tmp_path, dtype, method, layout, zeros, M):
    K, N, g = 1024, 384, 128
    case = W4Case(500 + M, M, K, N, g=g, kind=method, dtype=dtype)
    d = str(tmp_path)
    {"gptq": case.gptq_qweight, "awq": case.awq_qweight, "rowmajor": case.rowmajor}[layout]().tofile(d + "/qweight.bin")
    if zeros == "awq":
        case.awq_qzeros().tofile(d + "/qzeros.bin")
    elif zeros == "uint8":
        case.z.tofile(d + "/qzeros.bin")
    elif zeros == "additive":
        orc.awq_additive_zeros(case.scales, ORC_DT[dtype], case.z).tofile(d + "/qzeros.bin")
    case.scales.tofile(d + "/scales.bin")
    case.act.tofile(d + "/act.bin")
    rc, out = _run(["w4a16", d, dtype, M, K, N, g, method, layout, zeros])
    assert rc == 0 and out.splitlines()[-1] == f"OK {M} {N} {DTYPE_ENUM[dtype]}", out  # shape and dtype set by Forward
    got = orc.from_bits(np.fromfile(d + "/out.bin", dtype=np.uint16).reshape(M, N), ORC_DT[dtype])
    orc.assert_parity(got, case.oracle(), f"GroupMatMulLayer {method}/{layout}/{zeros} {dtype}")


@pytest.mark.parametrize("dtype,extra,layout,M", [
    ("f16", "none", "cutlass80", 16),    # the reference loader's own output, accepted as it is
    ("bf16", "none", "cutlass90", 70),
    ("f16", "desc", "gptq", 24),         # desc_act checkpoint: perm from g_idx, activations gathered at run time
    ("bf16", "desc", "gptq", 130),
    ("f16", "silu", "awq", 16),          # fused gate/up with the SiLU-mul epilogue
    ("bf16", "silu", "awq", 200),
    ("f16", "bias", "awq", 40),
])
def test_group_matmul_layer_widened(gpu, tmp_path, dtype, extra, layout, M):
    """The same layer fed by an untouched CUTLASS-backend loader, serving a desc_act checkpoint, and with the step
    after the GEMM folded in."""
    K, N, g = 1024, 384, 128
    method = "gptq" if layout == "gptq" else "awq"
    case = W4Case(600 + M, M, K, N, g=g, kind=method, dtype=dtype)
    d = str(tmp_path)
    zeros = "none"
    if layout.startswith("cutlass"):
        orc.cutlass_preprocess(case.rowmajor(), int(layout[-2:])).tofile(d + "/qweight.bin")
        orc.awq_additive_zeros(case.scales, ORC_DT[dtype], case.z).tofile(d + "/qzeros.bin")
        zeros = "additive"
    elif layout == "gptq":
        case.gptq_qweight().tofile(d + "/qweight.bin")
    else:
        case.awq_qweight().tofile(d + "/qweight.bin")
        case.awq_qzeros().tofile(d + "/qzeros.bin")
        zeros = "awq"
    case.scales.tofile(d + "/scales.bin")
    case.act.tofile(d + "/act.bin")
    want, cols = case.oracle(), N
    if extra == "desc":
        rng = np.random.default_rng(601)
        order = rng.permutation(K)
        g_idx = np.empty(K, dtype=np.int32)
        g_idx[order] = np.arange(K, dtype=np.int32) // g
        g_idx.tofile(d + "/g_idx.bin")
        s = orc.from_bits(case.scales, ORC_DT[dtype])
        wdq = (s[g_idx] * (case.u.astype(np.float32) - 8.0)).astype(np.float32)
        want = orc.gemm_f32(orc.from_bits(case.act, ORC_DT[dtype]), wdq)
    elif extra == "silu":
        want, cols = orc.silu_mul(want), N // 2
    elif extra == "bias":
        bias = orc.to_bits(np.random.default_rng(602).standard_normal(N).astype(np.float32), ORC_DT[dtype])
        bias.tofile(d + "/bias.bin")
        want = want + orc.from_bits(bias, ORC_DT[dtype])[None, :]
    rc, out = _run(["w4a16", d, dtype, M, K, N, g, method, layout, zeros, extra])
    assert rc == 0 and out.splitlines()[-1] == f"OK {M} {cols} {DTYPE_ENUM[dtype]}", out
    got = orc.from_bits(np.fromfile(d + "/out.bin", dtype=np.uint16).reshape(M, cols), ORC_DT[dtype])
    orc.assert_parity(got, want, f"GroupMatMulLayer {layout} {extra} {dtype}")


@pytest.mark.parametrize("dtype,layout,kind,M", [("f16", "cutlass80", "awq", 16), ("bf16", "cutlass80", "gptq", 70),
                                                 ("f16", "cutlass90", "awq", 5)])
def test_group_matmul_layer_takes_the_reference_loaders_tensors_at_forward(gpu, tmp_path, dtype, layout, kind, M):
    """No load-time repack at all: the weight reaches Forward as KsanaLLM's loader leaves it (CUTLASS-preprocessed
    bytes, `.scales` in T, `.zeros` additive in T or absent) and is converted on first use; two calls, same result."""
    _adopt_case(_run, tmp_path, dtype, layout, kind, M)


def _adopt_case(run, tmp_path, dtype, layout, kind, M):
    K, N, g = 1024, 384, 128
    case = W4Case(660 + M, M, K, N, g=g, kind=kind, dtype=dtype)
    d = str(tmp_path)
    orc.cutlass_preprocess(case.rowmajor(), int(layout[-2:])).tofile(d + "/qweight.bin")
    zeros = "none"
    if kind == "awq":
        orc.awq_additive_zeros(case.scales, ORC_DT[dtype], case.z).tofile(d + "/qzeros.bin")
        zeros = "additive"
    case.scales.tofile(d + "/scales.bin")
    case.act.tofile(d + "/act.bin")
    rc, out = run(["w4a16", d, dtype, M, K, N, g, kind, layout, zeros, "adopt"])
    assert rc == 0 and out.splitlines()[-1] == f"OK {M} {N} {DTYPE_ENUM[dtype]}", out
    got = orc.from_bits(np.fromfile(d + "/out.bin", dtype=np.uint16).reshape(M, N), ORC_DT[dtype])
    orc.assert_parity(got, case.oracle(), f"GroupMatMulLayer loader tensors at Forward {layout} {kind} {dtype}")


@pytest.mark.parametrize("dtype,M,parts", [("f16", 16, None), ("bf16", 70, None), ("f16", 5, [64, 32, 32]),
                                           ("bf16", 130, [64, 64])])
def test_group_matmul_layer_k_not_a_multiple_of_128(gpu, tmp_path, dtype, M, parts):
    """K = 192 under group size 64: the repack pads the last k tile, so the repacked tensors are larger than
    k * n / 2 bytes and k / g * n words -- the layer must size them as the library says (single and fused weight)."""
    _odd_k_case(_run, tmp_path, dtype, M, parts)


def _odd_k_case(run, tmp_path, dtype, M, parts):
    K, g = 192, 64
    N = sum(parts) if parts else 128
    case = W4Case(640 + M, M, K, N, g=g, kind="awq", dtype=dtype)
    d = str(tmp_path)
    n0 = 0
    for i, w in enumerate(parts or []):
        orc.awq_pack(np.ascontiguousarray(case.u[:, n0:n0 + w])).tofile(f"{d}/qweight_{i}.bin")
        orc.awq_pack(np.ascontiguousarray(case.z[:, n0:n0 + w])).tofile(f"{d}/qzeros_{i}.bin")
        np.ascontiguousarray(case.scales[:, n0:n0 + w]).tofile(f"{d}/scales_{i}.bin")
        n0 += w
    case.awq_qweight().tofile(d + "/qweight.bin")
    case.awq_qzeros().tofile(d + "/qzeros.bin")
    case.scales.tofile(d + "/scales.bin")
    case.act.tofile(d + "/act.bin")
    args = ["w4a16", d, dtype, M, K, N, g, "awq", "awq", "awq"]
    if parts:
        args.append("parts:" + ":".join(map(str, parts)))
    rc, out = run(args)
    assert rc == 0 and out.splitlines()[-1] == f"OK {M} {N} {DTYPE_ENUM[dtype]}", out
    got = orc.from_bits(np.fromfile(d + "/out.bin", dtype=np.uint16).reshape(M, N), ORC_DT[dtype])
    orc.assert_parity(got, case.oracle(), f"GroupMatMulLayer K=192 g=64 {dtype} parts={parts}")


@pytest.mark.parametrize("dtype,M", [("f16", 16), ("bf16", 70)])
def test_group_matmul_layer_fused_from_separate_projections(gpu, tmp_path, dtype, M):
    """q_proj / k_proj / v_proj of an AWQ checkpoint as three tensors, repacked side by side into one fused weight
    (RepackFusedGroupQuantWeight) and served by one layer: equals the GEMM against the concatenated weight."""
    K, g = 1024, 128
    widths = [256, 64, 64]
    N = sum(widths)
    case = W4Case(620 + M, M, K, N, g=g, kind="awq", dtype=dtype)
    d = str(tmp_path)
    n0 = 0
    for i, w in enumerate(widths):
        orc.awq_pack(np.ascontiguousarray(case.u[:, n0:n0 + w])).tofile(f"{d}/qweight_{i}.bin")
        orc.awq_pack(np.ascontiguousarray(case.z[:, n0:n0 + w])).tofile(f"{d}/qzeros_{i}.bin")
        np.ascontiguousarray(case.scales[:, n0:n0 + w]).tofile(f"{d}/scales_{i}.bin")
        n0 += w
    case.awq_qweight().tofile(d + "/qweight.bin")   # the driver reads these too; the parts are what it repacks
    case.awq_qzeros().tofile(d + "/qzeros.bin")
    case.scales.tofile(d + "/scales.bin")
    case.act.tofile(d + "/act.bin")
    rc, out = _run(["w4a16", d, dtype, M, K, N, g, "awq", "awq", "awq", "parts:" + ":".join(map(str, widths))])
    assert rc == 0 and out.splitlines()[-1] == f"OK {M} {N} {DTYPE_ENUM[dtype]}", out
    got = orc.from_bits(np.fromfile(d + "/out.bin", dtype=np.uint16).reshape(M, N), ORC_DT[dtype])
    orc.assert_parity(got, case.oracle(), f"fused q/k/v {dtype}")


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("wscales,static,M", [("1", 0, 7), ("1", 1, 7), ("n", 0, 40)])
def test_fp8_matmul_layer_forward(gpu, tmp_path, dtype, wscales, static, M):
    K, N = 512, 208
    rng = np.random.default_rng(600 + M)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    if wscales == "n":
        ws = orc.fp8_compute_scale(w, orc.F32, N, K)
        wq = orc.fp8_quantize(w, orc.F32, ws, N, K)
    else:
        ws = orc.fp8_compute_scale(w, orc.F32, 1, N * K)
        wq = orc.fp8_quantize(w, orc.F32, ws, 1, N * K).reshape(N, K)
    x = orc.to_bits(rng.standard_normal((M, K)).astype(np.float32), ORC_DT[dtype])
    d = str(tmp_path)
    wq.tofile(d + "/wq.bin")
    ws.tofile(d + "/wscale.bin")
    x.tofile(d + "/act.bin")
    if static:
        xs = np.array([0.0201], dtype=np.float32)
        xs.tofile(d + "/iscale.bin")
        xq = orc.fp8_quantize(x, ORC_DT[dtype], xs, 1, M * K).reshape(M, K)
    elif wscales == "n":  # per-channel weight scales select per-token activation scales
        xs = orc.fp8_compute_scale(x, ORC_DT[dtype], M, K)
        xq = orc.fp8_quantize(x, ORC_DT[dtype], xs, M, K)
    else:  # the reference's behaviour: one dynamic scale for the whole activation tensor
        xs = orc.fp8_compute_scale(x, ORC_DT[dtype], 1, M * K)
        xq = orc.fp8_quantize(x, ORC_DT[dtype], xs, 1, M * K).reshape(M, K)
    rc, out = _run(["fp8", d, dtype, M, K, N, wscales, static])
    assert rc == 0 and out.splitlines()[-1] == f"OK {M} {N} {DTYPE_ENUM[dtype]}", out
    raw = np.fromfile(d + "/out.bin", dtype=np.float32 if dtype == "f32" else np.uint16).reshape(M, N)
    got = orc.from_bits(raw, ORC_DT[dtype])
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, wq, ws), f"Fp8MatMulLayer wscales={wscales} static={static} {dtype}")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("per_channel", [0, 1])
def test_fp8_load_time_pipeline(gpu, tmp_path, dtype, per_channel):
    """A checkpoint with separate q/k/v weights in T: on-the-fly conversion, fusion, scale merge (the reference's max
    merge or the exact per-channel one), then the layer; every stage against the oracle."""
    M, K, nq, nkv = 9, 256, 96, 32
    rng = np.random.default_rng(610 + per_channel)
    d = str(tmp_path)
    parts, scales = [], []
    for name, rows, mag in (("wq_src", nq, 0.02), ("wk_src", nkv, 0.05), ("wv_src", nkv, 0.011)):
        w = orc.to_bits((rng.standard_normal((K, rows)) * mag).astype(np.float32), ORC_DT[dtype])
        w.tofile(f"{d}/{name}.bin")
        q, s = orc.fp8_convert_weight(w, ORC_DT[dtype])
        parts.append(q)
        scales.append(s[0])
    x = orc.to_bits(rng.standard_normal((M, K)).astype(np.float32), ORC_DT[dtype])
    x.tofile(d + "/act.bin")
    fused = np.concatenate(parts, axis=0)
    if per_channel:
        want_w = fused
        want_s = np.concatenate([np.full(nq, scales[0]), np.full(nkv, scales[1]), np.full(nkv, scales[2])]).astype(np.float32)
        xs = orc.fp8_compute_scale(x, ORC_DT[dtype], M, K)
        xq = orc.fp8_quantize(x, ORC_DT[dtype], xs, M, K)
    else:
        want_w, want_s = orc.fp8_merge_qkv_max(fused, scales[0], scales[1], scales[2], nq, nkv, nkv)
        xs = orc.fp8_compute_scale(x, ORC_DT[dtype], 1, M * K)
        xq = orc.fp8_quantize(x, ORC_DT[dtype], xs, 1, M * K).reshape(M, K)
    N = nq + 2 * nkv
    rc, out = _run(["fp8load", d, dtype, M, K, nq, nkv, per_channel])
    assert rc == 0 and out.splitlines()[-1] == f"OK {M} {N} {DTYPE_ENUM[dtype]}", out
    got_w = np.fromfile(d + "/fused.bin", dtype=np.uint8).reshape(N, K)
    nz = (want_w & 0x7F) != 0
    assert np.array_equal(got_w[nz], want_w[nz]) and np.all((got_w[~nz] & 0x7F) == 0)
    assert np.array_equal(np.fromfile(d + "/merged_scale.bin", dtype=np.float32), want_s)
    got = orc.from_bits(np.fromfile(d + "/out.bin", dtype=np.uint16).reshape(M, N), ORC_DT[dtype])
    orc.assert_parity(got, orc.fp8_gemm(xq, xs, want_w, want_s), f"fp8 load-time pipeline per_channel={per_channel}")


def test_error_conventions(gpu):
    rc, out = _run(["errors"])
    lines = [ln for ln in out.splitlines() if ln.startswith(("PASS", "FAIL"))]
    assert rc == 0 and len(lines) == 9, out
    assert all(ln.startswith("PASS") for ln in lines), out
