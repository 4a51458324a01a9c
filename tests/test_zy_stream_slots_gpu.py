"""Split-K arrival counters are owned per stream: the first 64 streams of a device that launch a split-K kernel get a
region each, any later stream runs the same GEMM without a split across workgroups.  This file runs late on purpose:
it uses up every region of the process."""
import ctypes

import numpy as np
import pytest

from oracle import oracle as orc
from tests.ksq_testlib import W4Case, W4Device, capi_dtype, torch_dtype

pytestmark = pytest.mark.gpu


def test_more_streams_than_counter_regions(gpu):
    import torch

    from ksanallm_amd import capi

    print("\n[case] 80 streams, split-K shape M=16 K=8192 N=272", flush=True)
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    case = W4Case(7100, 16, 8192, 272, kind="awq", dtype="f16")   # 64 k tiles: split in two by the planner
    dev = W4Device(case, gpu)
    assert dev.workspace_bytes > 0
    want = case.oracle()
    first = None
    streams = []
    try:
        for i in range(80):
            h = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(h)) == 0
            streams.append(h)
            out = torch.full((case.M, case.N), float("nan"), dtype=torch_dtype(case.dtype), device=gpu)
            for _ in range(2):  # twice per stream: the counters must be back at zero
                capi.w4a16_gemm(capi_dtype(case.dtype), out, dev.act, dev.weight, dev.sz, case.M, case.N, case.K, case.g,
                                dev.workspace, dev.workspace_bytes, h.value)
                assert hip.hipStreamSynchronize(h) == 0
            got = out.float().cpu().numpy()
            orc.assert_parity(got, want, f"stream {i}")
            if first is None:
                first = got
            elif i < 40:
                assert np.array_equal(got, first), f"stream {i}: same plan, same bits expected"
    finally:
        for h in streams:
            hip.hipStreamDestroy(h)
