"""The launch entry point that allocates nothing (rl_gemm_plan_launch_static) against
rl_gemm_plan_launch, through the C ABI on an MI355X: the same kernel with the same split, so the
same bits -- on two calls in a row, the second with a smaller input that finds the scratch array
as the first one left it."""

import numpy as np
import pytest

from mlir_roller_amd import hip
from mlir_roller_amd.hip import DeviceArray, GemmConfig, GemmPlan, HipError
from oracle import gemm_oracle as go

pytestmark = pytest.mark.gpu


def both_ways(plan, A, B):
    M, K = A.shape
    N = B.shape[1]
    dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B)
    outs = []
    for workspace in (None, "static"):
        dC = DeviceArray((M, N))
        dC.fill_bytes(0xFF)
        plan.launch(dA, dB, dC, M, N, K, workspace=workspace)
        hip.synchronize()
        outs.append(dC.get())
    return outs


def test_static_scratch_launch_matches_the_allocating_one(device):
    cfg = GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 2)
    plan = GemmPlan(cfg)
    for shape, dist in (((1500, 1300, 1100), "uniform"), ((700, 500, 260), "uniform"), ((1500, 1300, 1100), "integer"), ((130, 260, 96), "integer")):
        sched = hip.streamk_schedule(cfg, *shape, device.compute_units)
        assert sched.units > sched.tiles and sched.grid > sched.tiles        # every tile is split
        A, B = go.make_inputs(*shape, seed=shape[0], distribution=dist)
        allocating, static = both_ways(plan, A, B)
        assert np.array_equal(allocating.view(np.uint32), static.view(np.uint32)), shape
        if dist == "integer":
            assert np.array_equal(static, go.c_gemm_f32(A, B))
        else:
            assert go.error_report(static, A, B)["ok"]


def test_static_scratch_launch_of_a_plain_plan_and_of_degenerate_extents(device):
    plain = GemmPlan(GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 0))
    A, B = go.make_inputs(300, 260, 200, seed=1, distribution="integer")
    a, b = both_ways(plain, A, B)
    assert np.array_equal(a, b) and np.array_equal(b, go.c_gemm_f32(A, B))
    plan = GemmPlan(GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 2))
    dA, dB, dC = DeviceArray.zeros((64,)), DeviceArray.zeros((64,)), DeviceArray((8, 12))
    dC.fill_bytes(0xFF)
    plan.launch(dA, dB, dC, 8, 12, 0, workspace="static")           # K = 0: zeros, from a fill kernel
    hip.synchronize()
    assert not dC.get().any()


def test_static_scratch_launch_refuses_what_does_not_fit(device):
    # 256 x 256 tiles, one workgroup per CU: 2 * 256 * 256 KiB of slots = 128 MiB > 64 MiB
    plan = GemmPlan(GemmConfig(256, 256, 32, 128, 128, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 1))
    M = N = K = 4096
    dA, dB, dC = DeviceArray((M, K)), DeviceArray((K, N)), DeviceArray((M, N))
    with pytest.raises(HipError, match="static scratch"):
        plan.launch(dA, dB, dC, M, N, K, workspace="static")
    plan.launch(dA, dB, dC, M, N, K)                                  # the allocating entry point takes it
    hip.synchronize()
