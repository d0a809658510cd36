"""Property tests of the host policy over random problem sizes (hypothesis): the product equals
the independent restatement on the reference's device model, and on MI355X every emitted hint
maps to a kernel configuration that the C ABI accepts."""

import math

from hypothesis import given, settings, strategies as st

from mlir_roller_amd import hip
from mlir_roller_amd.analyze import MatmulConfig, Policy, get_roller_hints
from mlir_roller_amd.arch import CUDA, MI355X
from mlir_roller_amd.roller import hint_to_gemm_config
from oracle import policy_oracle as po

dims = st.sampled_from([16, 24, 48, 64, 96, 100, 128, 160, 192, 250, 256, 320, 384, 512, 768, 1000, 1024, 1536, 2048])


def row(td):
    return [*td.block_tile, *td.thread_tile, td.rstep, td.traffic, td.smem_cost, td.block_per_SM, td.num_wave, td.grid_size]


@settings(max_examples=40, deadline=None)
@given(dims, dims, dims)
def test_product_equals_restatement_on_the_a100_model(M, N, K):
    got = [row(h) for h in get_roller_hints(MatmulConfig(M, N, K, 32), CUDA(), topk=8)]
    want = [[*h["block_tile"], *h["thread_tile"], h["rstep"], h["traffic"], h["smem_cost"], h["block_per_SM"],
             h["num_wave"], h["grid_size"]] for h in po.hints(M, N, K, 8)]
    assert got == want


@settings(max_examples=40, deadline=None)
@given(st.integers(1, 5000), st.integers(1, 5000), st.integers(1, 5000))
def test_every_mi355x_hint_is_a_valid_kernel_configuration(hip_lib, M, N, K):
    cfg = MatmulConfig(M, N, K, 32)
    arch = MI355X()
    hints = get_roller_hints(cfg, arch, topk=12)
    assert hints, (M, N, K)
    policy = Policy(cfg, arch)
    estimates = [policy.estimate_seconds(h) for h in hints]
    assert all(e > 0 and math.isfinite(e) for e in estimates)
    for h in hints:
        g = hint_to_gemm_config(cfg, h, 3)
        lds, threads = hip.config_check(g)              # the C ABI's own validation
        assert threads == h.threads and lds <= arch.lds_bytes
        # K ragged (or dword-aligned rows loaded straight into LDS: always all three tests) / only M, N ragged / aligned
        assert g.edge == (1 if K % g.bk or (g.direct and g.vec == 1) else (2 if (M % g.bm or N % g.bn) else 0))
        assert g.vec == (4 if K % 4 == 0 and N % 4 == 0 else 1)
        assert h.grid_size == math.ceil(M / g.bm) * math.ceil(N / g.bn)
