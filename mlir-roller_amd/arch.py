"""Hardware descriptions consumed by the rTile policy.

``TileDevice`` and ``CUDA`` keep the field names and the A100 numbers of
/root/reference/src/arch.py:9-61, so a policy run on ``CUDA()`` reproduces the reference's
ranking.  ``MI355X`` is the model this package is built for.  The extra fields at the end of
``TileDevice`` default to the constants that the reference hard-codes inside its policy
(src/analyze.py:145, :361), which is what lets one policy serve both devices.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Tuple


@dataclass
class TileDevice:
    """One accelerator as the policy sees it.  Capacities are per compute core (SM / CU)."""

    reg_cap: int = 0            # 32-bit registers per core
    smem_cap: int = 0           # workgroup-memory bytes one block may use per pipeline stage
    compute_max_core: int = 0   # number of cores (SMs / CUs)
    warp_size: int = 0          # lanes that execute in lockstep
    sm_partition: int = 0       # schedulers (SIMDs) per core
    max_smem_usage: int = 0     # workgroup-memory bytes all resident blocks of a core may use
    platform: str = "unknown"
    compute_capability: str = "unknown"
    l2_cache_size_bytes: int = 0
    # [global write, workgroup-memory read] transaction sizes in bytes
    transaction_size: List[int] = field(default_factory=lambda: [0, 0])
    # [device memory, workgroup memory] bandwidth, GB/s
    bandwidth: List[int] = field(default_factory=lambda: [0, 0])

    # ---- not in the reference's dataclass; defaults = the reference's hard-coded constants ----
    # a block tile [m, n] is charged int(2*m*n*el_bytes / reg_estimate_divisor) registers
    reg_estimate_divisor: int = 32
    # a per-lane accumulator tile needing this many 32-bit registers or more is rejected
    thread_reg_limit: int = 256
    # elements of padding the kernel adds to every row of the [m, rstep] workgroup-memory tile
    # when it cannot use its unpadded (swizzled) layout
    lds_row_pad: int = 0
    # warps per scheduler that the block-size recommendation aims for
    waves_per_partition: int = 1
    # 32-bit registers one lane can address when a scheduler hosts a single warp (0 = not modelled)
    regs_per_lane: int = 0
    # matrix-instruction shapes (m, n, k); empty = no matrix cores modelled, SIMT outer product
    mfma_shapes: List[Tuple[int, int, int]] = field(default_factory=list)
    # dies with a private L2 that the dispatcher deals workgroups to round-robin
    xcd_count: int = 1
    # dense matrix peak for the dtype of the GEMM, TFLOP/s (0 = unknown)
    peak_matrix_tflops: float = 0.0
    # peak engine clock, MHz (0 = unknown)
    clock_mhz: int = 0
    # ranking model of devices with matrix cores (``Policy.estimate_seconds``): the matrix pipe's
    # issue efficiency on a block tile [m, n] is base - slope * (1/m + 1/n), and every tile pays
    # ``tile_fixed_seconds`` (pipeline fill) on top of storing its results; workgroups that share a
    # core fill one another's barrier stalls, which adds ``co_resident_gain`` to the efficiency
    mfma_efficiency: Tuple[float, float] = (1.0, 0.0)
    co_resident_gain: float = 0.0
    tile_fixed_seconds: float = 0.0
    # extra loss of issue efficiency per unit of (1/m + 1/n) beyond ``small_tile_knee``
    small_tile_slope: float = 0.0
    small_tile_knee: float = 1.0 / 64 + 1.0 / 128
    # shortest time one reduce step of one workgroup can take, whatever its arithmetic (0 = no floor),
    # and how much faster than device memory the caches deliver operand bytes that are read again
    step_latency_seconds: float = 0.0
    cache_bandwidth_ratio: float = 1.0
    # wave tiles of at most this many elements list the matrix instruction with the longer k first
    long_k_mfma_up_to: int = 0
    # whether the reduce step of a tile grows to what its share of workgroup memory allows (longer
    # contiguous rows, fewer loop trips: the reference's rule) or stays at the shortest step that
    # suits the loads (smaller stages, more blocks resident on a core)
    grow_reduce_step: bool = True
    # Stream-K: workgroups per core that a kernel may keep working through equal shares of all
    # (tile, reduce step) units instead of taking one tile each (0 = the device's kernels cannot).
    # Such a kernel pays no round of blocks that is only partly filled; it runs its reduce steps
    # ``stream_k_loss`` less efficiently, pays ``stream_k_fixed_seconds`` once for storing and adding up
    # the pieces of split tiles, and is preferred when the estimate gains more than ``stream_k_margin``.
    stream_k_workgroups: int = 0
    stream_k_loss: float = 0.0
    stream_k_fixed_seconds: float = 0.0
    stream_k_piece_bandwidth: float = 1.0e9    # GB/s at which one workgroup reads the pieces of a split tile back
    stream_k_margin: float = 0.0

    def get_avaliable_tensorintrin_shapes(self) -> List[Tuple[int, int, int]]:
        """Matrix-instruction shapes of the device (name kept from the reference, arch.py:36)."""
        if not self.mfma_shapes:
            raise NotImplementedError(f"{self.platform} model has no matrix-instruction shapes")
        return list(self.mfma_shapes)

    @property
    def has_matrix_cores(self) -> bool:
        return bool(self.mfma_shapes)


@dataclass
class CUDA(TileDevice):
    """NVIDIA A100 exactly as the reference models it (arch.py:41-61)."""

    platform: str = "CUDA"
    reg_cap: int = 65536
    smem_cap: int = 64 * 1024
    compute_max_core: int = 108
    warp_size: int = 32
    sm_partition: int = 4
    transaction_size: List[int] = field(default_factory=lambda: [32, 128])
    bandwidth: List[int] = field(default_factory=lambda: [750, 12080])
    max_smem_usage: int = field(init=False)

    def __post_init__(self) -> None:
        self.max_smem_usage = 2 * self.smem_cap


@dataclass
class MI355X(TileDevice):
    """AMD Instinct MI355X (gfx950, CDNA4).

    256 CUs in 8 XCDs, four SIMDs per CU, 64-lane wavefronts.  Every SIMD holds 512 32-bit
    registers per lane (256 architectural + 256 accumulation registers), so a CU holds
    4 * 512 * 64 = 131072.  A CU has 160 KB of LDS and one workgroup may take all of it; the
    kernel double-buffers its operand tiles, so the budget of one pipeline stage is half of that.
    fp32 MFMA (v_mfma_f32_32x32x2_f32 / v_mfma_f32_16x16x4_f32) retires 256 FLOP per clock per CU:
    256 CUs * 256 * 2.4 GHz = 157.3 TFLOP/s.  HBM3E delivers 8 TB/s; the LDS figure is
    256 CUs * 128 B/clk * 2.4 GHz.
    """

    platform: str = "ROCm"
    compute_capability: str = "gfx950"
    reg_cap: int = 4 * 512 * 64
    lds_bytes: int = 160 * 1024
    compute_max_core: int = 256
    warp_size: int = 64
    sm_partition: int = 4
    l2_cache_size_bytes: int = 4 * 1024 * 1024
    transaction_size: List[int] = field(default_factory=lambda: [64, 128])
    bandwidth: List[int] = field(default_factory=lambda: [8000, 78643])
    # accumulators (m*n) plus about as much again for operand fragments and staging registers
    reg_estimate_divisor: int = 4
    # 256 accumulation registers per lane are available next to the architectural ones
    thread_reg_limit: int = 257
    # the kernel's register-staged path pads every row of the LDS A tile by one 16-byte unit; its
    # direct-to-LDS path (the pipelined loop with a power-of-two reduce step) swizzles instead
    lds_row_pad: int = 4
    # waves per SIMD that the block-size recommendation tries first: one per workgroup (fitted to
    # the committed sweep, see ``calibrate.py``: a workgroup of eight waves takes 1.003 x the time of
    # one of four on the same block tile); further waves on a SIMD come from other workgroups
    # that are resident on the CU at the same time
    waves_per_partition: int = 1
    # 256 architectural + 256 accumulation registers per lane, shared by the waves of a SIMD
    regs_per_lane: int = 512
    mfma_shapes: List[Tuple[int, int, int]] = field(default_factory=lambda: [(32, 32, 2), (16, 16, 4)])
    xcd_count: int = 8
    peak_matrix_tflops: float = 157.3
    clock_mhz: int = 2400
    # fitted to the committed sweep under calibration/ by ``python -m mlir_roller_amd.calibrate fit``
    # (a test refits them): 0.980 for 256x256 tiles, 0.974 + 0.007 for 128x128 with two on a CU,
    # 0.968 + 0.007 for 64x128; below that knee the efficiency falls 2.7 per unit of (1/m + 1/n)
    # faster (0.94 for 64x64, 0.89 for 32x64)
    mfma_efficiency: Tuple[float, float] = (0.986, 0.75)
    co_resident_gain: float = 0.007
    small_tile_slope: float = 2.7
    tile_fixed_seconds: float = 1.0e-6
    # chosen on the committed sweep, not fitted in closed form: 0.2-0.4 us and ratios of 2.5-4 rank
    # its kernels identically (a test holds both ends); without the two, whole tiles of 32 x 32 lead on
    # problems with a long K and few tiles, where they take twice the time of the best kernel
    step_latency_seconds: float = 0.3e-6
    cache_bandwidth_ratio: float = 3.0
    # 16x16x4 wins on every wave tile it fits (up to 64x128; a wave keeps at most 32 blocks), by
    # 0.5-2 % in the committed sweep
    long_k_mfma_up_to: int = 64 * 128
    # a 32-wide K step already reads whole 128-byte lines; a longer one only takes the LDS that a
    # second workgroup on the CU would use and lengthens the fill of the pipeline (measured: 128x128
    # tiles at K steps of 32 against 64, 64x64 at 32 / 64 / 128: the shortest wins or ties)
    grow_reduce_step: bool = False
    # fitted like the constants above: stream-K against plain kernels of the same tile on problems that
    # fill whole rounds (0.3 % slower), and the rate at which the last workgroup of a tile that is split
    # many ways reads the pieces back (33 GB/s: a round trip past the L2 each); about 5 us per launch besides
    stream_k_workgroups: int = 2
    stream_k_loss: float = 0.003
    stream_k_fixed_seconds: float = 5.0e-6
    stream_k_piece_bandwidth: float = 33.0
    stream_k_margin: float = 0.02
    smem_cap: int = field(init=False)
    max_smem_usage: int = field(init=False)

    def __post_init__(self) -> None:
        self.smem_cap = self.lds_bytes // 2
        self.max_smem_usage = self.lds_bytes // 2

    @classmethod
    def from_device(cls, props) -> "MI355X":
        """Model with the CU count, clock and LDS size that the runtime reports
        (``rl_device_info``) in place of the data-sheet values."""
        model = cls()
        if getattr(props, "compute_units", 0) > 0:
            model.compute_max_core = int(props.compute_units)
        if getattr(props, "lds_bytes_per_block", 0) > 0:
            model.lds_bytes = int(props.lds_bytes_per_block)
            model.__post_init__()
        if getattr(props, "clock_khz", 0) > 0:
            model.clock_mhz = int(props.clock_khz) // 1000
        if getattr(props, "l2_bytes", 0) > 0:
            model.l2_cache_size_bytes = int(props.l2_bytes)
        model.peak_matrix_tflops = model.compute_max_core * 256 * model.clock_mhz * 1e6 / 1e12
        return model
