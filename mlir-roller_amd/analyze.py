"""rTile policy: enumerate, validate, rank and complete tile configurations for one fp32 GEMM.

Host surface of /root/reference/src/analyze.py, kept name for name: ``Shape``, ``MatmulConfig``
(:27-49), ``read_txn_elems`` / ``write_txn_elems`` (:52-59), ``compute_memory_traffic`` (:62-81),
``TileDict`` (:84-168), ``Policy`` (:171-381) and ``get_roller_hints`` (:384-387).

On the reference's ``CUDA()`` device model the hints that come out are the reference's, in the
same order (the golden fixtures under tests/golden pin that).  On a device model that has matrix
cores (``MI355X()``) three things change, all driven by fields of the device model:

* block tiles and reduce steps are multiples of the MFMA granule, and a ladder of such sizes is
  offered next to the exact divisors, because ragged tiles are predicated by the kernel;
* the "thread tile" step assigns a *wave* tile: the block tile is split over wavefronts so that
  every wave owns a grid of MFMA blocks, and ``thread_tile`` is that wave tile seen per lane
  (the 64 lanes as an 8x8 grid), which keeps ``block_tile // thread_tile`` = threads per block;
* candidates are ranked by a roofline estimate of the whole GEMM (``Policy.estimate_seconds``)
  instead of the reference's per-block traffic times wave count.
"""

from __future__ import annotations

import itertools
import math
from dataclasses import dataclass
from typing import Iterator, List, Optional, Sequence

from .arch import CUDA, TileDevice  # noqa: F401  (CUDA re-exported like the reference does)
from .utils import coalesced_factor, coalesced_tensor_shape, factorize, get_all_factors  # noqa: F401


@dataclass
class Shape:
    """Extent of one GEMM operand as (spatial, reduce)."""

    S: int
    R: int

    def to_list(self) -> List[int]:
        return [self.S, self.R]


@dataclass
class MatmulConfig:
    """C[M,N] = A[M,K] * B[K,N] with ``el_bits``-wide elements."""

    M: int
    N: int
    K: int
    el_bits: int

    def get_input_shapes(self):
        # Both operands are described as [spatial, reduce]: for the cost model B counts as
        # [N, K] although it is stored [K, N].
        return Shape(S=self.M, R=self.K), Shape(S=self.N, R=self.K)

    def get_output_shape(self):
        return self.M, self.N

    @property
    def el_bytes(self) -> int:
        return (self.el_bits + 7) // 8

    @staticmethod
    def propagate_inputs(tile: List[int], rstep: int):
        """Operand tiles needed for one output tile and ``rstep`` reduce elements."""
        return Shape(S=tile[0], R=rstep), Shape(S=tile[1], R=rstep)

    @staticmethod
    def propagate_outputs(tile: List[int]):
        return tile


def read_txn_elems(arch: TileDevice, el_bytes: int) -> int:
    """Elements per read transaction."""
    return arch.transaction_size[1] // el_bytes


def write_txn_elems(arch: TileDevice, el_bytes: int) -> int:
    """Elements per write transaction."""
    return arch.transaction_size[0] // el_bytes


def compute_memory_traffic(output_tile: List[int], matmul_config: MatmulConfig, arch: TileDevice) -> int:
    """Bytes one workgroup moves for ``output_tile`` over the whole of K: both operand panels
    in, the tile out, each rounded up to whole transactions."""
    eb = matmul_config.el_bytes
    rte, wte = read_txn_elems(arch, eb), write_txn_elems(arch, eb)
    panels = MatmulConfig.propagate_inputs(output_tile, matmul_config.K)
    moved = sum(
        coalesced_tensor_shape(panel.to_list(), full.to_list(), rte)
        for panel, full in zip(panels, matmul_config.get_input_shapes())
    )
    moved += coalesced_tensor_shape(output_tile, list(matmul_config.get_output_shape()), wte)
    return moved * eb


# Pipeline depth the MI355X sweep runs at (the reference's sweep runs its depth 2,
# /root/reference/src/benchmark.py:29): two LDS buffers plus a register stage.
DEFAULT_PIPELINE_DEPTH = 3


def kernel_stages(pipeline_depth: int) -> int:
    """STAGES of the kernel template for a ``pipeline_depth`` as the reference means it, the number
    of workgroup-memory buffers per operand (/root/reference/src/roller.py:200-205, :385): 1 -> one
    buffer, nothing overlapped; 2 -> two buffers and the fully pipelined loop (template STAGES 3: the
    template's own STAGES 2, two buffers with the loads staged through registers and waited for in
    the open, is kept for explicit configurations only -- it is 13 % slower and needs the same LDS);
    3 -> the same kernel (the depth the MI355X sweep asks for); 4, 5 -> three and four buffers."""
    depth = max(1, int(pipeline_depth))
    return 3 if depth == 2 else depth


def loads_go_direct_to_lds(matmul_config: "MatmulConfig", block_tile: Sequence[int], rstep: int,
                           pipeline_depth: int = DEFAULT_PIPELINE_DEPTH) -> bool:
    """Whether the MFMA kernel built for this tile uses its direct-to-LDS path (unpadded,
    XOR-swizzled rows; no staging registers): on the pipelined loop (pipeline depth 2 and up), with
    a power-of-two reduce step and operand tiles that are whole waves of 16-byte units.  Rows that
    are only dword-aligned (K or N not a multiple of 4) take it with two LDS buffers only (depths 2
    and 3).  The policy's LDS and register models and the mapping from a hint to template parameters
    all ask this one function."""
    m, n = block_tile
    stages = kernel_stages(pipeline_depth)
    aligned = matmul_config.K % 4 == 0 and matmul_config.N % 4 == 0
    return (stages >= 3 and (aligned or stages == 3)
            and rstep & (rstep - 1) == 0 and (m * rstep // 4) % 64 == 0 and (rstep * n // 4) % 64 == 0)


def lds_row_pad(rstep: int, mfma: int) -> int:
    """Floats of padding per row of a K-contiguous LDS tile ([rows][rstep + pad]) on the MFMA kernel's
    register-staged path, chosen so that the 128-bit fragment reads touch every bank once per LDS
    cycle.  With the 32x32x2 instruction a lane group is 32 rows at one k offset: an odd number of
    16-byte units per row does it.  With 16x16x4 the LDS serves quarter-waves of two lane groups (one
    unit apart in k) in the same cycle, and rows of 2 mod 4 units keep them apart (measured with a
    single-wave probe under the profiler: rows of 9 units conflict, rows of 10 do not)."""
    units = rstep // 4
    if mfma == 16:
        return (2 - units) % 4 * 4
    return 0 if units % 2 else 4


def _natural_size(nbytes: float) -> str:
    """1536 -> '1.5 KiB' (binary units, one decimal)."""
    if abs(nbytes) < 1024:
        return f"{int(nbytes)} Bytes"
    value = float(nbytes)
    for unit in ("KiB", "MiB", "GiB", "TiB", "PiB"):
        value /= 1024.0
        if abs(value) < 1024.0 or unit == "PiB":
            return f"{value:.1f} {unit}"
    return f"{value:.1f} PiB"


class TileDict:
    """One candidate: the schedule (block tile, thread tile, reduce step) plus what the cost
    model derived for it.  Attribute names are the reference's; ``wave_tile``, ``mfma`` and
    ``threads`` are filled on devices with matrix cores."""

    def __init__(self, block_tile: List[int], matmul_config: MatmulConfig, rstep: int) -> None:
        self.matmul_config = matmul_config
        # schedule
        self.block_tile = block_tile
        self.thread_tile: List[int] = []
        self.rstep = rstep
        self.wave_tile: List[int] = []
        self.mfma = 0
        self.threads = 0
        self.lds_row_pad = 0
        self.pipeline_depth = DEFAULT_PIPELINE_DEPTH
        self.stream_k = 0      # workgroups per core of a stream-K kernel; 0 = one workgroup per tile
        # analysis
        self.traffic = -1
        self.smem_cost = -1
        self.block_per_SM = -1
        self.num_wave = -1
        self.grid_size = -1
        self.valid = True

    def __hash__(self) -> int:
        return hash(tuple(self.block_tile + self.thread_tile))

    def __repr__(self) -> str:
        text = (
            f"TileDict(block_tile={self.block_tile}, thread_tile={self.thread_tile}, "
            f"rstep={self.rstep}, block traffic={_natural_size(self.traffic)}, "
            f"total traffic={_natural_size(self.traffic * self.grid_size)}, "
            f"smem_cost={_natural_size(self.smem_cost)}, block_per_SM={self.block_per_SM}, "
            f"num_wave={self.num_wave}, grid_size={self.grid_size}"
        )
        if self.wave_tile:
            text += f", wave_tile={self.wave_tile}, mfma={self.mfma}, threads={self.threads}"
        if self.stream_k:
            text += f", stream_k={self.stream_k}"
        return text + ")"

    def clone(self) -> "TileDict":
        twin = TileDict(list(self.block_tile), self.matmul_config, self.rstep)
        twin.__dict__.update(self.__dict__)
        twin.block_tile = list(self.block_tile)
        twin.thread_tile = list(self.thread_tile)
        twin.wave_tile = list(self.wave_tile)
        return twin

    def infer_smem_usage(self, rstep: Optional[int] = None) -> int:
        """Bytes of workgroup memory for one pipeline stage: an [m, rstep] and an [rstep, n] tile."""
        step = self.rstep if rstep is None else rstep
        cfg = self.matmul_config
        # The MFMA kernel keeps the [m, rstep] tile unpadded only on its direct-to-LDS path;
        # otherwise every row is padded to keep its 128-bit reads conflict-free (by how much depends
        # on the matrix instruction; before one is assigned, the 32x32x2 figure stands in).
        pad = 0
        if self.lds_row_pad and not loads_go_direct_to_lds(cfg, self.block_tile, step, self.pipeline_depth):
            pad = lds_row_pad(step, self.mfma or 32)
        return (step * sum(self.block_tile) + pad * self.block_tile[0]) * cfg.el_bytes

    @classmethod
    def from_block_tile(cls, block_tile: List[int], rstep: int, matmul_config: MatmulConfig,
                        arch: TileDevice, pipeline_depth: int = DEFAULT_PIPELINE_DEPTH) -> "TileDict":
        """Cost model of one block tile.  A tile that overflows workgroup memory or the register
        file comes back with ``valid = False`` and its analysis fields still at -1."""
        td = cls(block_tile, matmul_config, rstep)
        td.lds_row_pad = arch.lds_row_pad
        td.pipeline_depth = pipeline_depth

        td.smem_cost = td.infer_smem_usage()
        if td.smem_cost > arch.smem_cap:
            td.valid = False
            return td

        reg_usage = int(2 * math.prod(block_tile) * matmul_config.el_bytes / arch.reg_estimate_divisor)
        if reg_usage > arch.reg_cap:
            td.valid = False
            return td

        td.grid_size = math.prod(-(-full // tile) for tile, full in zip(block_tile, matmul_config.get_output_shape()))
        td.traffic = compute_memory_traffic(block_tile, matmul_config, arch)
        td.block_per_SM = min(
            arch.max_smem_usage // max(td.smem_cost, 1),
            arch.reg_cap // max(reg_usage, 1),
            arch.sm_partition,
        )
        resident = td.block_per_SM * arch.compute_max_core
        if resident <= 0:
            td.valid = False
            return td
        td.num_wave = -(-td.grid_size // resident)
        return td


def _similarity(a: float, b: float) -> float:
    """1 when a == b, falling towards 0 as the ratio a/b moves away from 1."""
    return (2 * a * b) / (a * a + b * b)


# MFMA blocks one wave may own: the kernel keeps one accumulator vector per block in an array that
# the compiler holds in registers only up to this many (128x128 with the 16x16x4 shape, 64 blocks,
# ends up in scratch memory and runs 50x slower)
MAX_BLOCKS_PER_WAVE = 32


def split_block_over_waves(block_tile: List[int], waves: int, rstep: int, arch: TileDevice, shapes=None):
    """Wave tile ``[wm, wn]`` and MFMA size for a block tile computed by ``waves`` wavefronts,
    or None.  A wave tile must be a grid of MFMA blocks (any column count: the kernel reads the
    second operand with the widest of 128-, 64- and 32-bit loads that divides it), the reduce
    step must hold whole 128-bit fragment reads (4 * wave / mi elements of k), and a wave owns at
    most ``MAX_BLOCKS_PER_WAVE`` blocks.  The larger instruction is preferred;
    among its wave tiles the most square wins, wider before taller."""
    m, n = block_tile
    for shape in (arch.mfma_shapes if shapes is None else shapes):
        mi = shape[0]
        if rstep % (4 * arch.warp_size // mi):
            continue
        best = None
        for rows in get_all_factors(waves):
            cols = waves // rows
            if m % rows or n % cols:
                continue
            wm, wn = m // rows, n // cols
            if wm % mi or wn % mi:
                continue
            if (wm // mi) * (wn // mi) > MAX_BLOCKS_PER_WAVE:
                continue
            key = (wm + wn, -wn)
            if best is None or key < best[0]:
                best = (key, [wm, wn])
        if best is not None:
            return best[1], mi
    return None


class Policy:
    """Roller's default policy: small memory traffic per block, few waves of blocks."""

    # tile sizes offered in addition to the exact divisors of a dimension
    SIMT_LADDER = (2, 4, 8, 16, 32)
    MFMA_LADDER = (16, 32, 48, 64, 96, 128, 160, 192, 256, 320, 384, 512)
    # registers per lane the MFMA kernel needs besides its accumulators and operand fragments:
    # addresses, loop state, buffer resources (measured: 40-60)
    REG_OVERHEAD = 50
    # ... and what the kernel for dword-aligned rows (K or N not a multiple of 4) needs on top:
    # exact buffer ranges, three extents of predicates (measured: 40 on whole tiles, 60 as stream-K)
    DWORD_ROWS_REGS = 60

    def __init__(self, config: MatmulConfig, arch: TileDevice,
                 pipeline_depth: int = DEFAULT_PIPELINE_DEPTH) -> None:
        self.arch = arch
        self.matmul_config = config
        # depth the kernels will be built at: decides whether the LDS tiles are padded and
        # whether loads are staged through registers (both cost model inputs on MI355X)
        self.pipeline_depth = pipeline_depth

    # ---- device-model helpers -------------------------------------------------------------

    @property
    def _granule(self) -> int:
        """Smallest m/n extent of a matrix instruction (0 on SIMT devices)."""
        shapes = self.arch.mfma_shapes
        return min(s[0] for s in shapes) if shapes else 0

    @property
    def _k_granule(self) -> int:
        """K extent that one 128-bit fragment read feeds on the smallest-k instruction's wave
        layout: 4 * (wave / m) for every shape, i.e. 8 for 32x32x2 and 16 for 16x16x4."""
        shapes = self.arch.mfma_shapes
        return max(4 * self.arch.warp_size // s[0] for s in shapes) if shapes else 0

    # ---- reduce step ------------------------------------------------------------------------

    def _coalesced_score(self, tile: List[int], rstep: int, mode: str = "sim") -> float:
        """Larger is better.  "sim": how close the contiguous run of each operand tile is to one
        read transaction (used to pick the base reduce step).  "raw": the summed run lengths
        (used when the reduce step is grown)."""
        tiles = MatmulConfig.propagate_inputs(tile, rstep)
        fulls = self.matmul_config.get_input_shapes()
        runs = [coalesced_factor(t.to_list(), f.to_list()) for t, f in zip(tiles, fulls)]
        if mode == "sim":
            rte = read_txn_elems(self.arch, self.matmul_config.el_bytes)
            return sum(_similarity(run, rte) for run in runs)
        return float(sum(runs))

    def get_reduce_step_candidates(self, rstep: int) -> List[int]:
        """Step sizes tried along a reduce axis of extent ``rstep``: its divisors (no remainder
        handling needed), or powers of two when it is a large prime.  With matrix cores only
        multiples of the instruction's k granule qualify and a ladder of such sizes is added,
        since the kernel predicates a ragged last step."""
        steps = get_all_factors(rstep)
        if len(steps) == 2 and rstep > 64:
            steps = [1]
            while steps[-1] * 2 < rstep:
                steps.append(steps[-1] * 2)
        kg = self._k_granule
        if kg:
            ladder = [s for s in (16, 32, 64, 128) if s % kg == 0]
            steps = sorted({s for s in steps if s % kg == 0} | set(ladder))
        return steps

    def _assign_reduce_step(self) -> int:
        steps = self.get_reduce_step_candidates(self.matmul_config.K)
        return max(steps, key=lambda s: self._coalesced_score([1, 1], s, "sim"))

    # ---- block tiles ------------------------------------------------------------------------

    def _priority(self, td: TileDict) -> float:
        """Smaller is better."""
        if self.arch.has_matrix_cores:
            return self.estimate_seconds(td)
        return (td.traffic + 1) * td.num_wave

    def simd_balance(self, block_tile: Sequence[int]) -> float:
        """Best share of a core's matrix pipes that a workgroup computing ``block_tile`` can keep
        busy: the tile splits into r x c wavefronts with r and c dividing its grid of (smallest)
        matrix-instruction blocks, and a wave count that is not a multiple of the SIMD count leaves
        pipes idle while the fullest SIMD finishes (48 x 16 is three blocks: three waves, one of
        four SIMDs idle)."""
        granule, simds = self._granule, self.arch.sm_partition
        if not granule:
            return 1.0
        rows, cols = block_tile[0] // granule, block_tile[1] // granule
        best = 0.0
        for r in get_all_factors(max(rows, 1)):
            for c in get_all_factors(max(cols, 1)):
                waves = r * c
                if waves * self.arch.warp_size <= 1024:
                    best = max(best, waves / (-(-waves // simds) * simds))
        return best or 1.0

    def estimate_seconds(self, td: TileDict, stream_k: Optional[int] = None) -> float:
        """Roofline estimate of the whole GEMM with block tile ``td`` on a device with matrix
        cores.  The busiest CU works through ceil(grid / CUs) tiles.  A tile costs the larger of
        its MFMA time at the CU's share of the matrix peak and its traffic at the CU's share of
        the memory bandwidth.  MFMA time is divided by an issue efficiency that falls with the
        operand traffic per FLOP, (1/m + 1/n); its two constants are fields of the device model,
        fitted to a committed sweep (``calibrate.py``).  A fixed cost per tile covers filling the
        pipeline and draining the accumulators; workgroups that are resident on a CU together
        (``block_per_SM``) hide it behind one another's MFMAs, so it is paid once per group of
        resident tiles.

        ``stream_k`` (default: the tile's own setting) estimates the stream-K kernel instead: every
        CU works grid / CUs tiles' worth of reduce steps, a fraction and not a whole number of
        rounds, at a slightly lower efficiency, with a fixed cost, and with the time the last workgroup
        of a tile needs to read the tile's pieces back (``stream_k_pieces`` of them at
        ``stream_k_piece_bandwidth``: what makes small tiles win where K is long and M x N small)."""
        a, cfg = self.arch, self.matmul_config
        m, n = td.block_tile
        stream_k = td.stream_k if stream_k is None else stream_k
        cu_flops = a.peak_matrix_tflops * 1e12 / a.compute_max_core
        cu_bw = a.bandwidth[0] * 1e9 / a.compute_max_core
        k_steps = -(-cfg.K // td.rstep)  # the kernel runs whole K steps also where K is ragged
        tiles_per_cu = -(-td.grid_size // a.compute_max_core)
        resident = max(1, min(td.block_per_SM, stream_k if stream_k else tiles_per_cu))
        base, slope = a.mfma_efficiency
        x = 1.0 / m + 1.0 / n
        efficiency = base - slope * x + (a.co_resident_gain if resident > 1 else 0.0)
        # below the knee (tiles smaller than about 64 x 128) a reduce step is too short to cover its own
        # barrier and round trips, and the efficiency leaves the line
        efficiency -= a.small_tile_slope * max(0.0, x - a.small_tile_knee)
        balance = self.simd_balance(td.block_tile)
        efficiency = max((efficiency - (a.stream_k_loss if stream_k else 0.0)) * balance, 0.05)
        t_mfma = 2.0 * m * n * k_steps * td.rstep / (cu_flops * efficiency)
        # a reduce step cannot be shorter than the round trip it hides (barrier, fragment reads, the
        # next loads' issue); workgroups that share the CU take turns in it.  Only tiles of a few MFMA
        # blocks get there.
        t_mfma = max(t_mfma, k_steps * a.step_latency_seconds / resident)
        # the tile's share of the operands has to come from device memory once; what the tiles read
        # again comes from the caches, at ``cache_bandwidth_ratio`` times that rate
        once = cfg.el_bytes * (cfg.M * cfg.K + cfg.K * cfg.N + cfg.M * cfg.N) / max(td.grid_size, 1)
        t_mem = (min(once, td.traffic) + max(td.traffic - once, 0.0) / a.cache_bandwidth_ratio) / cu_bw
        # filling the pipeline and draining the accumulators goes through the load and store ports of
        # the SIMDs that hold the tile's waves: a three-wave tile takes 4/3 of the time (measured on
        # 384 x 512 x 256: 48 x 16 tiles 4.4 us, 32 x 32 tiles 3.9 us)
        t_fixed = (a.tile_fixed_seconds + m * n * cfg.el_bytes / cu_bw) / balance
        if stream_k:
            share = td.grid_size / a.compute_max_core          # tiles' worth of reduce steps per CU
            t_pieces = self.stream_k_pieces(td, stream_k) * m * n * cfg.el_bytes / (a.stream_k_piece_bandwidth * 1e9)
            return share * max(t_mfma, t_mem) + (-(-math.ceil(share) // resident) + 1) * t_fixed + a.stream_k_fixed_seconds + t_pieces
        return tiles_per_cu * max(t_mfma, t_mem) + (-(-tiles_per_cu // resident)) * t_fixed

    def stream_k_pieces(self, td: TileDict, stream_k: int) -> float:
        """How many workgroups meet in one split tile of a stream-K launch.  The full rounds of the grid
        are worked as whole tiles (all but one of them, if fewer tiles than a quarter of the grid are
        left over) and the reduce steps of the remaining tiles are shared out: a share that is at least
        a tile long ends inside at most one tile, two pieces; with fewer reduce steps in a share than in
        a tile a tile has its steps / a share's steps pieces, plus one for the share that straddles its
        start; nothing is split if the grid divides the tile count.
        The workgroup that arrives last reads that many pieces of the tile back, one after the other,
        which is what a split costs."""
        k_steps = -(-self.matmul_config.K // td.rstep)
        tiles = td.grid_size
        grid = min(stream_k * self.arch.compute_max_core, tiles * k_steps)
        rounds = tiles // grid
        if rounds and tiles % grid and ((tiles % grid) * 4 < grid or (tiles % grid) * k_steps < grid):
            rounds -= 1
        units = (tiles - rounds * grid) * k_steps
        if not units:
            return 0.0
        share = units / grid
        return k_steps / share + 1.0 if share < k_steps else 2.0

    def _choose_stream_k(self, td: TileDict) -> None:
        """Sets ``td.stream_k`` where the estimate says that working equal shares of reduce steps
        beats whole tiles by more than the device model's margin (the kernels exist at pipeline
        depths with two workgroup-memory buffers and a register stage, i.e. from depth 2 on)."""
        a = self.arch
        td.stream_k = 0
        if not a.stream_k_workgroups or self.pipeline_depth < 2 or self.pipeline_depth > 3:
            return
        workgroups = max(1, min(a.stream_k_workgroups, td.block_per_SM))
        if self.estimate_seconds(td, workgroups) < self.estimate_seconds(td, 0) * (1.0 - a.stream_k_margin):
            td.stream_k = workgroups

    def _stream_k_fit(self, hint: TileDict, workgroups: int) -> int:
        """``workgroups`` per core of a stream-K kernel, cut down to what the register file holds once
        the wave tile is known (a stream-K grid of more workgroups than are resident runs in rounds
        again, with more pieces to add up)."""
        arch = self.arch
        if not workgroups or not hint.wave_tile or not arch.regs_per_lane:
            return workgroups
        acc_regs = int(math.prod(hint.wave_tile) // arch.warp_size * self.matmul_config.el_bytes / 4)
        regs = acc_regs + self._reg_overhead(hint, hint.wave_tile, hint.mfma, hint.threads)
        waves_per_simd = max(1, -(-(hint.threads // arch.warp_size) // arch.sm_partition))
        return max(1, min(workgroups, arch.regs_per_lane // (waves_per_simd * regs)))

    def get_block_tiles_candidates(self, init_tile: List[int], rstep: int) -> List[TileDict]:
        """All valid block tiles, best first (stable with respect to enumeration order:
        m outer, n inner, ascending)."""
        granule = self._granule
        ladder = self.MFMA_LADDER if granule else self.SIMT_LADDER
        steps = []
        for lower, extent in zip(init_tile, self.matmul_config.get_output_shape()):
            sizes = {f for f in get_all_factors(extent) if f >= lower}
            sizes |= {s for s in ladder if lower < s < extent}
            if granule:
                sizes = {s for s in sizes if s % granule == 0} or {granule}
            steps.append(sorted(sizes))

        tiles = []
        for m, n in itertools.product(*steps):
            td = TileDict.from_block_tile([m, n], rstep, self.matmul_config, self.arch, self.pipeline_depth)
            if td.valid:
                if granule:
                    self._choose_stream_k(td)
                tiles.append(td)
        return sorted(tiles, key=self._priority)

    def _expand_reduce_axis(self, td: TileDict) -> None:
        """Grows ``td.rstep`` to the multiple of the base step that gives the longest contiguous
        operand rows while one stage still fits the block's share of workgroup memory (the
        share among the blocks a core actually hosts, when matrix cores are modelled) -- or, on
        a device whose model says not to grow it, takes the shortest such step (among those that
        let the loads go straight to LDS, if any does).  Only ``rstep`` and ``smem_cost``
        change; occupancy figures keep their base-step values."""
        resident = td.block_per_SM
        if self.arch.has_matrix_cores:
            # a grid that does not fill the device leaves each core fewer blocks to host
            resident = max(1, min(resident, -(-td.grid_size // self.arch.compute_max_core)))
        limit = min(self.arch.max_smem_usage // resident, self.arch.smem_cap)
        steps = [
            s for s in self.get_reduce_step_candidates(self.matmul_config.K)
            if s % td.rstep == 0 and td.infer_smem_usage(s) <= limit
        ] or [td.rstep]
        if self.arch.has_matrix_cores:
            # a step that lets the loads go straight to LDS beats a longer one that does not
            direct = [s for s in steps if loads_go_direct_to_lds(self.matmul_config, td.block_tile, s, self.pipeline_depth)]
            steps = direct or steps
        if self.arch.grow_reduce_step:
            td.rstep = max(steps, key=lambda s: self._coalesced_score(td.block_tile, s, "raw"))
        else:
            td.rstep = min(steps)
        td.smem_cost = td.infer_smem_usage()

    # ---- threads per block --------------------------------------------------------------------

    def score_block_size(self, n: int):
        """(distance of the warp count from one warp per scheduler, fraction of idle lanes in
        the last warp); smaller is better.  On devices with matrix cores the imbalance between
        the SIMDs comes first."""
        warp, part = self.arch.warp_size, self.arch.sm_partition * self.arch.waves_per_partition
        warps = -(-n // warp)
        score = (max(warps / part, part / warps), (warps * warp - n) / n)
        if self.arch.has_matrix_cores:
            # a wave count that is not a multiple of the SIMD count leaves matrix pipes idle while
            # the fullest SIMD finishes (3 waves: one of four SIMDs idle; 5: one SIMD does double
            # duty): that imbalance ranks before the distance from the target
            simds = self.arch.sm_partition
            score = (-(-warps // simds) * simds / warps,) + score
        return score

    def recommend_block_size(self, td: TileDict) -> List[int]:
        """Thread counts worth trying for ``td``: divisors of the tile area up to 1024, best first."""
        sizes = [t for t in get_all_factors(math.prod(td.block_tile)) if t <= 1024]
        return sorted(sizes, key=self.score_block_size)

    def assign_thread_tile(self, td: TileDict, topk: int = 1) -> Iterator[TileDict]:
        """Yields completed copies of ``td`` for up to ``topk`` block sizes in recommended order.
        Without matrix cores the first block size that cannot be tiled ends the sequence (the
        reference's behaviour).  With matrix cores such a block size is skipped -- most thread
        counts are not a whole number of waves or do not split into MFMA blocks -- and a block
        size that works yields its wave tile with the matrix instruction the device model prefers
        for that size (``_assign_wave_tiles`` lists the alternatives)."""
        for block_size in self.recommend_block_size(td):
            if self.arch.has_matrix_cores:
                done = self._assign_wave_tiles(td, block_size)
                if not done:
                    continue
                yield done[0]
            else:
                one = self._assign_thread_tile(td, block_size)
                if one is None:
                    return
                yield one
            topk -= 1
            if topk == 0:
                return

    def _assign_thread_tile(self, td: TileDict, block_size: int) -> Optional[TileDict]:
        if self.arch.has_matrix_cores:
            done = self._assign_wave_tiles(td, block_size)
            return done[0] if done else None
        area = math.prod(td.block_tile) // block_size
        pairs = [[area // i, i] for i in range(1, math.isqrt(area) + 1) if area % i == 0]
        k, lds_bw = self.matmul_config.K, self.arch.bandwidth[1]
        # operand elements a thread reads per output tile: the most square tile reads least
        best = min(pairs, key=lambda p: sum(math.prod(s.to_list()) / lds_bw
                                            for s in MatmulConfig.propagate_inputs(p, k)))
        if int(math.prod(best) * self.matmul_config.el_bytes / 4) >= self.arch.thread_reg_limit:
            return None
        td.thread_tile = best
        return td.clone()

    def _reg_overhead(self, td: TileDict, wave_tile: Sequence[int], mi: int, block_size: int) -> int:
        """Registers per lane besides the accumulators.  The kernel keeps two sets of operand
        fragments (one 128-bit A value per row block and four B values per column block, i.e.
        ``4 * (blocks_m + blocks_n)`` registers a set); when its loads cannot go straight to LDS
        it also stages one K step of both operand tiles in registers."""
        blocks_m, blocks_n = wave_tile[0] // mi, wave_tile[1] // mi
        regs = self.REG_OVERHEAD + 2 * 4 * (blocks_m + blocks_n)
        if self.matmul_config.K % 4 or self.matmul_config.N % 4:
            regs += self.DWORD_ROWS_REGS
        if not loads_go_direct_to_lds(self.matmul_config, td.block_tile, td.rstep, self.pipeline_depth):
            regs += -(-(sum(td.block_tile) * td.rstep) // block_size)
        return regs

    def _assign_wave_tiles(self, td: TileDict, block_size: int) -> List[TileDict]:
        """The thread-tile step on a device with matrix cores: the block tile is split over
        ``block_size / wave`` wavefronts, once per matrix-instruction shape that admits a split
        (``split_block_over_waves``).  A split is dropped when its accumulators, plus room for
        operand fragments and staging, exceed the registers a lane can address at the number of
        waves this block puts on each SIMD."""
        arch = self.arch
        warp = arch.warp_size
        if block_size % warp:
            return []
        waves = block_size // warp
        lanes_side = math.isqrt(warp)  # 64 lanes seen as 8 x 8
        budget = arch.regs_per_lane // max(1, -(-waves // arch.sm_partition)) if arch.regs_per_lane else 0
        out: List[TileDict] = []
        for shape in arch.mfma_shapes:
            split = split_block_over_waves(td.block_tile, waves, td.rstep, arch, shapes=[shape])
            if split is None:
                continue
            wave_tile, mi = split
            if wave_tile[0] % lanes_side or wave_tile[1] % lanes_side:
                continue
            thread_tile = [wave_tile[0] // lanes_side, wave_tile[1] // lanes_side]
            acc_regs = int(math.prod(thread_tile) * self.matmul_config.el_bytes / 4)
            if acc_regs >= arch.thread_reg_limit:
                continue
            regs = acc_regs + self._reg_overhead(td, wave_tile, mi, block_size)
            if budget and regs > budget:
                continue
            done = td.clone()
            if budget and 2 * regs > budget and done.block_per_SM > 1:
                # more than half of the registers its waves can have: the workgroup runs alone on its core
                done.block_per_SM = 1
                done.num_wave = -(-done.grid_size // arch.compute_max_core)
            done.thread_tile = thread_tile
            done.wave_tile = wave_tile
            done.mfma = mi
            done.threads = block_size
            done.smem_cost = done.infer_smem_usage()   # the row padding follows the instruction
            if done.smem_cost > arch.smem_cap:
                continue
            td.thread_tile, td.wave_tile, td.mfma, td.threads = thread_tile, wave_tile, mi, block_size
            out.append(done)
        # The instruction with the longer k (16x16x4) moves half as many accumulator bytes per FLOP,
        # which leaves the register file free for LDS fragment reads; up to the wave-tile size the
        # device model names it is listed first.
        if len(out) > 1 and math.prod(out[0].wave_tile) <= arch.long_k_mfma_up_to:
            out.sort(key=lambda t: t.mfma)
        return out

    # ---- top level ------------------------------------------------------------------------------

    # a block tile whose plain and stream-K estimates are this close is emitted in both forms
    STREAM_K_TOSS_UP = 0.002

    def emit_config(self, topk: int = 10) -> List[TileDict]:
        """The first ``topk`` hints.  The reference completes every block tile with its first two
        block sizes (analyze.py:367-381).  With matrix cores the second block size of a tile is a
        near twin of the first (the fitted model: a second wave per SIMD changes nothing), so a
        tile yields one hint and the places go to more block tiles -- and to the other form of
        the kernel, whole tiles or stream-K, where the estimate cannot tell the two apart."""
        rstep = self._assign_reduce_step()
        hints: List[TileDict] = []
        late: List[Tuple[float, TileDict]] = []
        mfma = self.arch.has_matrix_cores
        for td in self.get_block_tiles_candidates([1, 1], rstep):
            self._expand_reduce_axis(td)
            # hints that lost their place when their wave tile was assigned (below) come back in
            # where their estimate puts them
            ranked = self._priority(td) if mfma else 0.0
            while late and late[0][0] <= ranked and len(hints) < topk:
                hints.append(late.pop(0)[1])
            if len(hints) >= topk:
                return hints[:topk]
            for hint in self.assign_thread_tile(td, 1 if mfma else 2):
                hint.stream_k = self._stream_k_fit(hint, hint.stream_k)
                if mfma and (hint.block_per_SM != td.block_per_SM or hint.stream_k != td.stream_k):
                    # the tile was ranked as if more of its workgroups shared a core than the registers
                    # of this wave tile allow: rank it again by what it is now expected to take
                    now = self.estimate_seconds(hint)
                    if now > ranked:
                        late.append((now, hint))
                        late.sort(key=lambda e: e[0])
                        continue
                hints.append(hint)
                if mfma and self.arch.stream_k_workgroups and 2 <= self.pipeline_depth <= 3:
                    other = self._stream_k_fit(hint, max(1, min(self.arch.stream_k_workgroups, hint.block_per_SM))) if not hint.stream_k else 0
                    mine, its = self.estimate_seconds(hint), self.estimate_seconds(hint, other)
                    if its < mine * (1.0 + self.STREAM_K_TOSS_UP) and len(hints) < topk:
                        twin = hint.clone()
                        twin.stream_k = other
                        hints.append(twin)
                if len(hints) >= topk:
                    return hints[:topk]
        return (hints + [hint for _, hint in late])[:topk]


def get_roller_hints(matmul_config: MatmulConfig, arch: TileDevice, topk: int = 10,
                     pipeline_depth: int = DEFAULT_PIPELINE_DEPTH) -> List[TileDict]:
    """Top-``topk`` tile configurations for ``matmul_config`` on ``arch``, best first.
    ``pipeline_depth`` (not in the reference's signature) is the depth the kernels will be
    compiled at; it only matters on device models with matrix cores."""
    return Policy(matmul_config, arch, pipeline_depth).emit_config(topk)
