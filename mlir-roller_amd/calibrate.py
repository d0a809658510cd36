"""Calibration of the MI355X ranking model against measurements.

    python -m mlir_roller_amd.calibrate measure [--out FILE] [--topk 48] [--shapes M0 M10 1024x1024x1024 ...]
    python -m mlir_roller_amd.calibrate fit     [--data FILE]
    python -m mlir_roller_amd.calibrate check   [--data FILE] [--topk 4]

The reference ranks block tiles by ``(traffic + 1) * num_wave`` and then simply tries its first
twenty (/root/reference/src/analyze.py:241-255, benchmark.py:10).  Here the ranking is a roofline
estimate (``Policy.estimate_seconds``) whose constants live in ``arch.MI355X`` and are fitted to a
sweep of the kernel on the device, so that few hints have to be tried:

``measure``  (needs the GPU) times, for every shape, the kernels of the policy's first ``topk``
             hints and writes one record per (shape, kernel) -- the data set committed under
             ``calibration/``;
``fit``      (no GPU) refits the constants from such a data set: per (shape, block tile) the best
             measured time gives an observed MFMA issue efficiency, and ordinary least squares of
             that efficiency against ``1/m + 1/n`` gives ``mfma_efficiency = (base, slope)``;
``check``    (no GPU) replays the policy on the data set: where does the measured best sit in the
             policy's order, and how far from it is the best of the first ``topk`` hints.

A CPU test refits the committed data set and compares the result with the committed constants,
so the two cannot drift apart.
"""

from __future__ import annotations

import argparse
import json
import math
import sys
from pathlib import Path
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

from .analyze import DEFAULT_PIPELINE_DEPTH, MatmulConfig, Policy, TileDict, get_roller_hints
from .arch import MI355X, TileDevice

DATA_DIR = Path(__file__).resolve().parent / "calibration"
DEFAULT_DATA = DATA_DIR / "mi355x_f32.json"

# the fourteen benchmark shapes, the ragged named configuration and three mid-size cubes ...
SHAPES: Dict[str, Tuple[int, int, int]] = {f"M{i}": s for i, s in enumerate([
    (2048, 2048, 2048), (2048, 2048, 8192), (2048, 4096, 2048), (2048, 4096, 4096), (2048, 8192, 2048),
    (2048, 8192, 4096), (2048, 8192, 8192), (4096, 2048, 2048), (4096, 4096, 8192), (4096, 8192, 2048),
    (4096, 8192, 4096), (8192, 2048, 8192), (8192, 4096, 2048), (8192, 4096, 4096)])}
SHAPES.update({"cfg4": (3000, 5000, 1536), "1024x1024x1024": (1024, 1024, 1024),
               "1536x1536x1536": (1536, 1536, 1536), "1000x1000x1000": (1000, 1000, 1000)})
# ... small cubes, tall, wide and skinny problems, and two whose tile grids fill a fraction of their last round
SHAPES.update({name: tuple(int(v) for v in name.split("x")) for name in (
    "256x256x256", "512x512x512", "768x768x768", "65536x128x128", "2560x2560x2560", "1920x2880x2048",
    "384x512x256", "4096x64x4096", "64x4096x4096")})


SETTLE_MS = 15.0   # run-up of every kernel ahead of its timed launches (the clocks follow the load, see tuner.time_candidates)
MIN_FIT_MS = 0.1   # shortest measurement the efficiency fit uses
MIN_FIT_TILE = 64 * 128  # smallest block tile it uses: below, a reduce step is too short to hide its own round trips
                         # and the efficiency falls away from the line (64 x 64: 0.90, 32 x 64: 0.87 where the line says 0.96)
LEADERS = 1.03     # ... and how close to its shape's fastest kernel a record has to be
WAVES_TIE = 0.005        # block sizes whose mean times differ by less are a tie
INSTRUCTION_TIE = 0.002  # so are the two matrix instructions on a wave-tile size


def shape_of(name: str) -> Tuple[int, int, int]:
    if name in SHAPES:
        return SHAPES[name]
    dims = tuple(int(v) for v in name.lower().split("x"))
    if len(dims) != 3 or min(dims) <= 0:
        raise ValueError(f"unknown shape {name!r}")
    return dims  # type: ignore[return-value]


# ---------------------------------------------------------------------------------------------
# the model, restated on plain numbers so that a fit can evaluate it without building TileDicts
# ---------------------------------------------------------------------------------------------

def ideal_tile_seconds(m: int, n: int, K: int, rstep: int, arch: TileDevice) -> float:
    """MFMA time of one block tile over the whole of K at a CU's share of the matrix peak."""
    k_steps = -(-K // rstep)
    return 2.0 * m * n * k_steps * rstep / (arch.peak_matrix_tflops * 1e12 / arch.compute_max_core)


def fixed_tile_seconds(m: int, n: int, arch: TileDevice, el_bytes: int = 4) -> float:
    """The part of a tile's time that does not scale with K (pipeline fill, storing C)."""
    return arch.tile_fixed_seconds + m * n * el_bytes / (arch.bandwidth[0] * 1e9 / arch.compute_max_core)


def resident_tiles(rec: dict, arch: TileDevice, depth: int = DEFAULT_PIPELINE_DEPTH) -> int:
    """Workgroups of this record's block tile that the policy's LDS and register model puts on
    one CU at a time."""
    td = TileDict.from_block_tile(list(rec["block_tile"]), rec["rstep"], MatmulConfig(*rec["shape"], 32), arch, depth)
    return max(1, td.block_per_SM)


def observed_efficiency(rec: dict, arch: TileDevice) -> Optional[float]:
    """MFMA issue efficiency that one measurement implies under the model's structure:
    tiles_per_cu * ideal / efficiency + ceil(tiles_per_cu / resident) * fixed = measured."""
    M, N, K = rec["shape"]
    m, n = rec["block_tile"]
    tiles = (-(-M // m)) * (-(-N // n))
    per_cu = -(-tiles // arch.compute_max_core)
    rounds = -(-per_cu // min(resident_tiles(rec, arch), per_cu))
    busy = (rec["ms"] * 1e-3 - rounds * fixed_tile_seconds(m, n, arch)) / per_cu
    if busy <= 0:
        return None
    return ideal_tile_seconds(m, n, K, rec["rstep"], arch) / busy


def plain(records: Iterable[dict]) -> List[dict]:
    """The records of kernels that take one tile per workgroup (the tile-level fits are about those)."""
    return [r for r in records if not r.get("stream_k")]


def best_per_block_tile(records: Iterable[dict]) -> List[dict]:
    """The fastest record of every (shape, block tile): wave split, instruction and K step are
    second-order choices that the fit of the tile-level efficiency must not see."""
    best: Dict[tuple, dict] = {}
    for r in plain(records):
        key = (tuple(r["shape"]), tuple(r["block_tile"]))
        if key not in best or r["ms"] < best[key]["ms"]:
            best[key] = r
    return [best[k] for k in sorted(best)]


def _solve(a: List[List[float]], b: List[float]) -> List[float]:
    """Gaussian elimination with partial pivoting for the small normal equations of ``fit``."""
    n = len(b)
    m = [row[:] + [rhs] for row, rhs in zip(a, b)]
    for col in range(n):
        piv = max(range(col, n), key=lambda r: abs(m[r][col]))
        if abs(m[piv][col]) < 1e-18:
            raise ValueError("the records do not pin the model (singular normal equations)")
        m[col], m[piv] = m[piv], m[col]
        for r in range(col + 1, n):
            f = m[r][col] / m[col][col]
            for c in range(col, n + 1):
                m[r][c] -= f * m[col][c]
    x = [0.0] * n
    for r in range(n - 1, -1, -1):
        x[r] = (m[r][n] - math.fsum(m[r][c] * x[c] for c in range(r + 1, n))) / m[r][r]
    return x


def fit(records: Sequence[dict], arch: Optional[TileDevice] = None) -> dict:
    """Least-squares ``efficiency = base - slope * (1/m + 1/n) + gain * [tiles share a CU]`` over
    the best record of every (shape, block tile) whose tile grid fills at least three quarters of
    its last round of CUs (a sparse last round measures the tail, not the tile), that ran for at
    least ``MIN_FIT_MS`` (below that the launch itself is a visible share), whose tile has at least
    ``MIN_FIT_TILE`` elements, and that came within ``LEADERS`` of its shape's fastest kernel: the model
    is asked to order the leaders of a shape, and how far behind an also-ran finishes (a 64 x 128 tile
    on 8192 x 4096 x 4096 loses 4 % to cache misses that 1/m + 1/n does not describe) must not bend the
    line -- nor should the fit depend on which also-rans a sweep happened to time.  The gain is fitted
    only when the records hold tiles of both kinds.  Deterministic: closed-form normal equations,
    records in sorted order."""
    arch = arch or MI355X()
    fastest: Dict[tuple, float] = {}
    for r in plain(records):
        fastest[tuple(r["shape"])] = min(fastest.get(tuple(r["shape"]), float("inf")), r["ms"])
    xs, ys, zs = [], [], []
    for r in best_per_block_tile(records):
        M, N, _ = r["shape"]
        m, n = r["block_tile"]
        if r["ms"] > LEADERS * fastest[tuple(r["shape"])]:
            continue
        tiles = (-(-M // m)) * (-(-N // n))
        last_round = tiles % arch.compute_max_core or arch.compute_max_core
        if M % m or N % n or last_round < 0.75 * arch.compute_max_core or r["ms"] < MIN_FIT_MS or m * n < MIN_FIT_TILE:
            continue
        eff = observed_efficiency(r, arch)
        if eff is None or not 0.3 < eff < 1.05:
            continue
        xs.append(1.0 / m + 1.0 / n)
        ys.append(eff)
        zs.append(1.0 if min(resident_tiles(r, arch), -(-tiles // arch.compute_max_core)) > 1 else 0.0)
    if len(set(xs)) < 3:
        raise ValueError(f"only {len(set(xs))} usable block-tile sizes; need at least 3")
    with_gain = 0.0 < math.fsum(zs) < len(zs)
    cols = [[1.0] * len(xs), xs] + ([zs] if with_gain else [])
    normal = [[math.fsum(p * q for p, q in zip(ci, cj)) for cj in cols] for ci in cols]
    rhs = [math.fsum(p * y for p, y in zip(ci, ys)) for ci in cols]
    sol = _solve(normal, rhs)
    base, slope, gain = sol[0], -sol[1], (sol[2] if with_gain else 0.0)
    resid = [y - (base - slope * x + gain * z) for x, y, z in zip(xs, ys, zs)]
    return {"mfma_efficiency": (round(base, 3), round(slope, 2)), "co_resident_gain": round(gain, 3), "base": base,
            "slope": slope, "gain": gain, "points": len(xs),
            "rms_residual": math.sqrt(math.fsum(e * e for e in resid) / len(xs))}


def fit_small_tiles(records: Sequence[dict], arch: Optional[TileDevice] = None) -> dict:
    """How fast the efficiency leaves the line below the knee (``small_tile_slope``): over the best
    record of every (shape, block tile) beyond ``arch.small_tile_knee`` that fills its last round and
    ran for at least ``MIN_FIT_MS`` -- leaders or not: small tiles never lead where a kernel runs that
    long -- a least-squares line through the knee of (line - observed efficiency) against
    (1/m + 1/n - knee).  The line is the one ``fit`` gives for the same records."""
    arch = arch or MI355X()
    line = fit(records, arch)
    xx = xy = 0.0
    points = 0
    for r in best_per_block_tile(records):
        M, N, _ = r["shape"]
        m, n = r["block_tile"]
        x = 1.0 / m + 1.0 / n
        tiles = (-(-M // m)) * (-(-N // n))
        last_round = tiles % arch.compute_max_core or arch.compute_max_core
        if x <= arch.small_tile_knee or M % m or N % n or last_round < 0.75 * arch.compute_max_core or r["ms"] < MIN_FIT_MS:
            continue
        eff = observed_efficiency(r, arch)
        if eff is None or not 0.3 < eff < 1.05:
            continue
        together = min(resident_tiles(r, arch), -(-tiles // arch.compute_max_core)) > 1
        expected = line["base"] - line["slope"] * x + (line["gain"] if together else 0.0)
        dx = x - arch.small_tile_knee
        xx += dx * dx
        xy += dx * (expected - eff)
        points += 1
    if points < 5:
        raise ValueError(f"only {points} block tiles below the knee; need at least 5")
    return {"small_tile_slope": round(max(xy / xx, 0.0), 1), "points": points}


def _geo_mean(ratios: Sequence[float]) -> float:
    return math.exp(math.fsum(math.log(r) for r in ratios) / len(ratios))


def fit_waves_per_simd(records: Sequence[dict], arch: Optional[TileDevice] = None, min_tile: int = 128 * 128) -> dict:
    """Which block size the recommendation should try first: for every (shape, block tile) of at
    least ``min_tile`` elements measured both with one and with two waves per SIMD, the ratio of
    the two best times; the geometric mean over all pairs decides (``waves_per_partition``): two
    waves only where they win by more than ``WAVES_TIE`` -- within that, a coin that re-measuring
    would flip, the smaller block (larger wave tiles, fewer operand reads per FLOP) stays first."""
    arch = arch or MI355X()
    one, two = arch.warp_size * arch.sm_partition, 2 * arch.warp_size * arch.sm_partition
    best: Dict[tuple, Dict[int, float]] = {}
    for r in plain(records):
        if math.prod(r["block_tile"]) < min_tile or r["threads"] not in (one, two):
            continue
        slot = best.setdefault((tuple(r["shape"]), tuple(r["block_tile"])), {})
        slot[r["threads"]] = min(slot.get(r["threads"], float("inf")), r["ms"])
    ratios = [t[two] / t[one] for _, t in sorted(best.items()) if one in t and two in t]
    if not ratios:
        raise ValueError("no block tile was measured at both block sizes")
    mean = _geo_mean(ratios)
    return {"waves_per_partition": 1 if mean >= 1.0 - WAVES_TIE else 2, "two_over_one": mean, "pairs": len(ratios)}


def fit_long_k_mfma(records: Sequence[dict], arch: Optional[TileDevice] = None) -> dict:
    """Up to which wave-tile size the instruction with the longer k (16x16x4) should be listed
    first: for every wave-tile size, the geometric mean of time(32x32x2) / time(16x16x4) over the
    (shape, block tile, wave tile) triples measured with both; the largest size whose mean is
    above ``1 - INSTRUCTION_TIE``, with every smaller size above it as well (``long_k_mfma_up_to``;
    a tie keeps the instruction that wins on the smaller wave tiles)."""
    by: Dict[tuple, Dict[int, float]] = {}
    for r in plain(records):
        key = (tuple(r["shape"]), tuple(r["block_tile"]), tuple(r["wave_tile"]))
        slot = by.setdefault(key, {})
        slot[r["mfma"]] = min(slot.get(r["mfma"], float("inf")), r["ms"])
    per_size: Dict[int, List[float]] = {}
    for (_, _, wave_tile), t in sorted(by.items()):
        if 16 in t and 32 in t:
            per_size.setdefault(math.prod(wave_tile), []).append(t[32] / t[16])
    means = {size: _geo_mean(v) for size, v in sorted(per_size.items())}
    up_to = 0
    for size, mean in means.items():
        if mean <= 1.0 - INSTRUCTION_TIE:
            break
        up_to = size
    return {"long_k_mfma_up_to": up_to, "mi32_over_mi16_by_wave_tile_elems": {k: round(v, 4) for k, v in means.items()},
            "pairs": sum(len(v) for v in per_size.values())}


def fit_stream_k(records: Sequence[dict], arch: Optional[TileDevice] = None, min_ms: float = 0.25) -> dict:
    """What the stream-K form of a kernel costs where it has nothing to gain: over every kernel
    measured in both forms on a problem whose tile grid fills whole rounds of CUs, that runs for
    at least ``min_ms`` and whose tile has at least ``MIN_FIT_TILE`` elements (smaller tiles pay the
    walk from segment to segment more often, and how many of them a sweep holds should not move the
    figure), the geometric mean of time(stream-K) / time(plain), minus one
    (``stream_k_loss``).  Per shape, the best plain time over the best stream-K time is listed for the
    record (above 1: a stream-K kernel is the fastest one measured)."""
    arch = arch or MI355X()
    by: Dict[tuple, Dict[int, float]] = {}
    for r in records:
        key = (tuple(r["shape"]), tuple(r["block_tile"]), tuple(r["wave_tile"]), r["mfma"], r["rstep"])
        form = 1 if r.get("stream_k") else 0
        slot = by.setdefault(key, {})
        slot[form] = min(slot.get(form, float("inf")), r["ms"])
    whole = []
    best: Dict[tuple, Dict[int, float]] = {}
    for (shape, tile, _, _, _), t in sorted(by.items()):
        for form, ms in t.items():
            slot = best.setdefault(shape, {})
            slot[form] = min(slot.get(form, float("inf")), ms)
        tiles = (-(-shape[0] // tile[0])) * (-(-shape[1] // tile[1]))
        if 0 in t and 1 in t and tiles % arch.compute_max_core == 0 and t[0] >= min_ms and tile[0] * tile[1] >= MIN_FIT_TILE:
            whole.append(t[1] / t[0])
    if not whole:
        raise ValueError("no kernel was measured in both forms on a problem that fills whole rounds")
    gains = {"x".join(str(v) for v in shape): round(t[0] / t[1], 4) for shape, t in sorted(best.items()) if 0 in t and 1 in t}
    return {"stream_k_loss": round(_geo_mean(whole) - 1.0, 3), "pairs": len(whole), "best_plain_over_best_stream_k": gains}


def fit_stream_k_pieces(records: Sequence[dict], arch: Optional[TileDevice] = None, min_pieces: float = 6.0,
                        depth: int = DEFAULT_PIPELINE_DEPTH) -> dict:
    """The rate at which the last workgroup of a split tile gets the tile's pieces back
    (``stream_k_piece_bandwidth``, GB/s): over the stream-K kernels whose tiles are split
    ``min_pieces`` ways or more -- long K, few tiles -- a least-squares line through the origin of
    (measured time - the estimate without that term) against the bytes of pieces read per tile."""
    import dataclasses

    arch = arch or MI355X()
    free = dataclasses.replace(arch, stream_k_piece_bandwidth=1.0e12)   # the term switched off
    xx = xy = 0.0
    points = 0
    for r in records:
        if not r.get("stream_k"):
            continue
        cfg = MatmulConfig(*r["shape"], 32)
        policy = Policy(cfg, free, depth)
        td = TileDict.from_block_tile(list(r["block_tile"]), r["rstep"], cfg, free, depth)
        pieces = policy.stream_k_pieces(td, r["stream_k"])
        if pieces < min_pieces:
            continue
        x = pieces * r["block_tile"][0] * r["block_tile"][1] * cfg.el_bytes
        y = r["ms"] * 1e-3 - policy.estimate_seconds(td, r["stream_k"])
        xx += x * x
        xy += x * y
        points += 1
    if points < 8 or xy <= 0.0:
        raise ValueError("too few heavily split stream-K kernels in the data to fit the piece bandwidth")
    return {"stream_k_piece_bandwidth": float(f"{xx / xy / 1e9:.2g}"), "points": points}


# ---------------------------------------------------------------------------------------------
# replaying the policy on a data set
# ---------------------------------------------------------------------------------------------

def _key_of_hint(hint: TileDict) -> tuple:
    return (tuple(hint.block_tile), tuple(hint.wave_tile), hint.mfma, hint.rstep, 1 if hint.stream_k else 0)


def _key_of_record(rec: dict) -> tuple:
    return (tuple(rec["block_tile"]), tuple(rec["wave_tile"]), rec["mfma"], rec["rstep"], 1 if rec.get("stream_k") else 0)


def check(records: Sequence[dict], arch: Optional[TileDevice] = None, topk: int = 4, depth: int = DEFAULT_PIPELINE_DEPTH) -> List[dict]:
    """Per shape of the data set: rank (in the policy's current order) of the fastest measured
    kernel, time of the first hint over the fastest, time of the best of the first ``topk`` hints
    over the fastest, and how many of those first hints the data set has no measurement for."""
    arch = arch or MI355X()
    by_shape: Dict[tuple, Dict[tuple, float]] = {}
    for r in records:
        by_shape.setdefault(tuple(r["shape"]), {})[_key_of_record(r)] = r["ms"]
    rows = []
    for shape in sorted(by_shape):
        measured = by_shape[shape]
        hints = get_roller_hints(MatmulConfig(*shape, 32), arch, topk=200, pipeline_depth=depth)
        order = [_key_of_hint(h) for h in hints]
        fastest_key = min(measured, key=measured.get)
        fastest = measured[fastest_key]
        head = [measured.get(k) for k in order[:topk]]
        known = [t for t in head if t is not None]
        rows.append({
            "shape": list(shape),
            "fastest_ms": fastest,
            "fastest_rank": order.index(fastest_key) + 1 if fastest_key in order else None,
            "top1_over_fastest": (head[0] / fastest) if head and head[0] is not None else None,
            "topk_over_fastest": (min(known) / fastest) if known else None,
            "unmeasured_in_topk": sum(t is None for t in head),
        })
    return rows


# ---------------------------------------------------------------------------------------------
# measuring (GPU)
# ---------------------------------------------------------------------------------------------

def candidate_hints(cfg: MatmulConfig, arch: TileDevice, topk: int, depth: int = DEFAULT_PIPELINE_DEPTH) -> List[TileDict]:
    """What a calibration run times for one problem: the policy's block tiles in its current order
    and, for each, the first two block sizes that split into wave tiles with EVERY matrix
    instruction that fits -- also the alternatives the policy itself would not emit, because the
    fits of the wave and instruction preferences need both sides of each comparison."""
    policy = Policy(cfg, arch, depth)
    out: List[TileDict] = []
    for td in policy.get_block_tiles_candidates([1, 1], policy._assign_reduce_step()):
        policy._expand_reduce_axis(td)
        sizes = 0
        for block_size in policy.recommend_block_size(td):
            done = policy._assign_wave_tiles(td, block_size)
            if not done:
                continue
            for hint in done:
                # both forms of every kernel, whole tiles and stream-K, whatever the estimate prefers
                for form in ((0, max(1, min(arch.stream_k_workgroups, hint.block_per_SM))) if arch.stream_k_workgroups and 2 <= depth <= 3 else (0,)):
                    twin = hint.clone()
                    twin.stream_k = form
                    out.append(twin)
            sizes += 1
            if sizes == 2:
                break
        if len(out) >= topk:
            break
    return out[:topk]


def measure(shape_names: Sequence[str], topk: int, depth: int = DEFAULT_PIPELINE_DEPTH, chunk: int = 8,
            say=lambda *a: print(*a, file=sys.stderr, flush=True)) -> dict:
    import numpy as np

    from . import hip
    from .hip import DeviceArray, GemmPlan, Stream
    from .roller import hint_to_gemm_config, make_inputs
    from .tuner import time_candidates

    hip.init(0)
    props = hip.device_info()
    arch = MI355X.from_device(props)
    stream = Stream()
    records: List[dict] = []
    for name in shape_names:
        shape = shape_of(name)
        M, N, K = shape
        cfg = MatmulConfig(M, N, K, 32)
        A, B = make_inputs(cfg, 0, "uniform")
        bufs = (DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray.zeros((M, N)))
        del A, B
        cands = []
        for rank, hint in enumerate(candidate_hints(cfg, arch, topk, depth), 1):
            try:
                g = hint_to_gemm_config(cfg, hint, depth)
                cands.append((rank, hint, g, GemmPlan(g)))
            except Exception as e:  # a hint the device refuses is simply not part of the data
                say(f"[calibrate] {name} hint {rank} skipped: {e}")
        for i in range(0, len(cands), chunk):
            part = cands[i:i + chunk]
            times = time_candidates([c[3] for c in part], bufs, shape, stream=stream, settle_ms=SETTLE_MS)
            for (rank, hint, g, _), ms in zip(part, times):
                records.append({"shape": list(shape), "block_tile": list(hint.block_tile), "wave_tile": list(hint.wave_tile),
                                "mfma": hint.mfma, "rstep": hint.rstep, "threads": hint.threads, "edge": g.edge,
                                "direct": g.direct, "stream_k": g.streamk, "rank_when_measured": rank, "ms": round(ms, 6)})
        best = min((r for r in records if r["shape"] == list(shape)), key=lambda r: r["ms"])
        say(f"[calibrate] {name} {shape}: {len(cands)} kernels, best {best['ms']:.4f} ms "
            f"({2.0 * M * N * K / best['ms'] / 1e9:.1f} TFLOP/s) rank {best['rank_when_measured']} {best['block_tile']}/{best['wave_tile']}/mi{best['mfma']}/k{best['rstep']}")
        for b in bufs:
            b.free()
    return {"device": {"name": props.name.decode(), "arch": props.arch.decode(), "compute_units": props.compute_units,
                       "clock_khz": props.clock_khz},
            "pipeline_depth": depth, "protocol": "per kernel: best of 2 alternating batches of 8 launches, each behind 15 ms of the same kernel, behind a 40 ms clock ramp; HIP events on the launch stream",
            "records": records}


def merge(data: dict, earlier: dict) -> dict:
    """Two sessions of the same sweep as one data set: the union of their kernels, each with the
    shortest time either session measured for it."""
    def key(r: dict) -> tuple:
        return (tuple(r["shape"]), tuple(r["block_tile"]), tuple(r["wave_tile"]), r["mfma"], r["rstep"], r["threads"], r.get("stream_k", 0))
    best = {key(r): r for r in earlier["records"]}
    for r in data["records"]:
        if key(r) not in best or r["ms"] < best[key(r)]["ms"]:
            best[key(r)] = r
    out = dict(data)
    out["records"] = sorted(best.values(), key=lambda r: (list(SHAPES.values()).index(tuple(r["shape"])) if tuple(r["shape"]) in SHAPES.values() else len(SHAPES),
                                                          r["shape"], r["rank_when_measured"], r["block_tile"], r["wave_tile"], r["mfma"], r.get("stream_k", 0)))
    out["sessions"] = data.get("sessions", 1) + earlier.get("sessions", 1)
    return out


def load(path: Path = DEFAULT_DATA) -> dict:
    return json.loads(Path(path).read_text())


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="fit / check the MI355X ranking model of the rTile policy")
    sub = ap.add_subparsers(dest="cmd", required=True)
    m = sub.add_parser("measure")
    m.add_argument("--out", default=str(DEFAULT_DATA))
    m.add_argument("--topk", type=int, default=96, help="kernels per shape, both forms (whole tiles and stream-K) counted")
    m.add_argument("--shapes", nargs="*", default=list(SHAPES))
    m.add_argument("--merge", nargs="*", default=[], help="earlier data sets of the same sweep: per kernel the shortest time of all "
                   "sessions is kept (a session's slow outliers -- a busy neighbour, a cold cache -- drop out)")
    pc = sub.add_parser("precompile", help="no GPU: fill the code-object cache with the kernels that `measure` will time")
    pc.add_argument("--topk", type=int, default=96)
    pc.add_argument("--shapes", nargs="*", default=list(SHAPES))
    f = sub.add_parser("fit")
    f.add_argument("--data", default=str(DEFAULT_DATA))
    c = sub.add_parser("check")
    c.add_argument("--data", default=str(DEFAULT_DATA))
    c.add_argument("--topk", type=int, default=4)
    args = ap.parse_args(argv)

    if args.cmd == "precompile":
        from . import hip
        from .roller import hint_to_gemm_config
        todo = []
        for name in args.shapes:
            cfg = MatmulConfig(*shape_of(name), 32)
            for hint in candidate_hints(cfg, MI355X(), args.topk):
                try:
                    g = hint_to_gemm_config(cfg, hint, DEFAULT_PIPELINE_DEPTH)
                    hip.config_check(g)
                    todo.append(g)
                except Exception:
                    pass
        failed = hip.precompile_many(todo)
        print(f"{len(set(todo))} kernels, {len(failed)} failed to compile")
        return 1 if failed else 0
    if args.cmd == "measure":
        earlier_sets = [load(Path(earlier)) for earlier in args.merge]   # (read first: a missing file should not cost a session)
        data = measure(args.shapes, args.topk)
        data["sessions"] = 1
        for earlier in earlier_sets:
            data = merge(data, earlier)
        out = Path(args.out)
        out.parent.mkdir(parents=True, exist_ok=True)
        out.write_text(json.dumps(data, separators=(",", ":")).replace('},{"shape"', '},\n{"shape"'))
        print(f"{len(data['records'])} records written to {out}")
        return 0
    data = load(Path(args.data))
    if args.cmd == "fit":
        res = fit(data["records"])
        now = MI355X()
        print(f"fitted mfma_efficiency = {res['mfma_efficiency']}, co_resident_gain = {res['co_resident_gain']} from {res['points']} "
              f"block tiles (rms residual {res['rms_residual']:.4f}); arch.MI355X has {tuple(now.mfma_efficiency)}, {now.co_resident_gain}")
        waves = fit_waves_per_simd(data["records"])
        print(f"fitted waves_per_partition = {waves['waves_per_partition']} (two waves per SIMD take {waves['two_over_one']:.4f} x "
              f"the time of one, {waves['pairs']} block tiles); arch.MI355X has {now.waves_per_partition}")
        try:
            sk = fit_stream_k(data["records"])
            print(f"fitted stream_k_loss = {sk['stream_k_loss']} ({sk['pairs']} kernels in both forms on whole rounds); arch.MI355X has "
                  f"{now.stream_k_loss}; best plain over best stream-K per shape: {sk['best_plain_over_best_stream_k']}")
        except ValueError as e:
            print(f"stream_k_loss not fitted: {e}")
        try:
            pc = fit_stream_k_pieces(data["records"])
            print(f"fitted stream_k_piece_bandwidth = {pc['stream_k_piece_bandwidth']} GB/s ({pc['points']} heavily split kernels); "
                  f"arch.MI355X has {now.stream_k_piece_bandwidth}")
        except ValueError as e:
            print(f"stream_k_piece_bandwidth not fitted: {e}")
        try:
            small = fit_small_tiles(data["records"])
            print(f"fitted small_tile_slope = {small['small_tile_slope']} ({small['points']} block tiles below the knee); arch.MI355X has {now.small_tile_slope}")
        except ValueError as e:
            print(f"small_tile_slope not fitted: {e}")
        instr = fit_long_k_mfma(data["records"])
        print(f"fitted long_k_mfma_up_to = {instr['long_k_mfma_up_to']} (32x32x2 over 16x16x4 by wave-tile elements: "
              f"{instr['mi32_over_mi16_by_wave_tile_elems']}); arch.MI355X has {now.long_k_mfma_up_to}")
        return 0
    rows = check(data["records"], topk=args.topk)
    for r in rows:
        fmt = lambda v: "-" if v is None else f"{v:.4f}"
        print(f"{'x'.join(map(str, r['shape'])):>18}  fastest rank {r['fastest_rank']!s:>4}  top1/fastest {fmt(r['top1_over_fastest'])}  "
              f"top{args.topk}/fastest {fmt(r['topk_over_fastest'])}  unmeasured {r['unmeasured_in_topk']}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
