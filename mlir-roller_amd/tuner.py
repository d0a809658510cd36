"""Picking one kernel among the policy's first hints by measurement.

The reference times every one of its top-20 hints and keeps the fastest
(/root/reference/src/benchmark.py:41-54).  On MI355X the calibrated policy puts near-equal
kernels at the head of its list (the first hint is within about half a percent of the measured
best on the benchmark shapes), so two things change:

* the **policy's order decides ties**: a later hint replaces an earlier one only when it is
  faster by more than the run-to-run spread of such a measurement (``TIE_MARGIN``); otherwise
  noise would pick a different "winner" on every run;
* few hints are tried (``DEFAULT_TOPK``), which keeps search + JIT + tuning short.

``choose`` is the rule itself (pure, no device); ``time_candidates`` measures loaded plans on a
stream with the engine-clock ramp queued ahead of the timed launches.
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

DEFAULT_TOPK = 4      # hints tried per shape (the reference: 20, benchmark.py:10)
TIE_MARGIN = 0.01     # relative spread of two timings of the same kernel: about half a percent a few milliseconds
                      # apart, up to three percent for small-tile kernels between one batch of launches and the next
PICK_SETTLE_MS = 2.0  # run-up of each candidate ahead of its timed launches when the tuner compares hints (a long
                      # list, as the reference's top-20, holds kernels of very different load)
RAMP_MS = 40.0        # continuous load queued ahead of a timed region: the engine clock drops within
                      # microseconds of the GPU going idle and needs about 25 ms to come back


def choose(timings: Sequence[Tuple[int, float]], margin: float = TIE_MARGIN) -> int:
    """Rank of the hint to keep.  ``timings`` holds ``(rank, milliseconds)`` pairs; ranks are
    the policy's order (1 = first hint).  Walking in that order, a hint displaces the incumbent
    only if it is faster by more than ``margin`` (relative).  Non-finite or non-positive times
    are ignored; with nothing usable the result is -1."""
    keep_rank, keep_ms = -1, float("inf")
    for rank, ms in sorted(timings, key=lambda t: t[0]):
        if not (ms == ms and 0.0 < ms < float("inf")):
            continue
        if keep_rank < 0 or ms < keep_ms * (1.0 - margin):
            keep_rank, keep_ms = rank, ms
    return keep_rank


def ramp_launches(shape: Tuple[int, int, int], at_least: int = 0) -> int:
    """Launches of a GEMM of ``shape`` that cover ``RAMP_MS`` at roughly 120 TFLOP/s."""
    M, N, K = shape
    est_ms = max(2.0 * M * N * K / 120e9, 1e-3)
    return max(at_least, int(RAMP_MS / est_ms) + 1)


def time_candidates(plans: Sequence, bufs, shape: Tuple[int, int, int], stream=None, reps: int = 8,
                    rounds: int = 2, gap_launches: int = 2, settle_ms: float = 0.0) -> List[float]:
    """Milliseconds per launch for each plan in ``plans`` (objects with ``launch(A, B, C, M, N, K,
    stream=)``), all measured behind ONE clock ramp and with no host synchronisation in between:
    a synchronisation (or the host loading the next module) between candidates would idle the
    GPU and put the next measurement into the ramp again.  Every candidate is timed ``rounds``
    times in alternation with the others and its best mean is returned, which takes slow drifts
    (temperature, clock) out of the comparison.

    ``settle_ms``: untimed launches of a candidate, worth that many milliseconds, ahead of each of its
    timed batches.  The clocks follow the load: after 20 ms of a kernel that keeps half of the SIMDs
    busy, a full-rate kernel ran 12 % slow and needed 14 ms to recover (measured), so a sweep that
    mixes good and poor kernels gives every candidate its own run-up; the policy's first hints are
    all full-rate kernels and need none."""
    from . import hip
    from .hip import Event

    if not plans:
        return []
    M, N, K = shape
    launch = lambda plan: plan.launch(bufs[0], bufs[1], bufs[2], M, N, K, stream=stream)
    for _ in range(ramp_launches(shape)):
        launch(plans[0])
    run_up = max(gap_launches, math.ceil(ramp_launches(shape) * settle_ms / RAMP_MS)) if settle_ms > 0 else gap_launches
    marks = []
    for _ in range(max(rounds, 1)):
        for i, plan in enumerate(plans):
            for _ in range(run_up):
                launch(plan)
            e0, e1 = Event(), Event()
            e0.record(stream)
            for _ in range(reps):
                launch(plan)
            e1.record(stream)
            marks.append((i, e0, e1))
    marks[-1][2].synchronize()
    best = [float("inf")] * len(plans)
    for i, e0, e1 in marks:
        best[i] = min(best[i], hip.get_elapsed_time(e0, e1) / reps)
    return best


def pick(plans_by_rank: Sequence[Tuple[int, object]], bufs, shape: Tuple[int, int, int], stream=None,
         margin: float = TIE_MARGIN) -> Tuple[int, List[Tuple[int, float]]]:
    """Times the candidates and applies ``choose``.  Returns ``(kept rank, [(rank, ms), ...])``."""
    ms = time_candidates([p for _, p in plans_by_rank], bufs, shape, stream=stream, settle_ms=PICK_SETTLE_MS)
    timings = [(rank, t) for (rank, _), t in zip(plans_by_rank, ms)]
    return choose(timings, margin), timings


def summarise(timings: Sequence[Tuple[int, float]], kept: int) -> dict:
    """What a report says about one tuning decision."""
    by_rank = dict(timings)
    fastest: Optional[int] = min(by_rank, key=by_rank.get) if by_rank else None
    out = {"kept_rank": kept, "fastest_rank": fastest}
    if fastest is not None and kept in by_rank:
        out["kept_over_fastest"] = round(by_rank[kept] / by_rank[fastest], 4)
        if 1 in by_rank:
            out["top1_over_fastest"] = round(by_rank[1] / by_rank[fastest], 4)
    return out
