"""Headline benchmark: fp32 GEMM TFLOP/s of the Roller-selected HIP kernels over M0..M13 on one
MI355X, as one JSON line on stdout (everything else goes to stderr).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload sweep|M0..M13|cfg4|MxNxK|copy] [--topk 4]

A "step" is one pass over the workload: one launch of the chosen kernel for every shape in it,
with A, B and C resident in HBM.  Before the timed region, and reported separately, the Roller
flow of the reference runs per shape (benchmark.py:28-58 there): policy search, JIT of the
top-k hints, a short timing of each, one kept.  The policy's order decides near ties: a later hint
displaces an earlier one only if it is faster by more than the run-to-run spread
(``mlir_roller_amd.tuner``).  The kept kernel is verified against a float32 and a float64 host
GEMM before it is timed; a kernel outside tolerance is discarded and the next candidate takes
its place.  Winners are remembered in the code-object cache directory so that a second run on
the same machine (for example under rocprofv3) launches the chosen kernels only
(``tuned_from_cache`` says when that happened; ``--retune`` ignores the memory).

The line also carries
  roofline       the GEMM kernel against the fp32 MFMA peak: algorithmic FLOPs (2*M*N*K per launch,
                 summed over the launches of a step) over the HIP-event time of the timed region,
                 taken on the stream the kernels run on; ``traffic`` = HBM-side bytes per launch
                 from the committed counter summary when it was taken with the same kernels;
  cpu_baseline   numpy float32 matmul (its BLAS, all host cores) timed on the same inputs, one
                 pass over the workload; a reported figure, not a target;
  compile_s_cold hiprtc time of the top-k kernels of every shape with every cache bypassed (what a
                 first run pays; the reference recompiles every (shape, hint), roller.py:358-387);
  named_configs  the four named problem sizes incl. the ragged 3000x5000x1536 with standard-normal
                 entries: TFLOP/s, fraction of peak, both error measures, bitwise rerun;
  device         name, CU count, data-sheet clock and the engine clock measured under MFMA load
                 right after the timed region;
  per_shape      ms (mean of a batch, minimum and median of single launches), TFLOP/s, % of peak,
                 kept hint and its rank for every shape.
"""

from __future__ import annotations

import argparse
import contextlib
import ctypes
import hashlib
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

import numpy as np  # noqa: E402

PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix peak: 256 CUs * 256 FLOP/clk * 2.4 GHz
# HBM-side bytes per launch of the chosen kernels, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script (scaled by what the same counters read for the copy workload); keyed by workload and by
# the kernel that ran for every shape, so a run that picked other kernels reports null instead
TRAFFIC_FILE = ROOT / "profiles" / "traffic.json"

NAMED_CONFIGS = [("cfg1", (2048, 2048, 2048), "uniform"), ("cfg2", (2048, 2048, 8192), "uniform"),
                 ("cfg3", (4096, 8192, 4096), "uniform"), ("cfg4", (3000, 5000, 1536), "normal")]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def blas_threads() -> int:
    try:
        from threadpoolctl import threadpool_info
        counts = [p.get("num_threads", 0) for p in threadpool_info() if p.get("user_api") == "blas"]
        if counts:
            return int(max(counts))
    except Exception:
        pass
    return int(os.environ.get("OPENBLAS_NUM_THREADS") or os.environ.get("OMP_NUM_THREADS") or os.cpu_count() or 1)


COPY_KERNEL = r"""
extern "C" __global__ void copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) dst[i] = src[i];
}
"""

# Engine clock under matrix load: every wave runs a chain of MFMAs and reads the shader cycle counter
# and the constant 100 MHz counter around it.
CLOCK_KERNEL = r"""
typedef float v4f __attribute__((ext_vector_type(4)));
extern "C" __global__ __launch_bounds__(256) void clock_probe(long long* out, float* sink, int iters) {
  v4f acc[8];
  for (int i = 0; i < 8; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
  const float a = 1.0f + threadIdx.x, b = 0.5f;
  long long c0 = __builtin_readcyclecounter();
  long long r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
  }
  long long c1 = __builtin_readcyclecounter();
  long long r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
  for (int i = 0; i < 8; ++i) s += acc[i][0];
  if ((threadIdx.x & 63) == 0) {
    const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
    out[2 * w] = c1 - c0;
    out[2 * w + 1] = r1 - r0;
    sink[w] = s;
  }
}
"""


# Engine clock under the GEMM load itself: one wave on a second stream sleeps and samples the two
# counters while the timed steps run.  It starts sampling when `flag` is raised (a one-thread kernel
# queued on the GEMM stream right ahead of the timed region does that; the wait gives up after
# `max_wait` naps) and ends after `ticks` of the 100 MHz counter or `max_iters` samples, whichever
# comes first.
SAMPLER_KERNEL = r"""
extern "C" __global__ void raise_flag(long long* flag) { __hip_atomic_store(flag, 1LL, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT); }
extern "C" __global__ void clock_sampler(long long* out, long long* flag, long long ticks, int max_wait, int max_iters) {
  int waited = 0;
  while (__hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) == 0 && waited < max_wait) {
    __builtin_amdgcn_s_sleep(127);
    ++waited;
  }
  const long long r0 = __builtin_amdgcn_s_memrealtime();
  const long long c0 = __builtin_readcyclecounter();
  long long r = r0, c = c0;
  int it = 0;
  while (r - r0 < ticks && it < max_iters) {
    __builtin_amdgcn_s_sleep(64);
    r = __builtin_amdgcn_s_memrealtime();
    c = __builtin_readcyclecounter();
    ++it;
  }
  if (threadIdx.x == 0) { out[0] = c - c0; out[1] = r - r0; out[2] = it; out[3] = waited; }
}
"""


def copy_workload(args) -> int:
    """Calibration workload for the HBM traffic counters: a plain copy of 256 MiB per launch
    (256 MiB read, 256 MiB written), so that FETCH_SIZE / WRITE_SIZE of the GEMM kernel can be
    scaled by what the same counters read for a known amount of traffic."""
    from mlir_roller_amd import hip
    from mlir_roller_amd.hip import DeviceArray, Event, Module, Stream

    hip.init(0)
    nbytes = 256 << 20
    src = DeviceArray.from_host(np.ones(nbytes // 4, np.float32))
    dst = DeviceArray.zeros((nbytes // 4,))
    code, _ = hip.compile_source(COPY_KERNEL, "copy.hip")
    func = Module(code).get_function("copy_kernel")
    stream = Stream()
    n16 = ctypes.c_long(nbytes // 16)
    launch = lambda: func((4096,), (256,), (src, dst, n16), stream=stream)
    for _ in range(args.warmup):
        launch()
    e0, e1 = Event(), Event()
    e0.record(stream)
    for _ in range(args.steps):
        launch()
    e1.record(stream)
    e1.synchronize()
    ms = hip.get_elapsed_time(e0, e1) / max(args.steps, 1)
    ok = bool(np.all(dst.get() == 1.0))
    print(json.dumps({"metric": "copy_kernel GB/s (read+write)", "value": round(2 * nbytes / ms / 1e6, 1), "unit": "GB/s",
                      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
                      "config": {"workload": "copy: 256 MiB read + 256 MiB written per launch"},
                      "bytes_read_per_launch": nbytes, "bytes_written_per_launch": nbytes, "ok": ok}), flush=True)
    return 0 if ok else 1


def traffic_key(kernel_tag: str) -> str:
    """The part of a kernel's tag that decides its HBM-side traffic: block tile, K step, depth,
    layout and workgroup order -- not how the block tile is split over waves or which matrix
    instruction multiplies it."""
    import re
    return re.sub(r"_w\d+x\d+_mi\d+", "", kernel_tag)


def measured_traffic(workload: str, kernels: dict):
    """(bytes per launch, note) from the committed counter summary, or (None, reason).  The summary
    holds, per workload and shape, the bytes one launch moved and the kernel it was measured with;
    the figure is used only if every shape of this run kept a kernel with the same traffic key."""
    try:
        table = json.loads(TRAFFIC_FILE.read_text())
    except Exception:
        return None, f"{TRAFFIC_FILE.name} not found"
    # counter runs that cover these shapes: the workload's own and, for shapes of the sweep, the sweep's
    entries = [table[w] for w in (workload, "sweep") if w in table and set(kernels) <= set(table[w].get("per_shape", {}))]
    if not entries:
        return None, f"no counter run recorded for workload {workload!r}"
    total, differing = 0.0, []
    for name, tag in kernels.items():
        measured = []
        for entry in entries:
            measured.append(entry["per_shape"][name])
            measured += entry.get("other_kernels", {}).get(name, [])   # the same workload run with other kernels kept
        hit = [m for m in measured if traffic_key(m["kernel"]) == traffic_key(tag)]
        if hit:
            total += hit[0]["traffic_bytes"]
        else:
            differing.append(name)
    if differing:
        differing.sort()
        return None, ("counter run was taken with other block tiles for " + ", ".join(differing[:4])
                      + ("..." if len(differing) > 4 else ""))
    return total / len(kernels), entries[0].get("source", "")


def main() -> int:
    from mlir_roller_amd.tuner import DEFAULT_TOPK, TIE_MARGIN

    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="sweep", help="sweep (M0..M13), one of M0..M13, cfg4 (3000x5000x1536), any MxNxK, or copy (traffic-counter calibration)")
    ap.add_argument("--topk", type=int, default=DEFAULT_TOPK)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--retune", action="store_true", help="ignore remembered winners")
    ap.add_argument("--depth", type=int, default=None, help="pipeline depth 1..5 (default: the sweep's, 3; the reference's 2 is the same kernel)")
    ap.add_argument("--trans-b", action="store_true", help="the kernels that take the second operand as Bt[N, K]")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--lean", action="store_true",
                    help="profiling mode: no cold-compile timing, no named configurations, no clock probe")
    args = ap.parse_args()

    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (the GEMM path has no multi-GPU part); got --gpus {args.gpus}",
              file=sys.stderr)
        return 2

    if args.workload == "copy":
        return copy_workload(args)

    from mlir_roller_amd import hip, tuner
    from mlir_roller_amd.analyze import MatmulConfig, get_roller_hints
    from mlir_roller_amd.arch import MI355X
    from mlir_roller_amd.benchmark import README_SHAPES
    from mlir_roller_amd import benchmark as sweep
    from mlir_roller_amd.hip import DeviceArray, Event, GemmConfig, GemmPlan, Module, Stream
    PIPELINE_DEPTH = sweep.PIPELINE_DEPTH if args.depth is None else args.depth
    from mlir_roller_amd.roller import gemm_errors, hint_to_gemm_config, make_inputs

    if args.workload == "sweep":
        names = [f"M{i}" for i in range(14)]
        shapes = list(README_SHAPES)
        workload = "M0-M13: the 14 fp32 GEMM shapes of the reference's table, (M,N,K) in {2048,4096,8192}^3"
    elif args.workload == "cfg4":
        names, shapes = ["cfg4"], [(3000, 5000, 1536)]
        workload = "cfg4: M=3000 N=5000 K=1536, standard-normal entries (ragged tiles)"
    elif "x" in args.workload:
        dims = tuple(int(v) for v in args.workload.lower().split("x"))
        if len(dims) != 3 or min(dims) <= 0:
            print(f"bench.py: --workload {args.workload}: expected MxNxK", file=sys.stderr)
            return 2
        names, shapes = [args.workload.lower()], [dims]
        workload = f"M={dims[0]} N={dims[1]} K={dims[2]}"
    else:
        idx = int(args.workload.lstrip("Mm"))
        names, shapes = [f"M{idx}"], [README_SHAPES[idx]]
        workload = f"M{idx}: M={shapes[0][0]} N={shapes[0][1]} K={shapes[0][2]}"
    dist = "normal" if args.workload == "cfg4" else "uniform"

    hip.init(0)
    props = hip.device_info()
    arch = MI355X.from_device(props)
    device_name = props.name.decode().strip() or f"{props.arch.decode().split(':')[0]} (the runtime reports no product name)"
    log(f"[bench] {device_name} {props.arch.decode()} CUs={props.compute_units} clock={props.clock_khz / 1e6:.2f} GHz")

    cache_dir = Path(os.environ.get("ROLLER_HIP_CACHE", str(hip.DEFAULT_CACHE_DIR)))
    cache_dir.mkdir(parents=True, exist_ok=True)
    template_id = hashlib.sha1(hip.template_source().encode()).hexdigest()[:12]
    tuned_path = cache_dir / f"tuned_{template_id}_top{args.topk}_d{PIPELINE_DEPTH}{'_tb' if args.trans_b else ''}.json"
    tuned = {}
    if tuned_path.exists() and not args.retune:
        try:
            tuned = json.loads(tuned_path.read_text())
        except Exception:
            tuned = {}

    stream = Stream()
    timers = {"search_s": 0.0, "compile_s": 0.0, "tune_s": 0.0, "verify_s": 0.0}
    cpu = {"time": 0.0, "flops": 0.0}
    candidates_seen: dict = {}   # GemmConfig -> None, every kernel a cold run would have to compile
    pairs_seen: list = []        # one entry per (shape, hint): what the reference's flow compiles
    from_cache_shapes = prepared_shapes = 0

    def time_plan(plan, bufs, shape, reps, warm):
        # every measurement is preceded, without a synchronisation in between, by enough launches
        # of the same kernel to bring the engine clock back up
        M, N, K = shape
        for _ in range(tuner.ramp_launches(shape, warm)):
            plan.launch(bufs[0], bufs[1], bufs[2], M, N, K, stream=stream)
        e0, e1 = Event(), Event()
        e0.record(stream)
        for _ in range(reps):
            plan.launch(bufs[0], bufs[1], bufs[2], M, N, K, stream=stream)
        e1.record(stream)
        e1.synchronize()
        return hip.get_elapsed_time(e0, e1) / reps

    def prepare(name, shape, distribution, baseline: bool):
        """Policy search, JIT, tuning and verification for one shape.  Returns a case record."""
        nonlocal from_cache_shapes, prepared_shapes
        prepared_shapes += 1
        M, N, K = shape
        cfg = MatmulConfig(M, N, K, 32)
        A, B = make_inputs(cfg, args.seed, distribution)
        bufs = (DeviceArray.from_host(A), DeviceArray.from_host(B.T if args.trans_b else B), DeviceArray.zeros((M, N)))

        t0 = time.perf_counter()
        hints = get_roller_hints(cfg, arch, topk=args.topk, pipeline_depth=PIPELINE_DEPTH)
        timers["search_s"] += time.perf_counter() - t0

        usable = []  # (rank, GemmConfig, hint text)
        for rank, hint in enumerate(hints, 1):
            try:
                g = hint_to_gemm_config(cfg, hint, PIPELINE_DEPTH, trans_b=args.trans_b)
                hip.config_check(g)
                usable.append((rank, g, repr(hint)))
                candidates_seen[g] = None
                pairs_seen.append(g)
            except Exception as e:  # a hint may not fit the device: skip it, like the reference's sweep
                log(f"[bench] {name} hint {rank} skipped: {e}")

        key = f"{M}x{N}x{K}:{distribution}"
        order = []   # ranks in the order in which verification tries them
        timings = []
        # A remembered winner is a kernel (its tag), not a rank: ranks move when the policy's constants
        # do.  It is reused only if today's hints still hold that kernel, at whatever rank.
        remembered = [r for r, g, _ in usable if key in tuned and g.tag() == tuned[key].get("kernel")]
        replayed = bool(remembered)
        if replayed:
            order = [remembered[0]]
            by_tag = {g.tag(): r for r, g, _ in usable}
            timings = [(by_tag[tag], ms) for tag, ms in tuned[key].get("timings", []) if tag in by_tag]
            from_cache_shapes += 1
        else:
            t0 = time.perf_counter()
            plans = []
            for rank, g, _ in usable:
                try:
                    plan = GemmPlan(g)
                    timers["compile_s"] += plan.compile_ms / 1e3
                    plans.append((rank, plan))
                except Exception as e:
                    log(f"[bench] {name} hint {rank} failed to build: {e}")
            kept, timings = tuner.pick(plans, bufs, shape, stream=stream)
            # verification order: the kept one, then the others by measured time
            order = [kept] + [r for r, _ in sorted(timings, key=lambda t: t[1]) if r != kept]
            timers["tune_s"] += time.perf_counter() - t0
        if not order or order[0] < 0:
            raise RuntimeError(f"{name}: no usable hint")

        # host results: the float32 GEMM doubles as the CPU baseline sample
        t0 = time.perf_counter()
        C32 = A @ B
        t_host = time.perf_counter() - t0
        if baseline and not args.no_cpu_baseline:
            t0 = time.perf_counter()
            C32 = np.matmul(A, B, out=C32)
            t_host = min(t_host, time.perf_counter() - t0)
            cpu["time"] += t_host
            cpu["flops"] += 2.0 * M * N * K

        t0 = time.perf_counter()
        by_rank = {r: (g, text) for r, g, text in usable}
        chosen = None
        for rank in order:
            g, text = by_rank[rank]
            plan = GemmPlan(g)
            bufs[2].fill_bytes(0xFF)
            plan.launch(bufs[0], bufs[1], bufs[2], M, N, K, stream=stream)
            hip.synchronize()
            first = bufs[2].get()
            rep = gemm_errors(first, A, B, C32)
            if rep["ok"]:
                bufs[2].fill_bytes(0xFF)
                plan.launch(bufs[0], bufs[1], bufs[2], M, N, K, stream=stream)
                hip.synchronize()
                rep["bitwise_rerun"] = bool(np.array_equal(first.view(np.uint32), bufs[2].get().view(np.uint32)))
                chosen = (rank, g, text, plan, rep)
                break
            log(f"[bench] {name} hint {rank} outside tolerance, discarded: {rep}")
        timers["verify_s"] += time.perf_counter() - t0
        if chosen is None:
            raise RuntimeError(f"{name}: every hint failed verification")
        rank, g, text, plan, rep = chosen
        tag_of = {r: gg.tag() for r, gg, _ in usable}
        tuned[key] = {"kernel": g.tag(), "timings": [[tag_of[r], t] for r, t in timings if r in tag_of]}
        summary = tuner.summarise(timings, rank)
        summary["tuning"] = "from_cache" if replayed else "this_run"
        ms = dict(timings).get(rank, float("nan"))
        log(f"[bench] {name} {shape}: rank {rank}/{len(hints)} {g.tag()}  {ms:.4f} ms  "
            f"{2.0 * M * N * K / ms / 1e9:.1f} TFLOP/s " + ("(tuning figures replayed from an earlier run's memory) " if replayed else "")
            + f" normwise {rep['normwise']:.2e} max_abs {rep['max_abs']:.2e}  {summary}")
        return {"name": name, "shape": shape, "plan": plan, "bufs": bufs, "rank": rank, "hints": len(hints), "tuned_ms": ms,
                "summary": summary, "cfg": g, "hint": text, "rep": rep, "host_ms": t_host * 1e3, "dist": distribution}

    cases = []
    try:
        for name, shape in zip(names, shapes):
            cases.append(prepare(name, shape, dist, baseline=True))
    except RuntimeError as e:
        log(f"[bench] {e}")
        return 1

    # ---- the timed region: W warm-up steps, then exactly K steps between two events -------------
    def one_step():
        for c in cases:
            M, N, K = c["shape"]
            c["plan"].launch(c["bufs"][0], c["bufs"][1], c["bufs"][2], M, N, K, stream=stream)

    # Warm-up and timed steps are queued back to back, as in the reference's protocol
    # (roller.py:564-578): a synchronisation between them would let the engine clock drop and put
    # its ramp inside the timed region.  Device-wide synchronisation brackets the whole.
    clock_probe = None
    if not args.lean:
        code, _ = hip.compile_source(CLOCK_KERNEL, "clock_probe.hip")
        probe_mod = Module(code)
        clock_probe = probe_mod.get_function("clock_probe")
        probe_waves = 4 * props.compute_units   # one workgroup of four waves per CU: one wave per SIMD
        probe_out, probe_sink = DeviceArray((2 * probe_waves,), np.int64), DeviceArray((probe_waves,))
        sampler_mod = Module(hip.compile_source(SAMPLER_KERNEL, "clock_sampler.hip")[0])
        clock_sampler = sampler_mod.get_function("clock_sampler")
        raise_flag = sampler_mod.get_function("raise_flag")
        sampler_out = DeviceArray.zeros((4,), np.int64)
        sampler_flag = DeviceArray.zeros((1,), np.int64)
        side_stream = Stream()
        # sample for about 70 % of what the timed steps should take (tuned times; 1 ms at least)
        expect_ms = args.steps * sum(c["tuned_ms"] if c["tuned_ms"] == c["tuned_ms"] else 2.0 * c["shape"][0] * c["shape"][1] * c["shape"][2] / 120e9
                                     for c in cases)
        sampler_ticks = int(max(1.0, 0.7 * expect_ms) * 1e5)       # 100 MHz: 1e5 ticks per millisecond
    hip.synchronize()
    step_est_ms = sum(2.0 * s[0] * s[1] * s[2] for s in shapes) / 120e9
    for _ in range(max(args.warmup, int(tuner.RAMP_MS / step_est_ms) + 1)):
        one_step()
    e0, e1 = Event(), Event()
    wall0 = time.perf_counter()
    if clock_probe is not None:
        # (the sampler naps about 3.4 us at a time: 200 000 naps outlast any warm-up that fits this script)
        clock_sampler((1,), (64,), (sampler_out, sampler_flag, ctypes.c_longlong(sampler_ticks), 200000, max(1000, sampler_ticks // 20)),
                      stream=side_stream)
        raise_flag((1,), (1,), (sampler_flag,), stream=stream)
    e0.record(stream)
    for _ in range(args.steps):
        one_step()
    e1.record(stream)
    if clock_probe is not None:
        # queued directly behind the timed steps, so it sees the clock the GEMMs ran at
        clock_probe((props.compute_units,), (256,), (probe_out, probe_sink, 20000), stream=stream)
    e1.synchronize()
    hip.synchronize()
    wall_ms = (time.perf_counter() - wall0) * 1e3
    total_ms = hip.get_elapsed_time(e0, e1)
    ms_per_step = total_ms / max(args.steps, 1)
    achieved_mhz = probe_mhz = None
    sampler_ms = None
    if clock_probe is not None:
        ticks = probe_out.get().reshape(-1, 2).astype(np.float64)
        probe_mhz = round(float(np.median(ticks[:, 0] / np.maximum(ticks[:, 1], 1.0))) * 100.0, 1)
        cycles, real, _samples, _naps = (int(v) for v in sampler_out.get())
        if real > 0:
            achieved_mhz = round(cycles / real * 100.0, 1)
            sampler_ms = round(real / 1e5, 3)

    # per-shape timing of the winners (outside the headline region)
    per_shape = []
    for c in cases:
        M, N, K = c["shape"]
        ms = time_plan(c["plan"], c["bufs"], c["shape"], reps=max(args.steps, 5), warm=2)
        # spread of single launches: an event after every launch of a second batch that follows at once
        marks = [Event() for _ in range(max(args.steps, 5) + 1)]
        marks[0].record(stream)
        for mark in marks[1:]:
            c["plan"].launch(c["bufs"][0], c["bufs"][1], c["bufs"][2], M, N, K, stream=stream)
            mark.record(stream)
        marks[-1].synchronize()
        each = sorted(hip.get_elapsed_time(a, b) for a, b in zip(marks, marks[1:]))
        tf = 2.0 * M * N * K / ms / 1e9
        c["tflops"] = tf
        per_shape.append({"name": c["name"], "M": M, "N": N, "K": K, "ms": round(ms, 5),
                          "min_ms": round(each[0], 5), "median_ms": round(each[len(each) // 2], 5), "tflops": round(tf, 2),
                          "pct_of_peak": round(100 * tf / PEAK_TFLOPS, 1), "kernel": c["cfg"].tag(),
                          "hint_rank": c["rank"], "hints": c["hints"], **c["summary"],
                          "normwise_err": c["rep"]["normwise"], "max_abs_err": c["rep"]["max_abs"],
                          "max_abs_bound": c["rep"]["bound"], "bitwise_rerun": c["rep"]["bitwise_rerun"],
                          "host_ms": round(c["host_ms"], 2)})

    # ---- the four named configurations (outside the timed region) ----------------------------------
    named = None
    if not args.lean and args.workload == "sweep":
        named = []
        by_shape = {tuple(c["shape"]): c for c in cases}
        for cname, shape, distribution in NAMED_CONFIGS:
            c = by_shape.get(shape) if distribution == dist else None
            if c is None:
                # free the sweep's buffers of other shapes first?  no: 3000x5000x1536 adds 110 MB
                try:
                    c = prepare(cname, shape, distribution, baseline=False)
                except RuntimeError as e:
                    log(f"[bench] {e}")
                    return 1
                M, N, K = shape
                c["tflops"] = 2.0 * M * N * K / time_plan(c["plan"], c["bufs"], shape, reps=max(args.steps, 5), warm=2) / 1e9
            named.append({"name": cname, "M": shape[0], "N": shape[1], "K": shape[2], "inputs": f"{distribution}, seed {args.seed}",
                          "tflops": round(c["tflops"], 2), "frac_of_peak": round(c["tflops"] / PEAK_TFLOPS, 4),
                          "kernel": c["cfg"].tag(), "hint_rank": c["rank"], "normwise_err": c["rep"]["normwise"],
                          "max_abs_err": c["rep"]["max_abs"], "max_abs_bound": c["rep"]["bound"],
                          "within_tolerance": c["rep"]["ok"], "bitwise_rerun": c["rep"]["bitwise_rerun"]})

    with contextlib.suppress(Exception):
        tuned_path.write_text(json.dumps(tuned, indent=1))

    # ---- cold JIT cost: hiprtc on every kernel a first run compiles, every cache bypassed ----------
    compile_cold = None
    if not args.lean:
        # the compiler library keeps a cache of its own on disk (AMD_COMGR_CACHE_DIR, on by default):
        # point it at an empty directory for this phase, or "cold" would be a lookup
        import shutil
        import tempfile
        scratch_dir = tempfile.mkdtemp(prefix="roller_cold_jit_")
        previous = os.environ.get("AMD_COMGR_CACHE_DIR")
        os.environ["AMD_COMGR_CACHE_DIR"] = scratch_dir
        t_unique = {}
        try:
            for g in candidates_seen:
                t0 = time.perf_counter()
                hip.compile_config(g)
                t_unique[g] = time.perf_counter() - t0
        finally:
            if previous is None:
                os.environ.pop("AMD_COMGR_CACHE_DIR", None)
            else:
                os.environ["AMD_COMGR_CACHE_DIR"] = previous
            shutil.rmtree(scratch_dir, ignore_errors=True)
        compile_cold = {"unique_kernels": len(t_unique), "unique_s": round(sum(t_unique.values()), 2),
                        "per_shape_hint_pairs": len(pairs_seen), "pairs_s": round(sum(t_unique[g] for g in pairs_seen), 2)}

    flops_per_step = sum(2.0 * s[0] * s[1] * s[2] for s in shapes)
    bytes_per_step = sum(4.0 * (s[0] * s[2] + s[2] * s[1] + s[0] * s[1]) for s in shapes)
    tflops = flops_per_step / (ms_per_step * 1e-3) / 1e12
    launches = len(cases)
    traffic, traffic_note = measured_traffic(args.workload, {c["name"]: c["cfg"].tag() for c in cases})

    out = {
        "metric": "fp32 GEMM TFLOP/s (Roller-selected HIP MFMA kernels) over " + ("M0-M13" if args.workload == "sweep" else names[0]),
        "value": round(tflops, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": workload, "launches_per_step": launches, "inputs": f"{dist}, seed {args.seed}",
                   "topk": args.topk, "tie_margin": TIE_MARGIN, "pipeline_depth": PIPELINE_DEPTH, "trans_b": bool(args.trans_b)},
        "pct_of_fp32_matrix_peak": round(100 * tflops / PEAK_TFLOPS, 2),
        "roofline": {
            "bound": "mfma", "achieved": round(tflops, 3), "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tflops / PEAK_TFLOPS, 4), "traffic": traffic, "traffic_note": traffic_note,
            "kernel": "gemm_kernel", "avg_launch_ms": round(ms_per_step / launches, 5),
            "flops_per_launch": flops_per_step / launches, "algorithmic_bytes_per_launch": bytes_per_step / launches,
        },
        "cpu_baseline": None if args.no_cpu_baseline else {
            "value": round(cpu["flops"] / cpu["time"] / 1e12, 4), "unit": "TFLOP/s", "cores": blas_threads(), "kind": "port",
            "sample": f"numpy float32 matmul, best of 2, one pass over the same {launches} shape(s) and inputs "
                      f"({cpu['flops'] / 1e12:.2f} TFLOP in {cpu['time']:.1f} s)",
        },
        "wall_ms_per_step": round(wall_ms / max(args.steps, 1), 5),
        "search_s": round(timers["search_s"], 3), "compile_s": round(timers["compile_s"], 3),
        "compile_s_cold": compile_cold["pairs_s"] if compile_cold else None, "compile_cold": compile_cold,
        "tune_s": round(timers["tune_s"], 3), "tuned_from_cache": from_cache_shapes == prepared_shapes,
        "verify_s": round(timers["verify_s"], 3),
        "device": {"name": device_name, "arch": props.arch.decode(), "compute_units": props.compute_units,
                   "clock_mhz": props.clock_khz // 1000, "achieved_clock_mhz": achieved_mhz, "achieved_clock_window_ms": sampler_ms,
                   "mfma_probe_clock_mhz": probe_mhz,
                   "achieved_clock_note": "shader cycle counter over the 100 MHz constant counter: achieved = one sampling wave on a second "
                                          "stream while the timed steps run; mfma_probe = a pure-MFMA kernel queued directly behind them"},
        "named_configs": named,
        "per_shape": per_shape,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
