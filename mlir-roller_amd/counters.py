"""Hardware counters for the winning kernels: MFMA busy %, LDS bank conflicts, HBM-side GB/s.

    python -m mlir_roller_amd.counters [--shapes M0 M10 ...] [--csv counters.csv]

The reference's sweep reports time and GFLOPS only (/root/reference/src/benchmark.py:69-85) and
wraps one launch in an NVTX range for an external profiler (roller.py:556-562).  Here the
profiler is driven for the user: for every requested shape this tool runs ``bench.py
--workload <shape>`` as a child of ``rocprofv3 --pmc ...`` -- one run per counter group, because
rocprofv3 does not split counters over passes -- and reads the per-dispatch values of
``gemm_kernel`` from the result database.  A copy kernel of known size calibrates the two
traffic counters.

This process never touches the GPU itself (it imports nothing that initialises HIP): a process
that has initialised the GPU must not start other programs on this class of machine.
"""

from __future__ import annotations

import argparse
import csv
import json
import os
import shutil
import sqlite3
import subprocess
import sys
import tempfile
from pathlib import Path
from typing import Dict, List, Optional

REPO_ROOT = Path(__file__).resolve().parent.parent
BENCH = REPO_ROOT / "bench.py"

# one rocprofv3 run each (limits: 8 SQ_, 2 GRBM_ counters per run; FETCH_SIZE / WRITE_SIZE use
# 3 resp. 2 of the 4 TCC_ counters, so they cannot share a run)
GROUPS = {
    "mfma": ["SQ_VALU_MFMA_BUSY_CYCLES", "GRBM_GUI_ACTIVE", "SQ_LDS_BANK_CONFLICT", "SQ_LDS_IDX_ACTIVE",
             "SQ_INSTS_VALU_MFMA_MOPS_F32"],
    "fetch": ["FETCH_SIZE"],
    "write": ["WRITE_SIZE"],
}
COPY_BYTES = 256 << 20      # what ``bench.py --workload copy`` reads and writes per launch
XCDS, SIMDS = 8, 256 * 4    # MI355X: GRBM_GUI_ACTIVE is summed over the XCDs; MFMA busy over the SIMDs
SHAPES = {f"M{i}": s for i, s in enumerate([
    (2048, 2048, 2048), (2048, 2048, 8192), (2048, 4096, 2048), (2048, 4096, 4096), (2048, 8192, 2048),
    (2048, 8192, 4096), (2048, 8192, 8192), (4096, 2048, 2048), (4096, 4096, 8192), (4096, 8192, 2048),
    (4096, 8192, 4096), (8192, 2048, 8192), (8192, 4096, 2048), (8192, 4096, 4096)])}
SHAPES["cfg4"] = (3000, 5000, 1536)


def shape_of(name: str):
    """(M, N, K) of a workload name: M0..M13, cfg4, or a literal ``MxNxK``."""
    if name in SHAPES:
        return SHAPES[name]
    dims = tuple(int(v) for v in name.lower().split("x"))
    if len(dims) != 3 or min(dims) <= 0:
        raise ValueError(f"unknown workload {name!r}")
    return dims


def workload_name(shape) -> str:
    """The shortest name ``bench.py --workload`` accepts for a shape."""
    shape = tuple(int(v) for v in shape)
    for name, known in SHAPES.items():
        if known == shape:
            return name
    return "x".join(str(v) for v in shape)


def _run(cmd: List[str], cwd: Path, timeout: int) -> subprocess.CompletedProcess:
    env = dict(os.environ, TMPDIR=str(cwd))
    return subprocess.run(cmd, cwd=str(cwd), env=env, capture_output=True, text=True, timeout=timeout)


def profiled_bench(workload: str, counters: Optional[List[str]], work: Path, tag: str, steps: int = 3) -> Dict:
    """Runs bench.py for one workload, under rocprofv3 when ``counters`` is given.  Returns the
    bench JSON line plus, per counter, the mean value over the kernel's dispatches."""
    bench_cmd = [sys.executable, str(BENCH), "--workload", workload, "--steps", str(steps), "--warmup", "1"]
    if workload != "copy":
        bench_cmd += ["--no-cpu-baseline", "--lean"]
    out_dir = work / tag
    cmd = bench_cmd
    if counters:
        cmd = ["rocprofv3", "--pmc", *counters, "-d", str(out_dir), "-o", "pmc", "--"] + bench_cmd
    proc = _run(cmd, work, timeout=600)
    if proc.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)} failed ({proc.returncode}):\n{proc.stderr[-2000:]}")
    line = next((l for l in reversed(proc.stdout.splitlines()) if l.startswith("{")), None)
    result = {"bench": json.loads(line) if line else {}}
    if counters:
        kernel = "copy_kernel" if workload == "copy" else "gemm_kernel"
        result["counters"] = read_counters(out_dir, kernel)
    return result


def read_counters(out_dir: Path, kernel: str) -> Dict[str, float]:
    """Mean per-dispatch value of every counter rocprofv3 collected for ``kernel``."""
    sums: Dict[str, List[float]] = {}
    for db in out_dir.rglob("*_results.db"):
        con = sqlite3.connect(str(db))
        try:
            rows = con.execute("select counter_name, value from counters_collection where kernel_name = ?",
                               (kernel,)).fetchall()
        finally:
            con.close()
        for name, value in rows:
            sums.setdefault(name, []).append(float(value))
    for path in out_dir.rglob("*counter_collection.csv"):
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row.get("Kernel_Name", "").startswith(kernel):
                    sums.setdefault(row["Counter_Name"], []).append(float(row["Counter_Value"]))
    if not sums:
        raise RuntimeError(f"no counter values for {kernel} under {out_dir}")
    return {k: sum(v) / len(v) for k, v in sums.items()}


def derive(shape, ms: float, c: Dict[str, float], fetch_scale: float, write_scale: float) -> Dict:
    """The figures a reader wants, from raw counters (KiB for the two size counters)."""
    M, N, K = shape
    out = {}
    if "SQ_VALU_MFMA_BUSY_CYCLES" in c and c.get("GRBM_GUI_ACTIVE"):
        out["MfmaUtil %"] = 100.0 * c["SQ_VALU_MFMA_BUSY_CYCLES"] / (c["GRBM_GUI_ACTIVE"] / XCDS * SIMDS)
    if "SQ_LDS_BANK_CONFLICT" in c and c.get("SQ_LDS_IDX_ACTIVE"):
        busy = c["SQ_LDS_IDX_ACTIVE"] - c["SQ_LDS_BANK_CONFLICT"]
        out["LdsBankConflict"] = c["SQ_LDS_BANK_CONFLICT"] / busy if busy > 0 else float("nan")
    if "SQ_INSTS_VALU_MFMA_MOPS_F32" in c:
        out["MFMA FLOP / 2MNK"] = c["SQ_INSTS_VALU_MFMA_MOPS_F32"] * 512 / (2.0 * M * N * K)
    if "FETCH_SIZE" in c and "WRITE_SIZE" in c:
        traffic = (c["FETCH_SIZE"] * fetch_scale + c["WRITE_SIZE"] * write_scale) * 1024
        out["Traffic (MB)"] = traffic / 1e6
        out["Traffic / algorithmic"] = traffic / (4.0 * (M * K + K * N + M * N))
        if ms > 0:
            out["HBM-side GB/s"] = traffic / (ms * 1e-3) / 1e9
    return out


def collect(shape_names: List[str], work: Path, verbose: bool = True) -> List[Dict]:
    say = (lambda *a: print(*a, file=sys.stderr, flush=True)) if verbose else (lambda *a: None)
    say("[counters] tuning run (remembers the winning hint per shape)")
    for name in shape_names:
        profiled_bench(name, None, work, f"tune_{name}", steps=2)
    say("[counters] calibrating FETCH_SIZE / WRITE_SIZE with the copy kernel")
    fetch_copy = profiled_bench("copy", ["FETCH_SIZE"], work, "copy_fetch")["counters"]["FETCH_SIZE"]
    write_copy = profiled_bench("copy", ["WRITE_SIZE"], work, "copy_write")["counters"]["WRITE_SIZE"]
    fetch_scale = COPY_BYTES / 1024 / fetch_copy
    write_scale = COPY_BYTES / 1024 / write_copy
    say(f"[counters] scale factors: FETCH_SIZE x{fetch_scale:.3f}, WRITE_SIZE x{write_scale:.3f}")
    rows = []
    for name in shape_names:
        shape = shape_of(name)
        plain = profiled_bench(name, None, work, f"plain_{name}")["bench"]
        ms = plain["per_shape"][0]["ms"]
        merged: Dict[str, float] = {}
        for group, names in GROUPS.items():
            say(f"[counters] {name}: {group}")
            merged.update(profiled_bench(name, names, work, f"{group}_{name}")["counters"])
        row = {"shape": name, "M": shape[0], "N": shape[1], "K": shape[2], "ms": ms,
               "TFLOP/s": plain["per_shape"][0]["tflops"], "kernel": plain["per_shape"][0]["kernel"]}
        row.update(derive(shape, ms, merged, fetch_scale, write_scale))
        row.update({f"raw {k}": v for k, v in sorted(merged.items())})
        rows.append(row)
    return rows


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="rocprofv3 counters for the Roller-selected GEMM kernels")
    ap.add_argument("--shapes", nargs="*", default=["M0", "M10"], help="M0..M13, cfg4 or MxNxK (default: M0 M10)")
    ap.add_argument("--csv", default="gemm_counters.csv")
    ap.add_argument("--keep", action="store_true", help="keep the rocprofv3 output directory")
    args = ap.parse_args(argv)
    if shutil.which("rocprofv3") is None:
        print("rocprofv3 not found on PATH", file=sys.stderr)
        return 2
    try:
        for s in args.shapes:
            shape_of(s)
    except ValueError as e:
        print(e, file=sys.stderr)
        return 2
    work = Path(tempfile.mkdtemp(prefix="roller_counters_", dir="/tmp"))
    try:
        rows = collect(args.shapes, work)
    finally:
        if not args.keep:
            shutil.rmtree(work, ignore_errors=True)
    cols: List[str] = []
    for r in rows:
        cols += [k for k in r if k not in cols]
    out = Path(args.csv).resolve()
    with open(out, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=cols)
        w.writeheader()
        w.writerows(rows)
    for r in rows:
        print("  ".join(f"{k}={r[k]:.4g}" if isinstance(r[k], float) else f"{k}={r[k]}"
                        for k in cols if not k.startswith("raw ") and k in r))
    print(f"written {out}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
