"""The parts of bench.py that need no device: the one-GPU rule, the traffic figure looked up from
the committed counter summary, and the kernels it compiles for the two clock readings."""

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2 and "ONE GPU" in proc.stderr and proc.stdout.strip() == ""


def test_traffic_key_ignores_the_wave_split_and_the_instruction():
    a = "b128x128x64_w32x64_mi16_s3_p0.0_v4_e0_z3.8_a0_d1"
    b = "b128x128x64_w64x64_mi32_s3_p0.0_v4_e0_z3.8_a0_d1"
    c = "b64x256x64_w64x64_mi16_s3_p0.0_v4_e0_z3.8_a0_d1"
    assert bench.traffic_key(a) == bench.traffic_key(b) == "b128x128x64_s3_p0.0_v4_e0_z3.8_a0_d1"
    assert bench.traffic_key(c) != bench.traffic_key(a)


def test_traffic_comes_from_the_committed_counter_summary_only_for_the_kernels_it_was_taken_with():
    table = json.loads(bench.TRAFFIC_FILE.read_text())
    sweep = table["sweep"]["per_shape"]
    assert sorted(sweep) == sorted(f"M{i}" for i in range(14))
    kept = {name: row["kernel"] for name, row in sweep.items()}
    total, source = bench.measured_traffic("sweep", kept)
    assert total == pytest.approx(sum(r["traffic_bytes"] for r in sweep.values()) / 14) and "profiles/" in source
    assert total == pytest.approx(table["sweep"]["traffic_bytes_per_launch"], rel=1e-6)
    # the algorithmic bytes are the formula 4(MK + KN + MN); measured traffic is above them, below 6x
    assert 1.0 < total / table["sweep"]["algorithmic_bytes_per_launch"] < 6.0
    # same block tile, other wave split: same figure; another block tile: no figure, with the reason
    import re
    other_split = dict(kept, M0=re.sub(r"_w\d+x\d+_mi\d+", "_w16x128_mi16", kept["M0"]))
    assert other_split["M0"] != kept["M0"]
    assert bench.measured_traffic("sweep", other_split)[0] == pytest.approx(total)
    other_tile = dict(kept, M0="b64x256x64_w64x64_mi16_s3_p0.0_v4_e0_z3.8_a0_d1")
    figure, reason = bench.measured_traffic("sweep", other_tile)
    assert figure is None and "M0" in reason
    # a single shape of the sweep falls back to its row; an unknown workload has no figure
    one, _ = bench.measured_traffic("M3", {"M3": kept["M3"]})
    assert one == sweep["M3"]["traffic_bytes"]
    own_row = table["M10"]["per_shape"]["M10"]                             # a workload with a counter run of its own
    assert bench.measured_traffic("M10", {"M10": own_row["kernel"]})[0] == own_row["traffic_bytes"]
    assert bench.measured_traffic("123x456x789", {"123x456x789": kept["M0"]})[0] is None
    for name in ("M10", "M0", "cfg4"):
        assert name in table and table[name]["per_shape"]


def test_traffic_lookup_uses_every_counter_run_that_covers_a_shape(tmp_path, monkeypatch):
    """A shape may have been measured with several kernels (the tuner keeps one of two near-equal
    tiles from run to run): the figure of the kernel that this run kept is used, from the
    workload's own counter run, from a second run of it, or from the sweep's row of the shape."""
    big, small = "b256x256x32_w128x128_mi32_s3_p0.0_v4_e0_z3.8_a0_d1", "b128x128x32_w64x64_mi16_s3_p0.0_v4_e0_z3.8_a0_d1"
    table = {"sweep": {"per_shape": {"M5": {"kernel": small, "traffic_bytes": 700}, "M6": {"kernel": big, "traffic_bytes": 300}},
                       "other_kernels": {"M5": [{"kernel": big, "traffic_bytes": 400}]}, "source": "s"},
             "M6": {"per_shape": {"M6": {"kernel": small, "traffic_bytes": 900}}, "source": "own"}}
    path = tmp_path / "traffic.json"
    path.write_text(json.dumps(table))
    monkeypatch.setattr(bench, "TRAFFIC_FILE", path)
    assert bench.measured_traffic("sweep", {"M5": small, "M6": big})[0] == 500.0
    assert bench.measured_traffic("sweep", {"M5": big, "M6": big})[0] == 350.0          # M5 from the second run
    assert bench.measured_traffic("sweep", {"M5": big, "M6": small})[0] is None         # nobody measured M6 with the small tile in the sweep
    assert bench.measured_traffic("M6", {"M6": small}) == (900.0, "own")
    assert bench.measured_traffic("M6", {"M6": big})[0] == 300.0                        # the sweep's row
    assert bench.measured_traffic("M5", {"M5": big})[0] == 400.0


def test_clock_kernels_compile_for_gfx950(hip_lib):
    from mlir_roller_amd import hip
    for source, symbol in ((bench.CLOCK_KERNEL, b"clock_probe"), (bench.SAMPLER_KERNEL, b"clock_sampler"), (bench.COPY_KERNEL, b"copy_kernel")):
        code, _ = hip.compile_source(source, "k.hip")
        assert code[:4] == b"\x7fELF" and symbol in code
    # the sampler starts on a flag that a second kernel of the same module raises
    assert b"raise_flag" in hip.compile_source(bench.SAMPLER_KERNEL, "k.hip")[0]


def test_named_configurations_are_the_four_of_the_baseline():
    assert [(n, s, d) for n, s, d in bench.NAMED_CONFIGS] == [
        ("cfg1", (2048, 2048, 2048), "uniform"), ("cfg2", (2048, 2048, 8192), "uniform"),
        ("cfg3", (4096, 8192, 4096), "uniform"), ("cfg4", (3000, 5000, 1536), "normal")]
    assert bench.PEAK_TFLOPS == pytest.approx(256 * 4 * 64 * 2.4e9 / 1e12, rel=1e-3)
