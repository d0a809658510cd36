"""The counter tool's arithmetic and result-file parsing (no GPU, no rocprofv3 needed)."""

import sqlite3

import pytest

from mlir_roller_amd import counters


def test_derived_figures_from_raw_counters():
    raw = {"SQ_VALU_MFMA_BUSY_CYCLES": 4294967296.0, "GRBM_GUI_ACTIVE": 35583765.0,
           "SQ_LDS_BANK_CONFLICT": 16777216.0, "SQ_LDS_IDX_ACTIVE": 67108864.0,
           "SQ_INSTS_VALU_MFMA_MOPS_F32": 536870912.0, "FETCH_SIZE": 393288.0, "WRITE_SIZE": 131072.0}
    d = counters.derive((4096, 8192, 4096), 1.85, raw, fetch_scale=2.0, write_scale=1.0)
    # busy SIMD-cycles / (cycles per XCD * 1024 SIMDs)
    assert d["MfmaUtil %"] == pytest.approx(100 * 4294967296 / (35583765 / 8 * 1024))
    assert d["LdsBankConflict"] == pytest.approx(16777216 / (67108864 - 16777216))     # conflicts per useful cycle
    assert d["MFMA FLOP / 2MNK"] == pytest.approx(1.0)                                 # 512 FLOP per counted op
    assert d["Traffic (MB)"] == pytest.approx((393288 * 2 + 131072) * 1024 / 1e6)
    assert d["Traffic / algorithmic"] == pytest.approx(d["Traffic (MB)"] * 1e6 / (4 * (4096 * 4096 + 4096 * 8192 + 4096 * 8192)))
    assert d["HBM-side GB/s"] == pytest.approx(d["Traffic (MB)"] / 1.85)
    assert counters.derive((8, 8, 8), 1.0, {}, 2.0, 1.0) == {}


def test_reads_rocprofv3_database_and_csv(tmp_path):
    db = tmp_path / "run" / "host" / "pmc_results.db"
    db.parent.mkdir(parents=True)
    con = sqlite3.connect(db)
    con.execute("create table counters_collection (kernel_name text, counter_name text, value real)")
    con.executemany("insert into counters_collection values (?, ?, ?)", [
        ("gemm_kernel", "FETCH_SIZE", 100.0), ("gemm_kernel", "FETCH_SIZE", 300.0),
        ("__amd_rocclr_fillBufferAligned", "FETCH_SIZE", 9999.0), ("gemm_kernel", "GRBM_GUI_ACTIVE", 8.0)])
    con.commit()
    con.close()
    got = counters.read_counters(tmp_path / "run", "gemm_kernel")
    assert got == {"FETCH_SIZE": 200.0, "GRBM_GUI_ACTIVE": 8.0}
    (tmp_path / "csvrun").mkdir()
    (tmp_path / "csvrun" / "pmc_counter_collection.csv").write_text(
        "Kernel_Name,Counter_Name,Counter_Value\ncopy_kernel(float4 const*),WRITE_SIZE,262144\ncopy_kernel(float4 const*),WRITE_SIZE,262144\nother,WRITE_SIZE,1\n")
    assert counters.read_counters(tmp_path / "csvrun", "copy_kernel") == {"WRITE_SIZE": 262144.0}
    with pytest.raises(RuntimeError):
        counters.read_counters(tmp_path / "csvrun", "gemm_kernel")


def test_counter_groups_respect_the_per_run_limits():
    for names in counters.GROUPS.values():
        assert sum(n.startswith("SQ_") for n in names) <= 8
        assert sum(n.startswith("GRBM_") for n in names) <= 2
        assert not ({"FETCH_SIZE", "WRITE_SIZE"} <= set(names))     # 3 + 2 TCC counters exceed the 4 available
    assert counters.SHAPES["M10"] == (4096, 8192, 4096) and len(counters.SHAPES) == 15


def test_workload_names_round_trip():
    assert counters.shape_of("M10") == (4096, 8192, 4096) and counters.shape_of("cfg4") == (3000, 5000, 1536)
    assert counters.shape_of("300x500x96") == (300, 500, 96)
    assert counters.workload_name((4096, 8192, 4096)) == "M10"
    assert counters.workload_name((300, 500, 96)) == "300x500x96"
    assert counters.shape_of(counters.workload_name((7, 8, 9))) == (7, 8, 9)
    for bad in ("M99", "3x4", "0x4x4", "axbxc"):
        with pytest.raises(ValueError):
            counters.shape_of(bad)
