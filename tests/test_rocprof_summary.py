"""The condenser of rocprofv3 databases (minerva_amd/rocprof_summary.py) on a small database
built here with the two tables it reads: grouping by (kernel, grid), the derived columns."""
import sqlite3

from minerva_amd import rocprof_summary as rs


def _db(tmp_path):
    path = str(tmp_path / "r.db")
    con = sqlite3.connect(path)
    con.execute("create table kernels (name text, duration integer, grid_size_x integer, grid_size_z integer)")
    con.execute("create table counters_collection (kernel_name text, counter_name text, value real, "
                "grid_size_x integer, grid_size_z integer)")
    gemm = "void mnv_gemm_kernel<MnvGemmTile<128, 128, 16, 2, 2, 0, 128>, (anonymous namespace)::SgemmNN>(int)"
    for dur, gx in ((1000000, 262144), (1100000, 262144), (90000, 65536)):
        con.execute("insert into kernels values (?, ?, ?, 1)", (gemm, dur, gx))
    con.execute("insert into kernels values ('void copy(float*)', 5000, 4096, 1)")
    for ctr, v in (("GRBM_GUI_ACTIVE", 8 * 2.0e6), ("SQ_VALU_MFMA_BUSY_CYCLES", 0.9 * 2.0e6 * 1024),
                   ("SQ_INSTS_VALU", 0.9 * 2.0e6 * 1024 / 64 + 1000), ("SQ_WAVE_CYCLES", 2.0e6 * 1024 * 3 / 4),
                   ("SQ_WAIT_INST_ANY", 2.0e6 * 1024 * 3 / 8)):
        con.execute("insert into counters_collection values (?, ?, ?, 262144, 1)", (gemm, ctr, v))
    con.commit()
    con.close()
    return path


def test_trace_table_groups_gemm_kernels_by_grid(tmp_path):
    text = rs.trace_table(rs.trace_rows(rs.open_db(_db(tmp_path)), "gemm"), 0.0)
    lines = text.splitlines()
    assert lines[0].split()[:3] == ["kernel", "grid.x", "z"]
    big = [l for l in lines if "262144" in l][0].split()
    assert "mnv_gemm_kernel<T128x128x16," in big[0] and big[-6] == "2" and abs(float(big[-4]) - 1050.0) < 1e-6
    assert any(l.startswith("copy") and " 0 " in l for l in lines)   # not split by grid


def test_counter_table_derives_utilisation(tmp_path):
    path = _db(tmp_path)
    rows = rs.counter_rows([rs.open_db(path)], "gemm")
    text = rs.counter_table(rows, rs.trace_rows(rs.open_db(path), "*"))
    head, row = text.splitlines()[:2]
    for col in ("cycles", "MFMA busy", "other VALU", "waves/SIMD", "waiting", "avg_us", "clock GHz"):
        assert col in head
    assert " 90.0%" in row and " 3.00" in row and " 50.0%" in row
    assert " 1050.00" in row and " 1.90" in row   # 2.0e6 cycles / 1050 us
