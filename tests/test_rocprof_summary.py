"""dmlx_amd/rocprof_summary.py on hand-made rocprofv3 CSV files: the derived figures that bench.py quotes from
profiles/counters.json (traffic scaled by the known-size copies, matrix-core busy share, vector instructions per
MFMA, waiting share) must follow from the counter rows by the formulas the tool documents."""
import csv
import io
import os
from contextlib import redirect_stdout

import pytest

from dmlx_amd import rocprof_summary as rs

KERNEL = "void dmoe::qgemm_wide_kernel<dmoe::FmtAffine4, true>(dmoe::GemmArgs)"
OTHER = "void dmoe::combine_kernel(unsigned short*)"
COPY = "__amd_rocclr_copyBuffer.kd"


def _write_pmc(path, rows):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "pmc_counter_collection.csv"), "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["Dispatch_Id", "Kernel_Name", "Grid_Size", "Workgroup_Size", "Counter_Name",
                                          "Counter_Value"])
        w.writeheader()
        for i, (name, wgs, counter, value) in enumerate(rows):
            disp = i if not isinstance(value, tuple) else value[1]
            w.writerow({"Dispatch_Id": disp, "Kernel_Name": name, "Grid_Size": wgs * 256, "Workgroup_Size": 256,
                        "Counter_Name": counter, "Counter_Value": value if not isinstance(value, tuple) else value[0]})


def test_traffic_is_scaled_by_the_probe_copies(tmp_path):
    fetch_dir, write_dir = str(tmp_path / "f"), str(tmp_path / "w")
    copy_kib = rs.COPY_BYTES / 1024
    # the counters read half / a quarter of the bytes that a known copy moves; a small stray copy must not shift the scale
    _write_pmc(fetch_dir, [(COPY, 1024, "FETCH_SIZE", copy_kib / 2), (COPY, 1024, "FETCH_SIZE", copy_kib / 2 * 0.995),
                           (COPY, 4, "FETCH_SIZE", 17.0),
                           (KERNEL, 10240, "FETCH_SIZE", 1000.0), (KERNEL, 10240, "FETCH_SIZE", 3000.0),
                           (KERNEL, 16, "FETCH_SIZE", 5.0),      # the small launch: below --min-workgroups
                           (OTHER, 64, "FETCH_SIZE", 123.0)])
    _write_pmc(write_dir, [(COPY, 1024, "WRITE_SIZE", copy_kib / 4), (KERNEL, 10240, "WRITE_SIZE", 100.0)])
    agg = rs.read_counters([fetch_dir, write_dir])
    rec = rs.derived(agg, "qgemm_wide_kernel<FmtAffine4, true>", min_workgroups=1000)
    f_scale = rs.COPY_BYTES / ((copy_kib / 2 + copy_kib / 2 * 0.995) / 2)
    w_scale = rs.COPY_BYTES / (copy_kib / 4)
    assert rec["traffic_bytes"] == int(round(2000.0 * f_scale + 100.0 * w_scale))
    assert rec["fetch_scale"] == pytest.approx(f_scale / 1024, abs=1e-3)
    assert rec["write_scale"] == pytest.approx(4.0, abs=1e-3)
    assert "mfma_busy" not in rec and "valu_per_mfma" not in rec and "wait_share" not in rec


def test_a_counter_split_over_rows_is_summed_per_dispatch(tmp_path):
    d = str(tmp_path / "c")
    # dispatch 7 reports SQ_INSTS_VALU in two rows (one per shader engine group), dispatch 8 in one
    _write_pmc(d, [(KERNEL, 512, "SQ_INSTS_VALU", (300.0, 7)), (KERNEL, 512, "SQ_INSTS_VALU", (436.0, 7)),
                   (KERNEL, 512, "SQ_INSTS_MFMA", (100.0, 7)),
                   (KERNEL, 512, "SQ_INSTS_VALU", (736.0, 8)), (KERNEL, 512, "SQ_INSTS_MFMA", (100.0, 8))])
    rec = rs.derived(rs.read_counters([d]), "qgemm_wide_kernel")
    assert rec == {"valu_per_mfma": 6.36}


def test_busy_and_wait_shares(tmp_path):
    d = str(tmp_path / "c")
    gui = 8 * 2.0e6                                   # summed over the 8 XCDs: 2.0 M cycles of launch
    busy = 0.634 * rs.N_SIMD * gui / rs.N_XCD
    _write_pmc(d, [(KERNEL, 512, "SQ_VALU_MFMA_BUSY_CYCLES", busy), (KERNEL, 512, "GRBM_GUI_ACTIVE", gui),
                   (KERNEL, 512, "SQ_WAIT_INST_ANY", 379.0), (KERNEL, 512, "SQ_WAVE_CYCLES", 1000.0)])
    rec = rs.derived(rs.read_counters([d]), "qgemm_wide_kernel")
    assert rec == {"mfma_busy": 0.634, "wait_share": 0.379}


def test_trace_summary_groups_by_kernel_and_grid(tmp_path):
    d = str(tmp_path / "t")
    os.makedirs(d)
    fields = ["Kernel_Name", "Workgroup_Size_X", "Workgroup_Size_Y", "Grid_Size_X", "Grid_Size_Y", "VGPR_Count",
              "Accum_VGPR_Count", "LDS_Block_Size", "Start_Timestamp", "End_Timestamp"]
    rows = [(KERNEL, 256, 1, 256 * 16, 640, 128, 128, 65536, 0, 1500000), (KERNEL, 256, 1, 256 * 16, 640, 128, 128, 65536, 0, 1400000),
            (KERNEL, 256, 1, 256 * 16, 8, 128, 128, 65536, 0, 100000), (OTHER, 256, 1, 256 * 64, 1, 16, 0, 0, 0, 5000),
            ("void at::native::elementwise_kernel()", 256, 1, 256, 1, 8, 0, 0, 0, 999999999)]
    with open(os.path.join(d, "kt_kernel_trace.csv"), "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(fields)
        w.writerows(rows)

    class Args:
        dirs = [d]
        title = "t"
        command = ["cmd"]
    out = io.StringIO()
    with redirect_stdout(out):
        rs.trace(Args)
    lines = [ln for ln in out.getvalue().splitlines() if ln.startswith("qgemm_wide_kernel") or ln.startswith("combine_kernel")]
    assert len(lines) == 3 and "elementwise" not in out.getvalue()
    big = next(ln for ln in lines if "16x640" in ln).split()
    assert big[-5:-1] == ["2", "1450.00", "1400.00", "1500.00"]
    small = next(ln for ln in lines if "16x8" in ln).split()
    assert small[-5] == "1" and small[-4] == "100.00"
