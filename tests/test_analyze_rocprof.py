"""rocprofv3 CSV -> per-pair tables, on small synthetic traces written by the test."""
import csv

import pytest

from hfuse_amd import analyze_rocprof as A

N = "void hfuse::native_kernel<hfuse::{b}, 1024>(hfuse::{b}::Args, unsigned int)"
F = "void hfuse::fused_kernel<hfuse::{a}, hfuse::{b}, 1024, {m}>(hfuse::{a}::Args, hfuse::{b}::Args, hfuse::FuseGeom)"
V = "void hfuse::vertical_kernel<hfuse::{a}, hfuse::{b}, 1024>(hfuse::{a}::Args, hfuse::{b}::Args, hfuse::FuseGeom)"
B = "void hfuse::blockidx_kernel<hfuse::{a}, hfuse::{b}, 1024>(hfuse::{a}::Args, hfuse::{b}::Args, hfuse::FuseGeom)"
TRACE_COLS = ["Kind", "Kernel_Name", "Start_Timestamp", "End_Timestamp", "VGPR_Count", "Workgroup_Size_X",
              "Workgroup_Size_Y", "Workgroup_Size_Z", "Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"]


def test_parse_kernel_name():
    assert A.parse_kernel_name(N.format(b="Im2colBody")) == ("ST", ("im2col_kernel",))
    capped = "void hfuse::native_kernel_capped<hfuse::Im2colBody, 1024, 4>(hfuse::Im2colBody::Args, unsigned int)"
    assert A.parse_kernel_name(capped) == ("ST", ("im2col_kernel",))
    assert A.parse_kernel_name(F.format(a="HistcBody", b="MaxPoolBody", m="false")) == ("HF", ("kernelHistogram1D", "MaxPoolForward"))
    assert A.parse_kernel_name(F.format(a="BnStatsBody", b="HistcBody", m="true"))[0] == "HF+M"
    assert A.parse_kernel_name(V.format(a="EthashBody", b="Blake2bBody<4, false>")) == ("VF", ("ethash_search", "sia_blake2b_gpu_hash"))
    assert A.parse_kernel_name(B.format(a="Blake2bBody<9, true>", b="Sha256dBody")) == ("BI", ("blake2b_gpu_hash", "sha256d_gpu_hash_shared"))
    # the register-bounded builds (the reference's *_lb presets)
    assert A.parse_kernel_name(F.replace("fused_kernel<", "fused_kernel_lb<").format(a="HistcBody", b="MaxPoolBody", m="false"))[0] == "HF-LB"
    assert A.parse_kernel_name(F.replace("fused_kernel<", "fused_kernel_lb<").format(a="HistcBody", b="BnStatsBody", m="true"))[0] == "HF+M-LB"
    assert A.parse_kernel_name(V.replace("vertical_kernel<", "vertical_kernel_lb<").format(a="Im2colBody", b="MaxPoolBody")) == ("VF-LB", ("im2col_kernel", "MaxPoolForward"))
    assert A.KernelKey("HF-LB", ("a", "b"), 512).label() == "HF-LB@512" and A.KernelKey("VF-LB", ("a", "b"), 512).label() == "VF-LB@512"
    assert A.parse_kernel_name("void at::native::vectorized_elementwise_kernel<4, Foo>(int)") is None
    assert A.parse_kernel_name("void hfuse::(anonymous namespace)::copy_f32_kernel(float const*, float*, unsigned long long)") is None
    # every body the library instantiates has a YAML name
    import os, re
    src = os.path.join(os.path.dirname(os.path.abspath(A.__file__)), "csrc", "device")
    bodies = set()
    for fn in ("dl_bodies.h", "crypto_bodies.h"):
        bodies |= set(re.findall(r"^struct (\w+Body) \{", open(os.path.join(src, fn)).read(), re.M))
    assert bodies - {"Blake2bBody"} <= set(A.BODY_TO_KERNEL)


def write_trace(path, rows):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=TRACE_COLS, quoting=csv.QUOTE_NONNUMERIC)
        w.writeheader()
        t = 1000
        for name, dur, block, grid in rows:
            w.writerow({"Kind": "KERNEL_DISPATCH", "Kernel_Name": name, "Start_Timestamp": t, "End_Timestamp": t + dur,
                        "VGPR_Count": 32, "Workgroup_Size_X": block, "Workgroup_Size_Y": 1, "Workgroup_Size_Z": 1,
                        "Grid_Size_X": grid, "Grid_Size_Y": 1, "Grid_Size_Z": 1})
            t += dur + 500


def test_exec_time_table_assigns_shared_natives_by_order(tmp_path):
    """Max-pool runs at two shapes for two pairs: each pair's ST uses the launches that precede its fused kernel."""
    im, mp, hi = N.format(b="Im2colBody"), N.format(b="MaxPoolBody"), N.format(b="HistcBody")
    f1 = F.format(a="Im2colBody", b="MaxPoolBody", m="false")
    f2 = F.format(a="HistcBody", b="MaxPoolBody", m="false")
    v2 = V.format(a="HistcBody", b="MaxPoolBody")
    rows = [("void at::native::fill<float>(float*)", 5000, 256, 4096)]
    for _ in range(3):   # pair 1: A, B, back-to-back, fused
        rows += [(im, 47000, 512, 1 << 20), (mp, 31000, 256, 1 << 20), (im, 47000, 512, 1 << 20), (mp, 31000, 256, 1 << 20),
                 (f1, 72000, 768, 1 << 20)]
    for _ in range(3):   # pair 2, max-pool at a smaller shape; two block shapes and the vertical baseline
        rows += [(hi, 47000, 512, 131072), (mp, 12000, 256, 1 << 18), (f2, 59000, 896, 1 << 18), (f2, 61000, 1024, 1 << 18),
                 (v2, 64000, 512, 1 << 18)]
    rows += [(mp, 12000, 256, 1 << 18)]   # a trailing native launch goes to the last pair that has the kernel
    p = tmp_path / "x_kernel_trace.csv"
    write_trace(p, rows)
    t = A.exec_time_table(A.load_kernel_trace(str(p)))
    assert set(t) == {"Im2Col+Maxpool", "Hist+Maxpool"}
    assert t["Im2Col+Maxpool"]["ST"] == pytest.approx(78.0) and t["Im2Col+Maxpool"]["HF@768"] == pytest.approx(72.0)
    assert t["Im2Col+Maxpool"]["Maxpool"] == pytest.approx(31.0)
    h = t["Hist+Maxpool"]
    assert h["ST"] == pytest.approx(59.0) and h["HF@896"] == pytest.approx(59.0) and h["HF@1024"] == pytest.approx(61.0)
    assert h["VF@512"] == pytest.approx(64.0) and h["Maxpool"] == pytest.approx(12.0)
    md = A.render_exec_table(t)
    assert "| Im2Col+Maxpool | 78.00 | * | 72.00 | * | * | HF@768 | +8.3 |" in md
    assert "| Hist+Maxpool | 59.00 | 64.00 | * | 59.00 | 61.00 | HF@896 | +0.0 |" in md
    assert "\\textcolor{green}{8.3}" in A.render_exec_table(t, "latex")
    assert A.main(["--trace", str(p), "--format", "json"]) == 0


def test_metric_table(tmp_path):
    cols = ["Dispatch_Id", "Kernel_Name", "Workgroup_Size", "Grid_Size", "VGPR_Count", "Counter_Name", "Counter_Value"]
    sha = N.format(b="Sha256dBody")
    fused = F.format(a="Sha256dBody", b="Blake2bBody<4, false>", m="false")
    p = tmp_path / "s_counter_collection.csv"
    with open(p, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=cols, quoting=csv.QUOTE_NONNUMERIC)
        w.writeheader()
        for d in range(3):
            for name, block, vals in ((sha, 128, {"GRBM_GUI_ACTIVE": 8000.0, "SQ_ACTIVE_INST_VALU": 253440.0,
                                                   "SQ_WAVE_CYCLES": 1474560.0, "SQ_WAIT_INST_ANY": 147456.0, "SQ_WAVES": 4096.0}),
                                      (fused, 256, {"GRBM_GUI_ACTIVE": 16000.0, "SQ_ACTIVE_INST_VALU": 256000.0,
                                                    "SQ_WAVE_CYCLES": 1638400.0, "SQ_WAVES": 8192.0})):
                for c, v in vals.items():
                    w.writerow({"Dispatch_Id": d, "Kernel_Name": name, "Workgroup_Size": block, "Grid_Size": 1 << 20,
                                "VGPR_Count": 64, "Counter_Name": c, "Counter_Value": v})
    rows = A.metric_table(A.load_counters([str(p)]))
    assert [(n, t) for n, t, _ in rows] == [("SHA256", "ST"), ("SHA256+Blake2B", "HF@256")]
    m = rows[0][2]
    # busy cycles per XCD = 8000 / 8 = 1000: 253440 / 256 CUs / 1000 = 99 %; 4 * 1474560 / 1000 / 256 / 32 = 72 %
    assert m["valu_busy_pct"] == pytest.approx(99.0) and m["occupancy_pct"] == pytest.approx(72.0)
    assert m["wait_issue_pct"] == pytest.approx(10.0) and m["waves"] == 4096
    assert rows[1][2]["valu_busy_pct"] == pytest.approx(50.0) and "wait_issue_pct" not in rows[1][2]
    md = A.render_metric_table(rows)
    assert "| SHA256 | ST | 99.0 | 10.0 | 72.0 | 4096 |" in md and "| SHA256+Blake2B | HF@256 | 50.0 | * | 40.0 | 8192 |" in md
    assert A.agent_shape(str(p)) == (256, 8)   # no agent_info.csv beside it: MI355X
    # the same kernel at a second grid size gets its own row, labelled with the grid
    with open(p, "a", newline="") as f:
        w = csv.DictWriter(f, fieldnames=cols, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow({"Dispatch_Id": 9, "Kernel_Name": sha, "Workgroup_Size": 128, "Grid_Size": 1 << 10, "VGPR_Count": 64,
                    "Counter_Name": "SQ_WAVES", "Counter_Value": 16.0})
    labels = [(n, t) for n, t, _ in A.metric_table(A.load_counters([str(p)]))]
    assert labels == [("SHA256", "ST grid 1024"), ("SHA256", "ST grid 1048576"), ("SHA256+Blake2B", "HF@256")]


def test_lds_metrics():
    m = A.derived_metrics({"GRBM_GUI_ACTIVE": 8 * 1000.0, "SQ_LDS_IDX_ACTIVE": 256 * 250.0, "SQ_LDS_BANK_CONFLICT": 256 * 100.0,
                           "SQ_INSTS_LDS": 4096.0})
    assert m["lds_busy_pct"] == pytest.approx(25.0) and m["lds_conflict_pct"] == pytest.approx(40.0) and m["lds_insts"] == 4096.0
    assert "lds_busy_pct" not in A.derived_metrics({"GRBM_GUI_ACTIVE": 8000.0})
