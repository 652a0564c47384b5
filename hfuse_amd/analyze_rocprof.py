"""Per-pair tables from rocprofv3 output: the counterpart of the reference's nvprof analysis.

The reference reads nvprof's CSV traces, keys every launch by the tag in its kernel name
(`..._fused_kernel_vfuse_idx_0`, `..._hfuse_lb_idx_2`, plain names for the natives), and prints
one table of execution times per pair and tag (ST = the two native kernels, VF, HF, with and
without launch bounds; scripts/analyze_nvprof.py:650-690) and two tables of metrics per kernel
(issue-slot utilisation, memory-dependency stalls, achieved occupancy; :696-827).

rocprofv3 names a launch by its HIP symbol, so the tag comes from the kernel template and the
block shape instead:

    native_kernel<XBody, ...>            ST   one original kernel (native_kernel_capped: the same with its
                                              residency capped, as im2col is launched)
    vertical_kernel<XBody, YBody, ...>   VF   the same threads run both bodies, tagged with the workgroup size
    fused_kernel<XBody, YBody, .., 0>    HF   horizontally fused, tagged with the workgroup size
    fused_kernel<XBody, YBody, .., 1>    HF+M the same with the shared hardware barrier
    blockidx_kernel<XBody, YBody, ...>   BI   block-index partition
    fused_kernel_lb / vertical_kernel_lb HF-LB, HF+M-LB, VF-LB: the register-bounded builds
                                         (the reference's hfuse_lb / vfuse_lb presets)

Input: the `*_kernel_trace.csv` of `rocprofv3 --kernel-trace --output-format csv` and, for the
metric table, any number of `*_counter_collection.csv` files of `rocprofv3 --pmc ...` runs of the
same command (one counter set per run).

    python -m hfuse_amd.analyze_rocprof --trace out/x_kernel_trace.csv \\
        --counters out/sq_counter_collection.csv --format md
"""
from __future__ import annotations

import argparse
import csv
import json
import os
import re
import statistics
import sys
from collections import defaultdict
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Tuple

BODY_TO_KERNEL = {
    "Im2colBody": "im2col_kernel",
    "MaxPoolBody": "MaxPoolForward",
    "BnStatsBody": "batch_norm_collect_statistics_kernel",
    "UpsampleNearestBody": "upsample_nearest2d_out_frame",
    "UpsampleBilinearBody": "upsample_bilinear2d_out_frame",
    "HistcBody": "kernelHistogram1D",
    "EthashBody": "ethash_search",
    "Sha256dBody": "sha256d_gpu_hash_shared",
    "Blake2bBody<4, false>": "sia_blake2b_gpu_hash",
    "Blake2bBody<9, true>": "blake2b_gpu_hash",
}
# Short names for table headers, as the reference abbreviates its kernels.
SHORT = {
    "im2col_kernel": "Im2Col", "MaxPoolForward": "Maxpool", "batch_norm_collect_statistics_kernel": "Batchnorm",
    "upsample_nearest2d_out_frame": "Upsample", "upsample_bilinear2d_out_frame": "UpsampleBilinear",
    "kernelHistogram1D": "Hist", "ethash_search": "Ethash", "sha256d_gpu_hash_shared": "SHA256",
    "sia_blake2b_gpu_hash": "Blake2B", "blake2b_gpu_hash": "Blake2B(cc)",
}
TAG_ORDER = ("ST", "VF", "VF-LB", "HF", "HF-LB", "HF+M", "HF+M-LB", "BI")

_TEMPLATE = re.compile(r"hfuse::(native_kernel_capped|native_kernel|fused_kernel_lb|fused_kernel|vertical_kernel_lb|vertical_kernel|blockidx_kernel)<(.*)>\(")
_BODY = re.compile(r"hfuse::(\w+Body(?:<[^<>]*>)?)")


@dataclass(frozen=True)
class KernelKey:
    tag: str                       # one of TAG_ORDER
    kernels: Tuple[str, ...]       # one YAML kernel name (ST) or two
    block: int                     # workgroup size of the launch

    def label(self) -> str:
        return self.tag if self.tag == "ST" else f"{self.tag}@{self.block}"


def parse_kernel_name(name: str) -> Optional[Tuple[str, Tuple[str, ...]]]:
    """-> (tag, YAML kernel names) for a kernel of this library, None for anything else."""
    m = _TEMPLATE.search(name)
    if not m:
        return None
    kind, params = m.group(1), m.group(2)
    bodies = [BODY_TO_KERNEL.get(b) for b in _BODY.findall(params)]
    if not bodies or any(b is None for b in bodies):
        return None
    if kind in ("native_kernel", "native_kernel_capped"):
        return "ST", (bodies[0],)
    if len(bodies) != 2:
        return None
    lb = "-LB" if kind.endswith("_lb") else ""
    if kind.startswith("vertical_kernel"):
        return "VF" + lb, tuple(bodies)
    if kind == "blockidx_kernel":
        return "BI", tuple(bodies)
    matched = re.search(r",\s*true\b", params) is not None   # fused_kernel<K1, K2, T, MATCHED> / fused_kernel_lb<..., MATCHED, W>
    return ("HF+M" if matched else "HF") + lb, tuple(bodies)


@dataclass
class Dispatch:
    key: KernelKey
    start: int
    end: int
    grid: int
    vgpr: int


def load_kernel_trace(path: str) -> List[Dispatch]:
    out = []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            p = parse_kernel_name(r["Kernel_Name"])
            if p is None:
                continue
            block = int(r["Workgroup_Size_X"]) * int(r.get("Workgroup_Size_Y", 1) or 1) * int(r.get("Workgroup_Size_Z", 1) or 1)
            grid = int(r["Grid_Size_X"]) * int(r.get("Grid_Size_Y", 1) or 1) * int(r.get("Grid_Size_Z", 1) or 1)
            out.append(Dispatch(KernelKey(p[0], p[1], block), int(r["Start_Timestamp"]), int(r["End_Timestamp"]), grid,
                                int(r.get("VGPR_Count", 0) or 0)))
    out.sort(key=lambda d: d.start)
    return out


def assign_natives(dispatches: List[Dispatch]) -> Dict[Tuple[str, str], Dict[str, List[int]]]:
    """Durations (ns) of the native launches that belong to each pair: {pair: {kernel: [ns]}}.

    One trace may hold several pairs that share a native kernel at different shapes.  A benchmark
    times a pair's natives before that pair's fused kernel, so a native launch is credited to the
    next fused launch (any tag) whose pair contains the kernel, or to the previous one at the end."""
    fused = [d for d in dispatches if len(d.key.kernels) == 2]
    res: Dict[Tuple[str, str], Dict[str, List[int]]] = defaultdict(lambda: defaultdict(list))
    for d in dispatches:
        if len(d.key.kernels) != 1:
            continue
        k = d.key.kernels[0]
        nxt = next((f for f in fused if f.start >= d.start and k in f.key.kernels), None)
        if nxt is None:
            nxt = next((f for f in reversed(fused) if k in f.key.kernels), None)
        if nxt is not None:
            res[nxt.key.kernels][k].append(d.end - d.start)
    return res


def exec_time_table(dispatches: List[Dispatch], reducer=statistics.median) -> Dict[str, Dict[str, float]]:
    """{"K1+K2": {"ST": us, "VF": us, "HF@512": us, ...}} -- the reference's table of execution times."""
    natives = assign_natives(dispatches)
    by_key: Dict[KernelKey, List[int]] = defaultdict(list)
    for d in dispatches:
        if len(d.key.kernels) == 2:
            by_key[d.key].append(d.end - d.start)
    table: Dict[str, Dict[str, float]] = {}
    for key, durs in by_key.items():
        name = "+".join(SHORT.get(k, k) for k in key.kernels)
        row = table.setdefault(name, {})
        row[key.label()] = reducer(durs) / 1e3
        nat = natives.get(key.kernels, {})
        if "ST" not in row and all(k in nat for k in set(key.kernels)):
            row["ST"] = sum(reducer(nat[k]) for k in key.kernels) / 1e3
            for k in set(key.kernels):
                row[SHORT.get(k, k)] = reducer(nat[k]) / 1e3
    return table


def load_counters(paths: Iterable[str]) -> Dict[Tuple[KernelKey, int], Dict[str, float]]:
    """Median per dispatch of every counter, per kernel, block shape and grid size (one kernel
    launched at two shapes, such as max-pool in two pairs, gives two rows)."""
    acc: Dict[Tuple[KernelKey, int], Dict[str, List[float]]] = defaultdict(lambda: defaultdict(list))
    for path in paths:
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                p = parse_kernel_name(r["Kernel_Name"])
                if p is None:
                    continue
                key = (KernelKey(p[0], p[1], int(r["Workgroup_Size"])), int(r.get("Grid_Size", 0) or 0))
                acc[key][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return {k: {c: statistics.median(v) for c, v in cs.items()} for k, cs in acc.items()}


def agent_shape(path: str) -> Tuple[int, int]:
    """(CUs, XCDs) of the GPU from the `*_agent_info.csv` next to a rocprofv3 output file; MI355X if absent."""
    d = os.path.dirname(path)
    for fn in sorted(os.listdir(d or ".")):
        if fn.endswith("agent_info.csv"):
            with open(os.path.join(d, fn), newline="") as f:
                for r in csv.DictReader(f):
                    if r.get("Agent_Type") == "GPU":
                        return int(r["Cu_Count"]), int(r["Num_Xcc"])
    return 256, 8


def derived_metrics(c: Dict[str, float], cus: int = 256, xcds: int = 8) -> Dict[str, float]:
    """The analogues of the reference's three nvprof metrics, from whatever counters are there.

    GRBM_GUI_ACTIVE comes back summed over the XCDs; per-XCD busy cycles are its share.
      valu_busy_pct   (issue_slot_utilization)   100 * SQ_ACTIVE_INST_VALU / CUs / busy
      mem_stalled_pct (stall_memory_dependency)  rocprofv3's own derived MemUnitStalled, when collected
      wait_issue_pct  (no nvprof counterpart)    100 * SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES: wave-cycles spent
                      waiting for an earlier instruction of any kind, other waves' turns on the SIMD included
      occupancy_pct   (achieved_occupancy)       100 * 4 * SQ_WAVE_CYCLES / busy / CUs / 32 wave slots
      lds_busy_pct    (no nvprof counterpart)    100 * SQ_LDS_IDX_ACTIVE / CUs / busy (rocprofv3's LdsUtil)
      lds_conflict_pct                           100 * SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE: share of the
                      LDS's active cycles lost to bank conflicts (the histogram's atomics on random bins)"""
    out: Dict[str, float] = {}
    busy = c.get("GRBM_GUI_ACTIVE", 0.0) / xcds
    if busy > 0 and "SQ_ACTIVE_INST_VALU" in c:
        out["valu_busy_pct"] = 100.0 * c["SQ_ACTIVE_INST_VALU"] / cus / busy
    if busy > 0 and "SQ_WAVE_CYCLES" in c:
        out["occupancy_pct"] = 400.0 * c["SQ_WAVE_CYCLES"] / busy / cus / 32
    if c.get("SQ_WAVE_CYCLES", 0.0) > 0 and "SQ_WAIT_INST_ANY" in c:
        out["wait_issue_pct"] = 100.0 * c["SQ_WAIT_INST_ANY"] / c["SQ_WAVE_CYCLES"]
    if "MemUnitStalled" in c:
        out["mem_stalled_pct"] = c["MemUnitStalled"]
    if busy > 0 and "SQ_LDS_IDX_ACTIVE" in c:
        out["lds_busy_pct"] = 100.0 * c["SQ_LDS_IDX_ACTIVE"] / cus / busy
    if c.get("SQ_LDS_IDX_ACTIVE", 0.0) > 0 and "SQ_LDS_BANK_CONFLICT" in c:
        out["lds_conflict_pct"] = 100.0 * c["SQ_LDS_BANK_CONFLICT"] / c["SQ_LDS_IDX_ACTIVE"]
    if "SQ_INSTS_LDS" in c:
        out["lds_insts"] = c["SQ_INSTS_LDS"]
    if "SQ_WAVES" in c:
        out["waves"] = c["SQ_WAVES"]
    if "SQ_INSTS_VALU" in c:
        out["valu_insts"] = c["SQ_INSTS_VALU"]
    if "FETCH_SIZE" in c:
        out["fetch_kib"] = c["FETCH_SIZE"]
    if "WRITE_SIZE" in c:
        out["write_kib"] = c["WRITE_SIZE"]
    return out


def metric_table(counters: Dict[Tuple[KernelKey, int], Dict[str, float]], cus: int = 256, xcds: int = 8):
    rows = []
    shapes = defaultdict(set)
    for key, grid in counters:
        shapes[key].add(grid)
    order = sorted(counters, key=lambda kg: (len(kg[0].kernels), kg[0].kernels, TAG_ORDER.index(kg[0].tag), kg[0].block, kg[1]))
    for key, grid in order:
        name = "+".join(SHORT.get(k, k) for k in key.kernels)
        label = key.label() + (f" grid {grid}" if len(shapes[key]) > 1 else "")   # grid in work-items, as rocprofv3 reports it
        rows.append((name, label, derived_metrics(counters[(key, grid)], cus, xcds)))
    return rows


# ------------------------------------------------------------------ rendering
def _tag_columns(table) -> List[str]:
    cols = {c for row in table.values() for c in row if c.split("@")[0] in TAG_ORDER}
    return sorted(cols, key=lambda c: (TAG_ORDER.index(c.split("@")[0]), int(c.split("@")[1]) if "@" in c else 0))


def render_exec_table(table, fmt: str = "md") -> str:
    cols = _tag_columns(table)
    if fmt == "json":
        return json.dumps(table, indent=1, sort_keys=True)
    lines = []
    if fmt == "latex":
        lines.append(" & " + " & ".join(cols) + " & best \\\\ \\hline")
    else:
        lines.append("| pair | " + " | ".join(f"{c} us" for c in cols) + " | best | speedup % |")
        lines.append("|---|" + "---:|" * len(cols) + "---|---:|")
    for pair in sorted(table):
        row = table[pair]
        st = row.get("ST")
        fused = {c: row[c] for c in cols if c != "ST" and c in row}
        best = min(fused, key=fused.get) if fused else ""
        gain = (st / fused[best] - 1.0) * 100.0 if st and best else float("nan")
        cells = [f"{row[c]:.2f}" if c in row else "*" for c in cols]
        if fmt == "latex":
            colour = "green" if gain > 0 else "red"
            lines.append(f"{pair} & " + " & ".join(cells) + f" & \\textcolor{{{colour}}}{{{gain:.1f}}} \\\\ \\hline")
        else:
            lines.append(f"| {pair} | " + " | ".join(cells) + f" | {best} | {gain:+.1f} |")
    return "\n".join(lines)


_METRIC_COLS = (("valu_busy_pct", "VALU busy %", "{:.1f}"), ("mem_stalled_pct", "mem unit stalled %", "{:.1f}"),
                ("wait_issue_pct", "waiting on issue %", "{:.1f}"),
                ("occupancy_pct", "occupancy %", "{:.1f}"), ("lds_busy_pct", "LDS busy %", "{:.1f}"),
                ("lds_conflict_pct", "LDS bank conflicts % of LDS cycles", "{:.1f}"), ("lds_insts", "LDS insts", "{:.0f}"),
                ("waves", "waves", "{:.0f}"),
                ("valu_insts", "VALU insts", "{:.0f}"), ("fetch_kib", "FETCH_SIZE KiB", "{:.1f}"),
                ("write_kib", "WRITE_SIZE KiB", "{:.1f}"))


def render_metric_table(rows, fmt: str = "md") -> str:
    if fmt == "json":
        return json.dumps([{"kernel": n, "tag": t, **m} for n, t, m in rows], indent=1)
    have = [c for c in _METRIC_COLS if any(c[0] in m for _, _, m in rows)]
    sep, end = (" & ", " \\\\") if fmt == "latex" else (" | ", " |")
    lines = []
    head = ["kernel", "tag"] + [h for _, h, _ in have]
    if fmt == "latex":
        lines.append(sep.join(head) + end + " \\hline")
    else:
        lines.append("| " + sep.join(head) + end)
        lines.append("|---|---|" + "---:|" * len(have))
    for name, tag, m in rows:
        cells = [name, tag] + [f.format(m[k]) if k in m else "*" for k, _, f in have]
        lines.append(("" if fmt == "latex" else "| ") + sep.join(cells) + end)
    return "\n".join(lines)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Per-pair execution-time and metric tables from rocprofv3 CSV output")
    ap.add_argument("--trace", help="*_kernel_trace.csv of a --kernel-trace run")
    ap.add_argument("--counters", nargs="*", default=[], help="*_counter_collection.csv files of --pmc runs")
    ap.add_argument("--format", choices=("md", "latex", "json"), default="md")
    ap.add_argument("--mean", action="store_true", help="average over launches instead of the median")
    args = ap.parse_args(argv)
    if not args.trace and not args.counters:
        ap.error("give --trace and / or --counters")
    if args.trace:
        table = exec_time_table(load_kernel_trace(args.trace), statistics.fmean if args.mean else statistics.median)
        print(render_exec_table(table, args.format))
    if args.counters:
        cus, xcds = agent_shape(args.counters[0])
        if args.trace:
            print()
        print(render_metric_table(metric_table(load_counters(args.counters), cus, xcds), args.format))
    return 0


if __name__ == "__main__":
    sys.exit(main())
