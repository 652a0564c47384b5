"""Split tuner: the reference's preset x split sweep as a launcher mode.

The reference generates one fused kernel per split of the enumeration 128*(n+1) < d1+d2
(tools/llvm-smart-fuser/main.cpp:215-236), builds and profiles each, and keeps the fastest.
Here every split is a launch-time choice of the same compiled kernel, so the sweep is a loop of
timed launches: block shapes (threads of kernel 1, threads of kernel 2) in wavefront multiples,
wave lending on and off, and the barrier modes legal for the pair.  The reference prints its vertical
presets next to the horizontal ones and the user keeps whichever profiles fastest (main.cpp:182-193), so
the sweep also times the vertical kernel: the threads that run each body and the workgroups each body
strides over (a few resident blocks whose threads take the two kernels' work in turn).  The winner is
written back into the fusion list as the `Split:` / `Threads:` / `Lending:` / `Barrier:` / `LaunchBound:`
keys the library applies when a plan is created with the table split, and, where a vertical form wins,
`Preset: vfuse` with its `Blocks:` and `Grids:` (the entry keeps the keys of its best thread partition too).

The register-cap half of the reference's experiments (its *_lb presets, `Reg` bound per
kernel): a gfx950 kernel's VGPR budget is fixed at compile time, so the library carries two
builds of every fused kernel, plain and bounded to 8 waves per SIMD, and the sweep times the
finalists in both.  How many blocks share a CU is the `grids` dimension of the sweep (blocks
per CU for each half of the fused grid).

    python -m hfuse_amd.tuner --out tuned_fusion.yaml            # all shipped tensor pairs
    python -m hfuse_amd.tuner --only Im2ColMaxPool,SummaryMaxpool --out tuned.yaml
"""
from __future__ import annotations

import argparse
import os
import re
import statistics
import sys
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

from . import _lib as L
from . import launcher as H

WAVE = 64
MAX_TENSOR_BLOCK = 1024
MAX_SEARCH_BLOCK = 512


@dataclass
class Candidate:
    threads1: int
    threads2: int
    lending: bool = True
    barrier_mode: Optional[int] = None   # None: the library's choice for the pair
    grids: Tuple[int, int] = (0, 0)      # (0, 0): the library's grids
    bounded: bool = False                # the register-bounded build (the reference's *_lb presets)
    preset: str = "hfuse"                # "vfuse": both bodies from thread 0, threads1 / threads2 run each

    @property
    def vertical(self) -> bool:
        return self.preset.startswith("vfuse")

    def label(self) -> str:
        s = f"{self.threads1}+{self.threads2}" if not self.vertical else f"vfuse {self.threads1}|{self.threads2}"
        if not self.lending:
            s += " nolend"
        if self.barrier_mode is not None:
            s += f" {BARRIER_NAMES[self.barrier_mode]}"
        if self.grids != (0, 0):
            s += f" grids{self.grids[0]}x{self.grids[1]}"
        if self.bounded:
            s += " lb"
        return s


@dataclass
class TuneResult:
    file: str
    kernels: Tuple[str, str]
    best: Candidate
    t_best_ms: float
    t_table_ms: float                 # the untuned table split of the kernel table
    t_b2b_ms: float                   # the two native launches back to back
    table: List[Tuple[str, float]] = field(default_factory=list)   # (candidate label, ms) of the whole sweep
    best_partition: Optional[Candidate] = None   # the fastest thread partition (== best unless a vertical form won)
    t_partition_ms: float = float("nan")

    @property
    def speedup_pct(self) -> float:
        return (self.t_b2b_ms / self.t_best_ms - 1.0) * 100.0


def block_candidates(cfg: H.Config, fusion_index: int, max_block: Optional[int] = None,
                     step: int = WAVE) -> List[Tuple[int, int]]:
    """Every (threads1, threads2) the pair can run with: positive multiples of `step` (itself a
    multiple of the 64-lane wavefront) that divide by each kernel's BlockDim.Y, total <= max_block
    (1024 for tensor pairs, 512 for the searches).  The reference's enumeration
    (128, 256, ... of a fixed total) is the subset with threads1 + threads2 = d1 + d2."""
    if step % WAVE:
        raise ValueError("step must be a multiple of the 64-lane wavefront")
    _, k1, k2 = cfg.fusion(fusion_index)
    r1, r2 = cfg.kernel(k1), cfg.kernel(k2)
    if max_block is None:
        max_block = MAX_SEARCH_BLOCK if k1 in SEARCH_NAMES or k2 in SEARCH_NAMES else MAX_TENSOR_BLOCK
    y1, y2 = r1.block_dim.y, r2.block_dim.y
    out = []
    for t1 in range(step, max_block, step):
        if t1 % y1:
            continue
        for t2 in range(step, max_block - t1 + 1, step):
            if t2 % y2 == 0:
                out.append((t1, t2))
    return out


SEARCH_NAMES = {"ethash_search", "ethash_search2", "ethash_search3", "ethash_search4",
                "sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash", "blake2b_gpu_hash"}


def _make_plan(cfg: H.Config, fusion_index: int, c: Candidate) -> H.Plan:
    plan = cfg.plan(fusion_index, c.preset, L.HF_SPLIT_TABLE)
    plan.set_block(c.threads1, c.threads2)
    if not c.vertical:
        plan.set_lending(c.lending)
        if c.barrier_mode is not None:
            plan.set_barrier_mode(c.barrier_mode)
    plan.set_grids(*c.grids)
    plan.set_launch_bound(c.bounded)
    return plan


def vertical_candidates(cfg: H.Config, fusion_index: int, cus: int, max_block: int = MAX_TENSOR_BLOCK) -> List[Candidate]:
    """Vertical forms of a pair: the same threads run both bodies, in blocks of 512 to 1024 threads, with the
    library's own grids (every thread one or two items) and with one or two resident blocks per CU whose
    threads stride over each kernel's work."""
    _, k1, k2 = cfg.fusion(fusion_index)
    y1, y2 = cfg.kernel(k1).block_dim.y, cfg.kernel(k2).block_dim.y
    out = []
    for t in (512, 768, 1024):
        if t > max_block or t % y1 or t % y2:
            continue
        for per_cu in (0, 1, 2):
            if per_cu * t > 2048:
                continue
            out.append(Candidate(t, t, grids=(per_cu * cus, per_cu * cus), preset="vfuse"))
        out.append(Candidate(t, t, grids=(cus, 0), preset="vfuse"))   # kernel 1 on resident blocks, kernel 2 one item a thread
        out.append(Candidate(t, t, grids=(0, cus), preset="vfuse"))
    return out


def tune(cfg: H.Config, fusion_index: int, args1: Sequence, args2: Sequence, *,
         blocks: Optional[Sequence[Tuple[int, int]]] = None, lending: Sequence[bool] = (True, False),
         barrier_modes: Sequence[Optional[int]] = (None,), grids: Sequence[Tuple[int, int]] = ((0, 0),),
         probe_iters: int = 20, final_iters: int = 100, finalists: int = 4, warmup: int = 3,
         grid_blocks=0, launch_bound: bool = True, verbose: bool = False,
         rotation: Optional[H.Rotation] = None, extra: Sequence[Candidate] = ()) -> TuneResult:
    """Sweep the candidates of one pair on the caller's argument sets and return the fastest.

    args1[i] / args2[i] are argument structs of independent buffer sets the timed launches rotate
    through (hf_time_pair); every call continues the rotation where the last one stopped, so even a
    20-launch probe reads buffers that have left the memory-side cache.  Every candidate gets `probe_iters` launches; the `finalists` fastest
    are timed again over `final_iters` launches in three interleaved rounds, together with the
    back-to-back native launches and the untuned table split, and the median decides.  With
    `launch_bound` each finalist also runs in the register-bounded build.

    `grid_blocks` is the launch grid (0: the library's) or a function (threads1, threads2) -> grid
    for kernels whose grid fixes their work: Ethash scans grid * its-threads nonces, so a fair
    sweep gives every block shape the grid that covers the same nonce range."""
    grid_of = grid_blocks if callable(grid_blocks) else (lambda t1, t2: grid_blocks)
    if rotation is None:
        rotation = H.Rotation()   # one cursor for the whole sweep: short calls keep walking all buffer sets
    file, k1, k2 = cfg.fusion(fusion_index)
    if blocks is None:
        blocks = block_candidates(cfg, fusion_index, step=2 * WAVE)
    cands = [Candidate(t1, t2, ln, bm, g) for (t1, t2) in blocks for ln in lending for bm in barrier_modes
             for g in grids] + list(extra)
    probed = []
    for c in cands:
        try:
            plan = _make_plan(cfg, fusion_index, c)
        except H.HfuseError:
            continue   # not legal for this pair (BlockDim.Y, barrier mode, block cap)
        t = plan.time(3, args1, args2, warmup, probe_iters, grid_of(c.threads1, c.threads2), rotation=rotation) / probe_iters
        probed.append((t, c, plan))
        if verbose:
            print(f"  {c.label():28s} {t * 1e3:9.2f} us", file=sys.stderr, flush=True)
    if not probed:
        raise RuntimeError(f"no legal candidate for {k1} + {k2}")
    probed.sort(key=lambda r: r[0])
    final = probed[:max(1, finalists)]
    if all(c.vertical for _, c, _ in final):      # keep the fastest thread partitions in the final as well
        final += [r for r in probed if not r[1].vertical][:2]
    if launch_bound:
        import dataclasses
        for t, c, _ in list(final):
            twin = dataclasses.replace(c, bounded=True)
            final.append((t, twin, _make_plan(cfg, fusion_index, twin)))
    # Untuned reference point: the kernel table's own split, whatever the fusion entry says.
    base_cfg_plan = cfg.plan(fusion_index, "hfuse", 0)
    d1 = cfg.kernel(k1).block_dim
    d2 = cfg.kernel(k2).block_dim
    base1, base2 = d1.x * d1.y * d1.z, d2.x * d2.y * d2.z
    try:
        base_cfg_plan.set_block(base1, base2)
        base_ok = True
    except H.HfuseError:
        base_ok = False
    samples = {i: [] for i in range(len(final))}
    s_b2b, s_table = [], []
    for _ in range(3):
        for i, (_, _, plan) in enumerate(final):
            samples[i].append(plan.time(3, args1, args2, 2, final_iters, grid_of(final[i][1].threads1, final[i][1].threads2),
                                        rotation=rotation) / final_iters)
        s_b2b.append(final[0][2].time(2, args1, args2, 2, final_iters, grid_of(base1, base2), rotation=rotation) / final_iters)
        if base_ok:
            s_table.append(base_cfg_plan.time(3, args1, args2, 2, final_iters, grid_of(base1, base2), rotation=rotation) / final_iters)
    med = sorted(((statistics.median(v), i) for i, v in samples.items()))
    # Timings this close are the same speed: among them prefer the library's defaults
    # (lending on, the pair's own barrier design) so that noise does not write keys.
    near = [(t, i) for t, i in med if t <= med[0][0] * 1.005]
    t_best, ibest = min(near, key=lambda r: ((not final[r[1]][1].lending) + (final[r[1]][1].barrier_mode is not None)
                                             + final[r[1]][1].bounded, r[0]))
    parts = [(t, i) for t, i in med if not final[i][1].vertical]
    return TuneResult(file=file, kernels=(k1, k2), best=final[ibest][1], t_best_ms=t_best,
                      t_table_ms=statistics.median(s_table) if s_table else float("nan"),
                      t_b2b_ms=statistics.median(s_b2b),
                      table=[(c.label(), t) for t, c, _ in probed] +
                            [(final[i][1].label(), t) for t, i in med if final[i][1].bounded],
                      best_partition=final[parts[0][1]][1] if parts else None,
                      t_partition_ms=parts[0][0] if parts else float("nan"))


# ------------------------------------------------------------------ three-kernel entries
def triple_block_candidates(cfg: H.Config, fusion_index: int, max_block: int, step: int = WAVE) -> List[Tuple[int, int, int]]:
    """Every (threads0, threads1, threads2) a three-kernel entry can run with: positive multiples of `step`
    that divide by each kernel's BlockDim.Y, total <= max_block."""
    ys = [cfg.kernel(k).block_dim.y for k in cfg.fusion_kernels(fusion_index)]
    out = []
    for t0 in range(step, max_block, step):
        for t1 in range(step, max_block - t0, step):
            for t2 in range(step, max_block - t0 - t1 + 1, step):
                if t0 % ys[0] == 0 and t1 % ys[1] == 0 and t2 % ys[2] == 0:
                    out.append((t0, t1, t2))
    return out


def tune_triple(cfg: H.Config, fusion_index: int, time_fused, blocks: Sequence[Tuple[int, int, int]], *,
                finalists: int = 4, verbose: bool = False):
    """Sweep the block shapes of a three-kernel entry.  `time_fused(plan)` returns milliseconds per launch of
    the plan on the caller's workload.  -> (best shape, its time, [(shape, ms), ...] of the whole sweep); the
    `finalists` fastest are timed three more times and the median decides."""
    probed = []
    for shape in blocks:
        plan = cfg.plan(fusion_index)
        try:
            plan.set_block_n(*shape)
        except H.HfuseError:
            continue
        t = time_fused(plan)
        probed.append((t, shape, plan))
        if verbose:
            print(f"  {'+'.join(map(str, shape)):16s} {t * 1e3:9.2f} us", file=sys.stderr, flush=True)
    if not probed:
        raise RuntimeError("no legal block shape")
    probed.sort(key=lambda r: r[0])
    final = probed[:max(1, finalists)]
    med = sorted((statistics.median([time_fused(plan) for _ in range(3)]), shape) for _, shape, plan in final)
    return med[0][1], med[0][0], [(shape, t) for t, shape, _ in probed]


def apply_blocks_to_fusion_yaml(text: str, shapes: dict) -> str:
    """Return the fusion list `text` with `Blocks:` of the entries in `shapes` {entry index: (t0, t1, t2)}
    replaced (or added); every other line is kept."""
    lines = text.splitlines()
    starts = [i for i, ln in enumerate(lines) if ln.startswith("- ")] + [len(lines)]
    out: List[str] = lines[:starts[0]] if starts else list(lines)
    for n in range(len(starts) - 1):
        entry = lines[starts[n]:starts[n + 1]]
        if n in shapes:
            kept, skipping = [], False
            for ln in entry:
                if re.match(r"^\s+Blocks\s*:", ln):
                    skipping = True
                    continue
                if skipping and re.match(r"^\s+-\s+\d+\s*$", ln):
                    continue
                skipping = False
                kept.append(ln)
            tail = []
            while kept and (not kept[-1].strip() or kept[-1].lstrip().startswith("#")):
                tail.insert(0, kept.pop())
            kept.append("  Blocks:")
            kept.extend(f"    - {t}" for t in shapes[n])
            entry = kept + tail
        out.extend(entry)
    return "\n".join(out) + "\n"


def tune_shipped_triples(out_path: str, verbose: bool = False, search_log2=(26, 26, 24)) -> int:
    """Tune the block shapes of the shipped three-kernel list on the benchmark workloads and write it to `out_path`."""
    import torch
    from . import workloads as W
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "configs")
    path = os.path.join(here, "gfx950_triples.yaml")
    text = open(path).read()
    cfg = H.Config(text, open(os.path.join(here, "gfx950_kernels.yaml")).read())
    shapes = {}
    for i in range(cfg.num_fusions):
        names = cfg.fusion_kernels(i)
        if len(names) != 3:
            continue
        print(f"[{i}] {' + '.join(names)}", file=sys.stderr, flush=True)
        if all(k in W.TENSOR_KERNELS for k in names):
            work = W.TensorTriple(names)
            n = len(work.sets)
            time_fused = lambda plan: work.time(plan, 3, 2, n) / n
            blocks = triple_block_candidates(cfg, i, MAX_TENSOR_BLOCK, 2 * WAVE)
            base = cfg.plan(i, "vfuse")
            t_b2b = statistics.median([work.time(base, 2, 2, n) / n for _ in range(3)])
        elif tuple(names) == W.SearchTriple.KERNELS:
            work = W.SearchTriple(search_log2)
            time_fused = lambda plan: work.time(plan, 3)
            blocks = triple_block_candidates(cfg, i, MAX_SEARCH_BLOCK, WAVE)
            t_b2b = statistics.median([work.time(cfg.plan(i, "vfuse"), 2) for _ in range(3)])
        else:
            continue
        best, t_best, table = tune_triple(cfg, i, time_fused, blocks, verbose=verbose)
        shapes[i] = best
        print(f"    best {'+'.join(map(str, best))}: {t_best * 1e3:.2f} us, three natives back to back {t_b2b * 1e3:.2f} us "
              f"({(t_b2b / t_best - 1) * 100:+.1f} %)", file=sys.stderr, flush=True)
        del work
        torch.cuda.empty_cache()
    with open(out_path, "w") as f:
        f.write(apply_blocks_to_fusion_yaml(text, shapes))
    print(f"wrote {out_path} ({len(shapes)} entries tuned)", file=sys.stderr)
    return 0


# ------------------------------------------------------------------ fusion list rewriting
_TUNED_KEY = re.compile(r"^\s+(Split|Threads|Lending|Barrier|LaunchBound|Preset|Grids|Blocks)\s*:")
BARRIER_NAMES = {L.HF_BARRIER_NONE: "none", L.HF_BARRIER_MATCHED: "matched", L.HF_BARRIER_SUBSET: "subset",
                 L.HF_BARRIER_BLOCKIDX: "blockidx"}


def apply_to_fusion_yaml(text: str, tuned: dict) -> str:
    """Return the fusion list `text` with the tuned keys of `tuned` {entry index: Candidate or None}
    written into those entries; comments and every other line are kept.  None removes an entry's
    tuned keys (the pair then runs at the kernel table's block shapes)."""
    lines = text.splitlines()
    starts = [i for i, ln in enumerate(lines) if ln.startswith("- ")]
    out: List[str] = []
    for n, s in enumerate(starts):
        if n == 0:
            out.extend(lines[:s])
        e = starts[n + 1] if n + 1 < len(starts) else len(lines)
        entry = lines[s:e]
        if n in tuned:
            entry = [ln for ln in entry if not _TUNED_KEY.match(ln)]
            # keep trailing comments / blank lines (they belong to the next entry) after the new keys
            tail = []
            while entry and (not entry[-1].strip() or entry[-1].lstrip().startswith("#")):
                tail.insert(0, entry.pop())
            c = tuned[n]
            part = c[1] if isinstance(c, tuple) else c      # (winner, best thread partition) or one candidate
            c = c[0] if isinstance(c, tuple) else c
            if part is not None and not part.vertical:
                entry.append(f"  Split: {part.threads1}")
                entry.append(f"  Threads: {part.threads1 + part.threads2}")
                if not part.lending:
                    entry.append("  Lending: false")
                if part.barrier_mode is not None:
                    entry.append(f"  Barrier: {BARRIER_NAMES[part.barrier_mode]}")
                if part.bounded:
                    entry.append("  LaunchBound: true")
            if c is not None and c.vertical:
                entry.append(f"  Preset: {c.preset}{'_lb' if c.bounded else ''}")
                entry.append(f"  Blocks: [{c.threads1}, {c.threads2}]")
            if c is not None and c.grids != (0, 0):
                entry.append(f"  Grids: [{c.grids[0]}, {c.grids[1]}]")
            entry.extend(tail)
        out.extend(entry)
    if not starts:
        out = lines
    return "\n".join(out) + "\n"


# ------------------------------------------------------------------ command line
def _default_paths():
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "configs")
    return os.path.join(here, "gfx950_fusion.yaml"), os.path.join(here, "gfx950_kernels.yaml")


def main(argv=None) -> int:
    fusion_default, kernels_default = _default_paths()
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--fusion", default=fusion_default, help="fusion list (YAML)")
    ap.add_argument("--kernels", default=kernels_default, help="kernel table (YAML)")
    ap.add_argument("--out", required=True, help="where to write the tuned fusion list")
    ap.add_argument("--only", default="", help="comma list of File names or k1+k2 to tune (default: every tensor pair)")
    ap.add_argument("--searches", action="store_true", help="also tune the nonce-search pairs (allocates a 4 GiB DAG)")
    ap.add_argument("--search-log2", type=int, default=24, help="log2 of the nonce range of a search launch while tuning")
    ap.add_argument("--search-log2-second", type=int, default=None,
                    help="log2 of the second kernel's nonce range (default: the same as --search-log2); the benchmark's "
                         "Ethash + Blake2b pair runs 2^28 against 2^30 nonces, i.e. a difference of 2")
    ap.add_argument("--step", type=int, default=64, help="granule of the block-shape sweep in threads")
    ap.add_argument("--min-gain", type=float, default=1.0,
                    help="keep an entry's current keys unless the winner beats the table split by this many percent")
    ap.add_argument("--blockidx", action="store_true",
                    help="also try the block-index partition (each workgroup runs one of the two kernels), "
                         "written as 'Barrier: blockidx' where it wins")
    ap.add_argument("--vertical", action="store_true",
                    help="also try the vertical kernel (the reference's vfuse preset) in blocks of 512-1024 threads, with the "
                         "library's grids and with one or two resident blocks per CU; written as 'Preset: vfuse' where it wins")
    ap.add_argument("--verbose", action="store_true")
    ap.add_argument("--triples", action="store_true",
                    help="tune the block shapes (`Blocks:`) of the shipped three-kernel list instead of the pairs")
    args = ap.parse_args(argv)
    if args.triples:
        return tune_shipped_triples(args.out, args.verbose)

    import torch
    from . import workloads as W
    if not torch.cuda.is_available():
        print("hfuse_amd.tuner: no GPU", file=sys.stderr)
        return 2
    text = open(args.fusion).read()
    # Measure on the list without anybody's tuned keys, so that "the table split" and every
    # candidate start from the library's defaults; the keys of entries that are not re-tuned
    # are kept in the output, which is written from the original text.
    entries = sum(1 for ln in text.splitlines() if ln.startswith("- "))
    cfg = H.Config(apply_to_fusion_yaml(text, {n: None for n in range(entries)}), open(args.kernels).read())
    only = {s for s in args.only.split(",") if s}
    tuned = {}
    seen = set()
    for i, (file, k1, k2) in enumerate(cfg.fusions()):
        if only and file not in only and f"{k1}+{k2}" not in only:
            continue
        if (k1, k2) in seen:
            continue
        tensor = k1 in W.TENSOR_KERNELS and k2 in W.TENSOR_KERNELS
        search = k1 in W.SEARCH_KERNELS and k2 in W.SEARCH_KERNELS
        if not tensor and not (search and args.searches):
            continue
        seen.add((k1, k2))
        print(f"[{i}] {file}: {k1} + {k2}", file=sys.stderr, flush=True)
        blocks = block_candidates(cfg, i, step=args.step)
        if tensor:
            bench_variant = {v[:2]: v[2:] for v in W.BENCH_TENSOR_PAIRS.values()}.get((k1, k2), ("", ""))
            pair = W.build_pair(file, k1, k2, *bench_variant)
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            r = tune(cfg, i, pair.args1, pair.args2, blocks=blocks,
                     barrier_modes=(None, L.HF_BARRIER_BLOCKIDX) if args.blockidx else (None,), verbose=args.verbose,
                     extra=vertical_candidates(cfg, i, cus) if args.vertical else (), rotation=pair.rotation)
            del pair
        else:
            sp = W.SearchPair(k1, k2, args.search_log2,
                              args.search_log2 if args.search_log2_second is None else args.search_log2_second)
            _, _, a1, a2 = sp.fresh()
            # ethash scans grid * its-threads nonces: every block shape gets the grid for the same range
            eth = 0 if k1 == "ethash_search" else 1 if k2 == "ethash_search" else None
            grid = (lambda t1, t2: sp.nonces[eth] // (t1, t2)[eth]) if eth is not None else 0
            vertical = [Candidate(t, t, preset="vfuse") for t in (64, 128, 256)] if args.vertical else []
            r = tune(cfg, i, [a1], [a2], blocks=blocks, lending=(True,), probe_iters=1, final_iters=2,
                     warmup=0, grid_blocks=grid, verbose=args.verbose, extra=vertical,
                     barrier_modes=(None, L.HF_BARRIER_BLOCKIDX) if args.blockidx else (None,))
            del sp
        torch.cuda.empty_cache()
        gain = (r.t_table_ms / r.t_best_ms - 1.0) * 100.0 if r.t_table_ms == r.t_table_ms else float("inf")
        keep = gain >= args.min_gain
        print(f"    best {r.best.label()}: {r.t_best_ms * 1e3:.2f} us, table split {r.t_table_ms * 1e3:.2f} us, "
              f"back to back {r.t_b2b_ms * 1e3:.2f} us ({r.speedup_pct:+.1f} %)"
              f"{'' if keep else ' -- within noise of the table split, keys left out'}", file=sys.stderr, flush=True)
        # the same pair may be listed more than once (the reference's lists repeat pairs): tune once, write all
        for j, (_, a, b) in enumerate(cfg.fusions()):
            if (a, b) == (k1, k2):
                tuned[j] = (r.best, r.best_partition) if keep else None
    with open(args.out, "w") as f:
        f.write(apply_to_fusion_yaml(text, tuned))
    print(f"wrote {args.out} ({len(tuned)} entries tuned)", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
