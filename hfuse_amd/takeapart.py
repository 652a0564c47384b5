"""Take a fused tensor pair apart: where its time goes.

Times, on the benchmark's rotating buffer sets, the two native kernels, their back-to-back launch, the form the
fusion list ships for the pair, its thread partition, and each kernel alone inside the fused kernel (its partner
given an empty tensor), and prints one JSON row.  Run once with the product library and once per timing-only build
of `make -C hfuse_amd/csrc takeapart` (the library with one part of a kernel switched off: max-pooling 2x2 without
its stores / its loads, the histogram without its LDS atomics / its loads), the rows make the take-apart table:

    python -m hfuse_amd.takeapart histc_maxpool
    HFUSE_LIB=hfuse_amd/takeapart/libhfuse_ta4.so python -m hfuse_amd.takeapart histc_maxpool

The timing-only builds compute wrong results on purpose; nothing here checks outputs (bench.py and the tests do,
with the product library).
"""
from __future__ import annotations

import json
import os
import statistics
import sys


def tiny_partner_args(kname):
    """Argument list of `kname` over a tensor so small that its half has (next to) nothing to do."""
    import torch
    from . import launcher as H
    if kname == "MaxPoolForward":
        y = torch.zeros((1, 1, 2, 4), device="cuda")
        val = torch.empty((1, 1, 1, 2), device="cuda")
        idx = torch.empty((1, 1, 1, 2), dtype=torch.int64, device="cuda")
        return (y, val, idx), H.maxpool_args(y, val, idx, (2, 2), (2, 2), (0, 0))
    if kname == "kernelHistogram1D":
        x = torch.zeros(4, device="cuda")
        hist = torch.zeros(1024, device="cuda")
        return (x, hist), H.histc_args(x, hist, 1024, 0.0, 1.0)
    raise KeyError(kname)


def run(name: str, rounds: int = 5, rotations: int = 2) -> dict:
    import torch
    import hfuse_amd
    from . import _lib as L
    from . import workloads as W
    cfg = hfuse_amd.default_config()
    pair = W.build_tensor_pairs([name])[name]
    i = cfg.find_fusion(pair.k1, pair.k2)
    nsets = len(pair.sets)
    per = rotations * nsets
    keep1, tiny1 = tiny_partner_args(pair.k1)
    keep2, tiny2 = tiny_partner_args(pair.k2)
    shipped, part = cfg.plan(i, "shipped"), cfg.plan(i, "hfuse")
    rot = pair.rotation

    def timed(plan, mode, a1, a2):
        return plan.time(mode, a1, a2, 2, per, rotation=rot) / per

    full1, full2 = pair.args1, pair.args2
    e1, e2 = [tiny1] * nsets, [tiny2] * nsets
    runs = [("native_a", shipped, 0, full1, full2), ("native_b", shipped, 1, full1, full2),
            ("back_to_back", shipped, 2, full1, full2), ("shipped", shipped, 3, full1, full2),
            ("partition", part, 3, full1, full2),
            ("shipped_a_alone", shipped, 3, full1, e2), ("shipped_b_alone", shipped, 3, e1, full2),
            ("partition_a_alone", part, 3, full1, e2), ("partition_b_alone", part, 3, e1, full2)]
    for _, p, m, a1, a2 in runs:
        p.time(m, a1, a2, 0, nsets, rotation=rot)
    samples = {k: [] for k, *_ in runs}
    for _ in range(rounds):
        for key, p, m, a1, a2 in runs:
            samples[key].append(timed(p, m, a1, a2))
    torch.cuda.synchronize()
    row = {"pair": name, "library": os.path.basename(L.LIB_PATH),
           "shipped_form": shipped.name, "partition_form": part.name,
           "us": {k: round(statistics.median(v) * 1e3, 2) for k, v in samples.items()},
           "launches_per_sample": per, "rounds": rounds, "buffer_sets": nsets}
    del keep1, keep2
    return row


if __name__ == "__main__":
    print(json.dumps(run(sys.argv[1] if len(sys.argv) > 1 else "histc_maxpool")))
