"""bench.py's command line and bookkeeping, without a GPU: the refusal of more than one GPU, the per-pair
judgement (speedup as the reference defines it, scripts/analyze_nvprof.py:551-552) and the byte / op constants
the roofline figures are computed from."""
import importlib.util
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_defaults_are_one_gpu_and_a_short_run(bench, monkeypatch):
    monkeypatch.setattr(sys, "argv", ["bench.py"])
    args = bench.parse()
    assert args.gpus == 1 and 1 <= args.steps <= 20 and 0 <= args.warmup <= 5


def test_judgement_of_a_pair(bench):
    """`t_fused_ms` is the form the fusion list ships; the thread partition, the vertical kernel and the block-index
    partition are judged next to it."""
    res = {"t_a_ms": 0.047, "t_b_ms": 0.031, "t_b2b_ms": 0.0785, "t_two_streams_ms": 0.074, "t_vfuse_ms": 0.075,
           "t_fused_ms": 0.0707, "t_hfuse_ms": 0.0707, "t_fused_lb_ms": 0.077}
    bench.judge(res)
    assert res["speedup_pct"] == pytest.approx((0.0785 / 0.0707 - 1) * 100)
    assert res["best_mode"] == "hfuse" and res["modes_within_0p5pct_of_best"] == ["hfuse"]
    assert res["hfuse_vs_vfuse_pct"] == pytest.approx((0.075 / 0.0707 - 1) * 100)
    res.update(t_blockidx_ms=0.069)
    bench.judge(res)
    assert res["best_mode"] == "blockidx"
    res.update(t_fused_ms=0.09)          # a shipped form that loses: the speedup says so, the thread partition keeps its own figure
    bench.judge(res)
    assert res["speedup_pct"] < 0 and res["best_mode"] == "blockidx"
    assert res["hfuse_speedup_pct"] == pytest.approx((0.0785 / 0.0707 - 1) * 100)
    res.update(t_vfuse_ms=0.0692)        # within 0.5 % of the fastest: the same speed for every practical purpose
    bench.judge(res)
    assert res["modes_within_0p5pct_of_best"] == ["blockidx", "vfuse"]


def test_spread_of_samples(bench):
    assert bench.spread({"t_fused_ms": [3.0, 1.0, 2.0]}) == {"t_fused_ms": [1.0, 2.0, 3.0]}


def test_valu_issue_rate_constants(bench):
    # 256 CUs x 64 lanes x 2.4 GHz: the rate the 64-lane VALU issue of the part sets (SHA-256d alone runs at it)
    assert bench.VALU_ISSUE_GLANES == pytest.approx(39321.6)
    assert bench.VALU_PEAK_GOPS == 2 * bench.VALU_ISSUE_GLANES
    assert 0.95 < bench.VALU_INSTS_SHA256D * 12.9 / bench.VALU_ISSUE_GLANES < 1.05
    assert 0.95 < bench.VALU_INSTS_BLAKE2B * 22.3 / bench.VALU_ISSUE_GLANES < 1.05     # Blake2b alone: 22.3 GH/s


def test_roofline_constants(bench):
    assert bench.HBM_PEAK_GBPS == 8000.0
    assert bench.ETHASH_BYTES == 64 * 128
    # SHA-256d: two compressions of 64 rounds x 24 + 48 schedule words x 13 + 8 feed-forward adds
    assert bench.OPS_SHA256D == 2 * (64 * 24 + 48 * 13 + 8)
    # Blake2b: 96 G functions x 26 32-bit ops + 32
    assert bench.OPS_BLAKE2B == 96 * 26 + 32
    # counter traffic is within 2 % of the algorithmic bytes of every covered pair
    algorithmic = {"bn_upsample": 25_692_160 + 128_450_560, "im2col_maxpool": 256_901_120 + 179_830_784,
                   "histc_maxpool": 268_439_552 + 58_720_256, "ethash_blake2b": (1 << 28) * 8192}
    for name, measured in bench.TRAFFIC_BYTES.items():
        assert 0.98 < measured / algorithmic[name] < 1.02, name
    # read + written bytes of a tensor pair are its algorithmic bytes
    for name, (rd, wr) in bench.PAIR_READ_WRITE_BYTES.items():
        assert rd + wr == algorithmic[name], name
