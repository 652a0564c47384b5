"""Split tuner: candidate enumeration and fusion-list rewriting (CPU), one small sweep (GPU)."""
import os

import pytest

import hfuse_amd
from hfuse_amd import _lib as L
from hfuse_amd import launcher as H
from hfuse_amd import tuner as T

CONFIGS = os.path.join(os.path.dirname(os.path.abspath(hfuse_amd.__file__)), "configs")


def shipped():
    return (open(os.path.join(CONFIGS, "gfx950_fusion.yaml")).read(),
            open(os.path.join(CONFIGS, "gfx950_kernels.yaml")).read())


def test_block_candidates_cover_the_reference_enumeration():
    fusion, kernels = shipped()
    cfg = H.Config(fusion, kernels)
    i = cfg.find_fusion("im2col_kernel", "MaxPoolForward")
    c = T.block_candidates(cfg, i, step=128)
    assert all(a % 128 == 0 and b % 128 == 0 and a > 0 and b > 0 and a + b <= 1024 for a, b in c)
    assert len(c) == len(set(c)) == 28
    # the reference's splits 128*(n+1) < d1+d2 of the 512+256 block are among them
    for n in range(cfg.num_splits(i)):
        assert (128 * (n + 1), 768 - 128 * (n + 1)) in c
    # searches are built for blocks of at most 512 threads
    j = cfg.find_fusion("ethash_search", "sia_blake2b_gpu_hash")
    assert max(a + b for a, b in T.block_candidates(cfg, j)) == 512
    # batch norm keeps BlockDim.Y = 8: every share divides by it
    k = cfg.find_fusion("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame")
    assert all(a % 8 == 0 for a, _ in T.block_candidates(cfg, k))
    with pytest.raises(ValueError):
        T.block_candidates(cfg, i, step=96)


def test_apply_to_fusion_yaml_round_trip():
    fusion, kernels = shipped()
    cfg = H.Config(fusion, kernels)
    i = cfg.find_fusion("im2col_kernel", "kernelHistogram1D")        # an entry without tuned keys
    j = cfg.find_fusion("kernelHistogram1D", "MaxPoolForward")       # an entry that has them
    k = cfg.find_fusion("im2col_kernel", "MaxPoolForward")
    text = T.apply_to_fusion_yaml(fusion, {i: T.Candidate(384, 256, lending=False), j: T.Candidate(640, 128), k: None})
    assert text.count("- File:") == fusion.count("- File:")
    assert [ln for ln in text.splitlines() if ln.startswith("#")] == [ln for ln in fusion.splitlines() if ln.startswith("#")]
    new = H.Config(text, kernels)
    assert new.fusions() == cfg.fusions()
    p = new.plan(i).partition
    assert (p.hi[0] - p.lo[0], p.hi[1] - p.lo[1], p.launch_threads) == (384, 256, 640)
    p = new.plan(j).partition
    assert (p.hi[0] - p.lo[0], p.hi[1] - p.lo[1]) == (640, 128)
    p = new.plan(k).partition                                        # keys removed: the table's 512 + 256
    assert (p.hi[0] - p.lo[0], p.hi[1] - p.lo[1]) == (512, 256)
    # applying the same result twice changes nothing
    assert T.apply_to_fusion_yaml(text, {i: T.Candidate(384, 256, lending=False)}) == text
    # untouched entries are byte-identical
    assert T.apply_to_fusion_yaml(fusion, {}) == fusion if fusion.endswith("\n") else True


def test_stripping_every_entry_gives_the_untuned_list():
    fusion, kernels = shipped()
    n = fusion.count("- File:")
    clean = T.apply_to_fusion_yaml(fusion, {i: None for i in range(n)})
    body = [ln for ln in clean.splitlines() if not ln.lstrip().startswith("#")]
    assert not any(ln.split(":")[0].strip() in ("Split", "Threads", "Lending", "Barrier", "LaunchBound") for ln in body)
    cfg = H.Config(clean, kernels)
    assert cfg.fusions() == H.Config(fusion, kernels).fusions()
    p = cfg.plan(cfg.find_fusion("kernelHistogram1D", "MaxPoolForward")).partition
    assert (p.hi[0] - p.lo[0], p.hi[1] - p.lo[1]) == (512, 256)


def test_barrier_key():
    _, kernels = shipped()
    base = "- File: a\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n"
    assert H.Config(base + "  Barrier: blockidx\n", kernels).plan(0).partition.barrier_mode == L.HF_BARRIER_BLOCKIDX
    assert H.Config(base, kernels).plan(0).partition.barrier_mode == L.HF_BARRIER_NONE
    with pytest.raises(hfuse_amd.HfuseError) as e:
        H.Config(base + "  Barrier: sometimes\n", kernels)
    assert e.value.code == L.HF_EPARSE and "Barrier" in e.value.message
    with pytest.raises(hfuse_amd.HfuseError) as e:      # neither kernel synchronises: nothing to match
        H.Config(base + "  Barrier: matched\n", kernels).plan(0)
    assert e.value.code == L.HF_EINVAL
    text = T.apply_to_fusion_yaml(base, {0: T.Candidate(256, 256, True, L.HF_BARRIER_BLOCKIDX)})
    assert text == base + "  Split: 256\n  Threads: 512\n  Barrier: blockidx\n"
    assert T.apply_to_fusion_yaml(text, {0: None}) == base


def test_lending_key():
    _, kernels = shipped()
    ok = "- File: a\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n  Lending: false\n"
    H.Config(ok, kernels).plan(0)
    with pytest.raises(hfuse_amd.HfuseError) as e:
        H.Config(ok.replace("false", "maybe"), kernels)
    assert e.value.code == L.HF_EPARSE and "Lending" in e.value.message


def test_launch_bound_key():
    _, kernels = shipped()
    base = "- File: a\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n"
    H.Config(base + "  LaunchBound: true\n", kernels).plan(0)
    H.Config(base + "  LaunchBound: false\n", kernels).plan(0, "hfuse_lb")
    with pytest.raises(hfuse_amd.HfuseError) as e:
        H.Config(base + "  LaunchBound: 8\n", kernels)
    assert e.value.code == L.HF_EPARSE and "LaunchBound" in e.value.message
    text = T.apply_to_fusion_yaml(base, {0: T.Candidate(256, 256, bounded=True)})
    assert text == base + "  Split: 256\n  Threads: 512\n  LaunchBound: true\n"
    assert T.apply_to_fusion_yaml(text, {0: T.Candidate(256, 256)}) == base + "  Split: 256\n  Threads: 512\n"
    assert T.Candidate(128, 64, bounded=True).label() == "128+64 lb"
    plan = H.Config(base, kernels).plan(0)
    for on in (True, False, None):
        plan.set_launch_bound(on)


def test_vertical_candidates_and_their_keys():
    """The vertical forms the tuner tries, and how a vertical winner is written next to the best thread partition."""
    fusion, kernels = shipped()
    cfg = H.Config(fusion, kernels)
    i = cfg.find_fusion("kernelHistogram1D", "MaxPoolForward")
    c = T.vertical_candidates(cfg, i, cus=256)
    assert all(x.vertical and x.preset == "vfuse" and x.threads1 == x.threads2 for x in c)
    assert {x.threads1 for x in c} == {512, 768, 1024}
    assert T.Candidate(1024, 1024, grids=(0, 256), preset="vfuse") in c      # histogram on its own grid, pooling on resident blocks
    assert T.Candidate(1024, 1024, grids=(512, 512), preset="vfuse") in c and T.Candidate(512, 512, preset="vfuse") in c
    assert not any(x.threads1 == 768 and x.grids == (0, 0) and x.bounded for x in c)
    # batch norm's blocks are rows of eight: 768 and 1024 divide, and so does 512
    k = cfg.find_fusion("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame")
    assert {x.threads1 for x in T.vertical_candidates(cfg, k, cus=256)} == {512, 768, 1024}
    base = "- File: a\n  Kernels:\n    - kernelHistogram1D\n    - MaxPoolForward\n"
    win, part = T.Candidate(1024, 1024, grids=(0, 256), preset="vfuse"), T.Candidate(832, 192)
    text = T.apply_to_fusion_yaml(base, {0: (win, part)})
    assert text == base + "  Split: 832\n  Threads: 1024\n  Preset: vfuse\n  Blocks: [1024, 1024]\n  Grids: [0, 256]\n"
    new = H.Config(text, kernels)
    v = new.plan(0, "shipped").partition
    assert v.name.decode().endswith("vfuse_block_1024_1024") and v.launch_threads == 1024
    h = new.plan(0, "hfuse").partition
    assert (list(h.hi), h.launch_threads) == ([832, 1024], 1024)
    assert T.apply_to_fusion_yaml(text, {0: None}) == base
    assert T.apply_to_fusion_yaml(text, {0: (win, part)}) == text
    # a bounded vertical winner names the bounded preset
    lb = T.apply_to_fusion_yaml(base, {0: (T.Candidate(512, 512, bounded=True, preset="vfuse"), None)})
    assert lb == base + "  Preset: vfuse_lb\n  Blocks: [512, 512]\n"
    assert H.Config(lb, kernels).plan(0, "shipped").partition.name.decode().endswith("vfuse_lb_block_512_512")


@pytest.mark.gpu
def test_small_sweep_and_tuned_launch(cuda):
    from test_gpu_tensor_kernels import Im2col, MaxPool, sync
    fusion, kernels = shipped()
    cfg = H.Config(fusion, kernels)
    i = cfg.find_fusion("im2col_kernel", "MaxPoolForward")
    a = [Im2col(cuda, 4, 8, 24, 24, seed=50 + s) for s in range(2)]
    b = [MaxPool(cuda, 4, 8, 32, 32, (3, 3), (2, 2), (1, 1)) for _ in range(2)]
    shapes = [(128, 128), (256, 256), (512, 256), (256, 512)]
    r = T.tune(cfg, i, [t.args for t in a], [t.args for t in b], blocks=shapes, probe_iters=5, final_iters=10, finalists=2)
    assert (r.best.threads1, r.best.threads2) in shapes
    # 4 shapes x lending on / off, plus the two finalists again in the register-bounded build
    assert len(r.table) == 10 and sum(lab.endswith(" lb") for lab, _ in r.table) == 2 and r.t_best_ms > 0 and r.t_b2b_ms > 0 and r.t_table_ms > 0
    for t in a + b:   # the sweep's own launches wrote correct results
        sync()
        t.check()
    tuned_cfg = H.Config(T.apply_to_fusion_yaml(fusion, {i: r.best}), kernels)
    plan = tuned_cfg.plan(i)
    assert plan.partition.launch_threads == r.best.threads1 + r.best.threads2
    plan.launch(a[0].args, b[0].args)
    sync()
    a[0].check()
    b[0].check()
