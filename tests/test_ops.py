"""The torch-tensor operator layer: same results as the PyTorch CPU operators the oracle is pinned to."""
import pytest
import torch
import torch.nn.functional as F

from hfuse_amd import ops
from util import normal, rel_err, torch_bn_stats, uniform


def test_operators_refuse_what_they_cannot_run():
    x = torch.zeros(2, 3, 8, 8)                     # a CPU tensor: there is no CPU path
    for make in (lambda: ops.im2col(x, 3), lambda: ops.max_pool2d(x, 2), lambda: ops.batch_norm_collect_statistics(x),
                 lambda: ops.upsample_nearest2d(x, scale_factor=2), lambda: ops.upsample_bilinear2d(x, size=(9, 9)),
                 lambda: ops.histc(x, 10, 0, 1)):
        with pytest.raises(TypeError):
            make()


@pytest.mark.gpu
def test_native_operators_match_pytorch(cuda):
    x = uniform((3, 5, 14, 18), 71)
    xd = x.to(cuda)
    (col,) = ops.run(ops.im2col(xd, (3, 2), dilation=(1, 2), padding=(1, 0), stride=(2, 1)))
    assert torch.equal(col.cpu(), F.unfold(x, (3, 2), dilation=(1, 2), padding=(1, 0), stride=(2, 1)))
    (col1,) = ops.run(ops.im2col(xd[0], 3, padding=1))                      # unbatched
    assert torch.equal(col1.cpu(), F.unfold(x[:1], 3, padding=1)[0])
    val, idx = ops.run(ops.max_pool2d(xd, 3, 2, 1))
    tv, ti = F.max_pool2d(x, 3, 2, 1, return_indices=True)
    assert torch.equal(val.cpu(), tv) and torch.equal(idx.cpu(), ti)
    val, idx = ops.run(ops.max_pool2d(xd, (2, 3)))                          # stride defaults to the window
    tv, ti = F.max_pool2d(x, (2, 3), return_indices=True)
    assert torch.equal(val.cpu(), tv) and torch.equal(idx.cpu(), ti)
    xn = normal((6, 7, 9, 4), 72)
    mean, invstd = ops.run(ops.batch_norm_collect_statistics(xn.to(cuda), 1e-5))
    wm, wi = torch_bn_stats(xn, 1e-5)
    assert rel_err(mean.cpu().numpy(), wm) < 1e-5 and rel_err(invstd.cpu().numpy(), wi) < 1e-5
    (up,) = ops.run(ops.upsample_nearest2d(xd, scale_factor=2))
    assert torch.equal(up.cpu(), F.interpolate(x, scale_factor=2, mode="nearest"))
    (up,) = ops.run(ops.upsample_nearest2d(xd, size=(20, 31)))
    assert torch.equal(up.cpu(), F.interpolate(x, size=(20, 31), mode="nearest"))
    (bl,) = ops.run(ops.upsample_bilinear2d(xd, scale_factor=2))
    assert (bl.cpu() - F.interpolate(x, scale_factor=2, mode="bilinear", align_corners=False)).abs().max() <= 2.4e-7
    (bl,) = ops.run(ops.upsample_bilinear2d(xd.transpose(2, 3), size=(30, 17), align_corners=True))   # strided input
    want = F.interpolate(x.transpose(2, 3), size=(30, 17), mode="bilinear", align_corners=True)
    assert (bl.cpu() - want).abs().max() <= 2.4e-7 * 19
    h = uniform((100000,), 73, 0.0, 1.0)
    (counts,) = ops.run(ops.histc(h.to(cuda), 256, 0.0, 1.0))
    assert torch.equal(counts.cpu(), torch.histc(h, 256, 0.0, 1.0))
    (counts,) = ops.run(ops.histc(h.to(cuda).reshape(100, 1000), 64))       # range from the data, any shape
    assert float(counts.sum()) == 100000.0 and torch.equal(counts.cpu(), torch.histc(h, 64))


@pytest.mark.gpu
def test_fused_operators_in_either_order(cuda):
    x, y = uniform((2, 4, 12, 12), 74), uniform((2, 4, 16, 16), 75)
    xd, yd = x.to(cuda), y.to(cuda)
    tv, ti = F.max_pool2d(y, 3, 2, 1, return_indices=True)
    want_col = F.unfold(x, 3, padding=1)
    (col,), (val, idx) = ops.run_fused(ops.im2col(xd, 3, padding=1), ops.max_pool2d(yd, 3, 2, 1))
    torch.cuda.synchronize()
    assert torch.equal(col.cpu(), want_col) and torch.equal(val.cpu(), tv) and torch.equal(idx.cpu(), ti)
    (val, idx), (col,) = ops.run_fused(ops.max_pool2d(yd, 3, 2, 1), ops.im2col(xd, 3, padding=1))    # listed the other way round
    torch.cuda.synchronize()
    assert torch.equal(col.cpu(), want_col) and torch.equal(val.cpu(), tv) and torch.equal(idx.cpu(), ti)
    xn = normal((4, 9, 6, 6), 76)
    (mean, invstd), (up,) = ops.run_fused(ops.batch_norm_collect_statistics(xn.to(cuda)), ops.upsample_nearest2d(xd, scale_factor=2),
                                          preset="vfuse")
    wm, wi = torch_bn_stats(xn, 1e-5)
    assert rel_err(mean.cpu().numpy(), wm) < 1e-5 and rel_err(invstd.cpu().numpy(), wi) < 1e-5
    assert torch.equal(up.cpu(), F.interpolate(x, scale_factor=2, mode="nearest"))
    with pytest.raises(KeyError):
        ops.run_fused(ops.upsample_nearest2d(xd, scale_factor=2), ops.upsample_bilinear2d(xd, scale_factor=2))


@pytest.mark.gpu
def test_search_operators(cuda):
    from oracle import oracle as O
    easy = (1 << 52) - 1
    hdr_a, hdr_b = O.seeded_bytes(80, 91), O.seeded_bytes(80, 92)
    a = ops.sha256d_search(hdr_a, easy, 1000, 1 << 15)
    ops.run(a)
    found, got = ops.hits(a)
    want = O.sha256d_search(hdr_a, 1000, 1 << 15, easy)
    assert found == want[0] > 0 and [g[0] for g in got] == [h.nonce for h in want[1]]
    assert all(g[1] == O.sha256d_80(hdr_a, g[0]) for g in got)
    # fused with the Sia search, named in the list as (sha256d, sia): pass them the other way round
    a, b = ops.sha256d_search(hdr_a, easy, 0, 1 << 14), ops.sia_blake2b_search(hdr_b, easy, 0, 1 << 15)
    ops.run_fused(b, a)
    fa, ga = ops.hits(a)
    fb, gb = ops.hits(b)
    assert fa == O.sha256d_search(hdr_a, 0, 1 << 14, easy)[0] > 0 and fb == O.sia_search(hdr_b, 0, 1 << 15, easy)[0] > 0
    assert all(g[1] == O.sia_blake2b_80(hdr_b, g[0]) for g in gb)
    # ethash over a small synthetic DAG, alone and next to blake2b
    from hfuse_amd import launcher as H
    n_items, seed = 1 << 12, 0x48467573
    dag = torch.empty(n_items * 32, dtype=torch.int32, device=cuda)
    H.fill_splitmix64(dag, seed)
    hdr = O.seeded_bytes(32, 93)
    target = (1 << 56) - 1
    want_n, want_h = O.ethash_search(None, seed, n_items, hdr, 0, 4096, target)
    e = ops.ethash_search(dag, n_items, hdr, target, 0, 4096)
    ops.run(e)
    assert ops.hits(e) == (want_n, [(h.nonce, h.digest_bytes(), h.mix_bytes()) for h in want_h]) and want_n > 0
    e, b = ops.ethash_search(dag, n_items, hdr, target, 0, 4096), ops.sia_blake2b_search(hdr_b, easy, 0, 1 << 15)
    ops.run_fused(e, b)
    assert ops.hits(e) == (want_n, [(h.nonce, h.digest_bytes(), h.mix_bytes()) for h in want_h])
    assert ops.hits(b)[0] == fb


@pytest.mark.gpu
def test_three_ops_in_one_launch(cuda):
    """run_fused3 on the reference's im2col + max_pool2d + batch-norm list and on max_pool2d + histc + batch-norm."""
    x, y, z = uniform((2, 8, 16, 16), 81), uniform((2, 8, 32, 32), 82), normal((4, 10, 7, 9), 83)
    (col,), (val, idx), (mean, invstd) = ops.run_fused3(ops.im2col(x.to(cuda), 3, padding=1), ops.max_pool2d(y.to(cuda), 3, 2, 1),
                                                        ops.batch_norm_collect_statistics(z.to(cuda), 1e-5))
    torch.cuda.synchronize()
    assert torch.equal(col.cpu(), F.unfold(x, 3, padding=1))
    tv, ti = F.max_pool2d(y, 3, 2, 1, return_indices=True)
    assert torch.equal(val.cpu(), tv) and torch.equal(idx.cpu(), ti)
    wm, wi = torch_bn_stats(z, 1e-5)
    assert rel_err(mean.cpu().numpy(), wm) < 1e-5 and rel_err(invstd.cpu().numpy(), wi) < 1e-5
    h = uniform((50000,), 84, 0.0, 1.0)
    (val, idx), (hist,), (mean, invstd) = ops.run_fused3(ops.max_pool2d(y.to(cuda), 2), ops.histc(h.to(cuda), 64, 0, 1),
                                                         ops.batch_norm_collect_statistics(z.to(cuda), 1e-5), preset="vfuse")
    torch.cuda.synchronize()
    tv, ti = F.max_pool2d(y, 2, return_indices=True)
    assert torch.equal(val.cpu(), tv) and torch.equal(idx.cpu(), ti)
    assert torch.equal(hist.cpu(), torch.histc(h, 64, 0, 1))
    assert rel_err(mean.cpu().numpy(), wm) < 1e-5
    with pytest.raises(KeyError):
        ops.run_fused3(ops.max_pool2d(y.to(cuda), 2), ops.im2col(x.to(cuda), 3), ops.histc(h.to(cuda), 64, 0, 1))
