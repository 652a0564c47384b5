"""Operator-level entry points over torch tensors: the counterpart of the caller that sat on
top of the reference's generated kernels (its README builds a torch extension, TorchKernel,
whose Python side calls each original kernel and each fused pair on torch tensors).

An `Op` is one original kernel bound to its inputs, with outputs allocated the way the PyTorch
operator of the same name allocates them.  `run(op)` launches it natively; `run_fused(op1, op2)`
launches both as one horizontally fused kernel (the pair must be in the fusion list, in either
order); `run_fused3(op0, op1, op2)` does the same for the reference's three-kernel lists.  Results are the op's outputs:

    from hfuse_amd import ops
    pooled, indices = ops.run(ops.max_pool2d(x, 3, 2, 1))
    (cols,), (pooled, indices) = ops.run_fused(ops.im2col(img, 3, padding=1), ops.max_pool2d(x, 3, 2, 1))

The nonce searches have the same shape: `sha256d_search`, `sia_blake2b_search`, `blake2b_search`
and `ethash_search` upload a job's constants and return an op; `hits(op)` reads the found nonces.

Tensors are float32 CUDA tensors (this build's kernels are the float instantiations the
reference fused); inputs are made contiguous where the original operator does so.  torch is used
for allocation and streams only; every launch goes through the C-ABI.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional, Sequence, Tuple

from . import launcher as H


def _pair(v) -> Tuple[int, int]:
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


def _check(x, dims: Sequence[int], what: str):
    import torch
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != torch.float32:
        raise TypeError(f"{what}: expected a float32 CUDA tensor")
    if x.dim() not in dims:
        raise ValueError(f"{what}: expected {' or '.join(str(d) for d in dims)} dimensions, got {x.dim()}")
    if x.numel() == 0:
        raise ValueError(f"{what}: non-empty tensor expected")


@dataclass
class Op:
    """One original kernel with its argument struct; `keep` holds the tensors the struct points at."""
    kernel: str
    args: Any
    outputs: Tuple[Any, ...]
    keep: Tuple[Any, ...] = ()


def im2col(x, kernel_size, dilation=1, padding=0, stride=1) -> Op:
    """torch.nn.functional.unfold: x [N, C, H, W] -> columns [N, C*kh*kw, Hc*Wc] (one launch for the batch)."""
    import torch
    _check(x, (3, 4), "im2col")
    x4 = (x if x.dim() == 4 else x.unsqueeze(0)).contiguous()
    k, d, p, s = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    n, c, h, w = x4.shape
    hc = (h + 2 * p[0] - (d[0] * (k[0] - 1) + 1)) // s[0] + 1
    wc = (w + 2 * p[1] - (d[1] * (k[1] - 1) + 1)) // s[1] + 1
    if hc <= 0 or wc <= 0:
        raise ValueError("im2col: the kernel does not fit the padded image")
    out = torch.empty((n, c * k[0] * k[1], hc * wc), device=x.device, dtype=torch.float32)
    res = out if x.dim() == 4 else out[0]
    return Op("im2col_kernel", H.im2col_args(x4, out, k, p, s, d), (res,), (x4, out))


def max_pool2d(x, kernel_size, stride=None, padding=0, dilation=1) -> Op:
    """torch max_pool2d with indices (floor mode): x [N, C, H, W] -> (values, int64 indices h*W+w)."""
    import torch
    _check(x, (3, 4), "max_pool2d")
    x4 = (x if x.dim() == 4 else x.unsqueeze(0)).contiguous()
    k = _pair(kernel_size)
    s = _pair(stride) if stride is not None else k
    p, d = _pair(padding), _pair(dilation)
    n, c, h, w = x4.shape
    ph = (h + 2 * p[0] - d[0] * (k[0] - 1) - 1) // s[0] + 1
    pw = (w + 2 * p[1] - d[1] * (k[1] - 1) - 1) // s[1] + 1
    if ph <= 0 or pw <= 0:
        raise ValueError("max_pool2d: output size is too small")
    val = torch.empty((n, c, ph, pw), device=x.device, dtype=torch.float32)
    idx = torch.empty((n, c, ph, pw), device=x.device, dtype=torch.int64)
    res = (val, idx) if x.dim() == 4 else (val[0], idx[0])
    return Op("MaxPoolForward", H.maxpool_args(x4, val, idx, k, s, p, d), res, (x4, val, idx))


def batch_norm_collect_statistics(x, eps: float = 1e-5) -> Op:
    """Per-channel mean and 1/sqrt(biased variance + eps) of x [N, C, ...] (training-mode batch-norm statistics)."""
    import torch
    _check(x, (2, 3, 4, 5), "batch_norm_collect_statistics")
    c = x.shape[1]
    mean = torch.empty(c, device=x.device, dtype=torch.float32)
    invstd = torch.empty(c, device=x.device, dtype=torch.float32)
    x3 = x.reshape(x.shape[0], c, -1)
    return Op("batch_norm_collect_statistics_kernel", H.bn_stats_args(x3, mean, invstd, eps, 0.0), (mean, invstd),
              (x3, mean, invstd))


def _out_size(x, size, scale_factor):
    if (size is None) == (scale_factor is None):
        raise ValueError("give exactly one of size and scale_factor")
    if size is not None:
        return _pair(size)
    sf = (scale_factor, scale_factor) if isinstance(scale_factor, (int, float)) else scale_factor
    return int(x.shape[-2] * sf[0]), int(x.shape[-1] * sf[1])


def upsample_nearest2d(x, size=None, scale_factor=None) -> Op:
    """F.interpolate(mode='nearest') of x [N, C, H, W]."""
    import torch
    _check(x, (4,), "upsample_nearest2d")
    xc = x.contiguous()
    out = torch.empty(tuple(x.shape[:2]) + _out_size(x, size, scale_factor), device=x.device, dtype=torch.float32)
    return Op("upsample_nearest2d_out_frame", H.upsample_nearest_args(xc, out), (out,), (xc, out))


def upsample_bilinear2d(x, size=None, scale_factor=None, align_corners: bool = False) -> Op:
    """F.interpolate(mode='bilinear') of x [N, C, H, W] (any strides)."""
    import torch
    _check(x, (4,), "upsample_bilinear2d")
    out = torch.empty(tuple(x.shape[:2]) + _out_size(x, size, scale_factor), device=x.device, dtype=torch.float32)
    return Op("upsample_bilinear2d_out_frame", H.upsample_bilinear_args(x, out, align_corners), (out,), (x, out))


def histc(x, bins: int = 100, min: float = 0.0, max: float = 0.0) -> Op:
    """torch.histc: float counts of x's elements in `bins` equal bins over [min, max] (both 0: the data's range)."""
    import torch
    _check(x, tuple(range(0, 9)), "histc")
    flat = x.reshape(-1)
    lo, hi = float(min), float(max)
    if lo == 0.0 and hi == 0.0:
        lo, hi = float(flat.min()), float(flat.max())
    if lo == hi:          # torch widens an empty range by one on each side
        lo, hi = lo - 1.0, hi + 1.0
    out = torch.zeros(int(bins), device=x.device, dtype=torch.float32)
    return Op("kernelHistogram1D", H.histc_args(flat, out, int(bins), lo, hi), (out,), (flat, out))


# ------------------------------------------------------------------ nonce searches
# The miners' host loop: constants of a search (header, target, DAG) are uploaded once per
# job, then a launch scans `count` nonces from `start` and appends its hits to a result record.
# The constants are per process, like the __constant__ symbols of the original kernels, so one
# job per kind of search is live at a time.  `hits(op)` reads the record back (it synchronises).

@dataclass
class SearchOp(Op):
    count: int = 0         # ethash only: nonces to scan; the launch grid is derived from it


def sha256d_search(header: bytes, target64: int, start: int, count: int) -> SearchOp:
    """Nonces in [start, start+count) (mod 2^32) whose SHA-256d of the 80-byte header, read as a
    little-endian 256-bit number, has its top 64 bits <= target64."""
    H.sha256d_set_block(header, target64)
    res = H.new_search_results()
    return SearchOp("sha256d_gpu_hash_shared", H.sha256d_args(res, count, start), (res,), (res,))


def sia_blake2b_search(header: bytes, target64: int, start: int, count: int) -> SearchOp:
    """Sia layout: 8-byte nonce at offset 32 of the 80-byte header, Blake2b-256, first digest word (big-endian) <= target64."""
    H.sia_blake2b_set_block(header)
    res = H.new_search_results()
    return SearchOp("sia_blake2b_gpu_hash", H.blake2b_args(res, count, start, target64), (res,), (res,))


def blake2b_search(header: bytes, target64: int, start: int, count: int) -> SearchOp:
    """ccminer layout: 4-byte nonce at offset 76 of the 80-byte header."""
    H.blake2b_set_block(header)
    res = H.new_search_results()
    return SearchOp("blake2b_gpu_hash", H.blake2b_args(res, count, start, target64), (res,), (res,))


def ethash_search(dag, dag_items: int, header: bytes, target64: int, start: int, count: int) -> SearchOp:
    """Ethash hashimoto over a resident DAG of `dag_items` 128-byte items.  The kernel scans
    grid * block nonces like the original, so `count` is rounded up to a multiple of its block
    (128 threads natively, its share of the fused block in a fused launch)."""
    H.ethash_set_constants(dag, dag_items, header, target64)
    res = H.new_search_results()
    return SearchOp("ethash_search", H.ethash_args(res, start), (res,), (res, dag), count=int(count))


def hits(op: SearchOp):
    """-> (number found, [(nonce, digest bytes, mix bytes)] sorted by nonce, at most 64 kept)."""
    import torch
    torch.cuda.synchronize()
    return H.read_search_results(op.outputs[0])


_default_cfg: Optional[H.Config] = None


def _config(cfg: Optional[H.Config]) -> H.Config:
    global _default_cfg
    if cfg is not None:
        return cfg
    if _default_cfg is None:
        from . import default_config
        _default_cfg = default_config()
    return _default_cfg


def run(op: Op, stream=None):
    """Launch one original kernel; returns its outputs (a tuple)."""
    count = getattr(op, "count", 0)
    if count:   # ethash: grid * 128 threads cover the requested nonces
        H.launch_native(op.kernel, op.args, (count + 127) // 128, 128, stream=stream)
    else:
        H.launch_native(op.kernel, op.args, stream=stream)
    return op.outputs


def run_fused(op1: Op, op2: Op, cfg: Optional[H.Config] = None, preset: str = "shipped", stream=None):
    """Launch the two ops as one fused kernel; returns (outputs of op1, outputs of op2).

    The pair is looked up in the fusion list of `cfg` (default: the shipped list) in either
    order; a pair the list does not name raises KeyError.  `preset`: one of the reference's four
    (hfuse, hfuse_lb, vfuse, vfuse_lb) or "shipped", the form the list's entry was tuned to."""
    c = _config(cfg)
    try:
        first, second = op1, op2
        index = c.find_fusion(op1.kernel, op2.kernel)
    except KeyError:
        first, second = op2, op1
        index = c.find_fusion(op2.kernel, op1.kernel)
    plan = c.plan(index, preset)
    grid = 0
    part = plan.partition
    for half, op in enumerate((first, second)):   # ethash: the grid times its share of the block covers the nonces
        count = getattr(op, "count", 0)
        if count:
            threads = part.hi[half] - part.lo[half]
            grid = max(grid, (count + threads - 1) // threads)
    plan.launch(first.args, second.args, grid_blocks=grid, stream=stream)
    return op1.outputs, op2.outputs


_default_triples: Optional[H.Config] = None


def run_fused3(op0: Op, op1: Op, op2: Op, cfg: Optional[H.Config] = None, preset: str = "hfuse", stream=None):
    """Launch three ops as one fused kernel; returns their outputs in the order given.

    The three kernels must be an entry of `cfg` (default: the shipped three-kernel list, the reference's
    configs/crypt_four.yaml, im2col_maxpool_norm.yaml and maxpool_summary_norm.yaml) in the entry's order."""
    global _default_triples
    if cfg is None:
        if _default_triples is None:
            from . import triples_config
            _default_triples = triples_config()
        cfg = _default_triples
    trio = (op0, op1, op2)
    index = cfg.find_fusion_n(*(op.kernel for op in trio))
    plan = cfg.plan(index, preset)
    part = plan.partition_n
    grid = 0
    for k, op in enumerate(trio):   # ethash: the grid times its share of the block covers the nonces
        count = getattr(op, "count", 0)
        if count:
            threads = part.hi[k] - part.lo[k]
            grid = max(grid, (count + threads - 1) // threads)
    plan.launch_n([op.args for op in trio], grid_blocks=grid, stream=stream)
    return tuple(op.outputs for op in trio)
