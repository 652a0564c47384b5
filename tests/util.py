"""Shared helpers of the tests: seeded inputs and torch-CPU reference ops."""
import numpy as np
import torch


def uniform(shape, seed, lo=-1.0, hi=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(shape, generator=g, dtype=torch.float32) * (hi - lo) + lo).contiguous()


def normal(shape, seed, mean=0.5, std=2.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std + mean).contiguous()


def pool_out(size, k, s, p, d=1):
    return (size + 2 * p - d * (k - 1) - 1) // s + 1


def torch_im2col(x, kernel, pad, stride, dil=(1, 1)):
    """x [N,C,H,W] -> [N, C*kh*kw, L] (PyTorch CPU unfold)."""
    return torch.nn.functional.unfold(x, kernel, dilation=dil, padding=pad, stride=stride)


def torch_maxpool(x, kernel, stride, pad, dil=(1, 1)):
    return torch.nn.functional.max_pool2d(x, kernel, stride, pad, dil, ceil_mode=False, return_indices=True)


def torch_bn_stats(x, eps):
    """save_mean, save_invstd of training-mode batch norm on CPU."""
    c = x.shape[1]
    _, mean, invstd = torch.native_batch_norm(x, None, None, None, None, True, 0.0, eps)
    assert mean.shape[0] == c
    return mean, invstd


def rel_err(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), 1e-30)))


def bilinear_tol(in_hw, out_hw, align):
    """Bound on |oracle - PyTorch CPU| for bilinear upsampling of inputs in [-1, 1].

    Both evaluate the same interpolant; they differ in how the four products are associated
    (2 ulp of the value) and, when the size ratio is not a power of two, in the rounding of
    the fp32 source index scale * (dst + 0.5) - 0.5, whose error of a few ulp of the index
    (<= max(H1, W1)) is multiplied by the difference of two neighbouring pixels (<= 2)."""
    def dyadic(i, o):
        r = o / i
        return r >= 1 and r == int(r) and int(r) & (int(r) - 1) == 0
    exact = not align and dyadic(in_hw[0], out_hw[0]) and dyadic(in_hw[1], out_hw[1])
    return 2.4e-7 if exact else 2.4e-7 * (1 + max(in_hw))
