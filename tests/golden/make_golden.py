"""Writes tests/golden/cp4_golden.npz: small seeded cases of the CP4 conv with
expected outputs computed in float64 by torch's CPU dense conv2d and autograd
on the recomposed kernel K = einsum('tr,cr,yr,xr->tcyx', FK, FC, FH, FW) -- the
check the reference's own tests use (Cuda_kernels/test/test_cp4Conv.cpp.cu:31-43,
test/test_conv2d_cp4.py:25-34), with a library routine in place of cuDNN / TF.
Neither the oracle nor the HIP library is involved in producing these vectors.

A second file, tests/golden/cp4_golden_geometry.npz, holds cases with a stride,
explicit padding and an output plane of their own (the "SAME" / "VALID" padding
and strides of the reference's Python layer, test/layers.py:264-279), from the
same library routine with stride.

Run from the repo root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

CASES = [
    # name, N, C, H, W, pad, T, Y, X, R
    ("tiny3x3", 1, 2, 4, 4, 1, 2, 3, 3, 2),
    ("five5x5", 2, 3, 6, 5, 2, 4, 5, 5, 3),
    ("one1x1", 2, 4, 3, 7, 0, 5, 1, 1, 4),
    ("config1", 1, 16, 32, 32, 1, 16, 3, 3, 8),
    ("ragged", 3, 5, 9, 11, 1, 7, 3, 3, 6),
    ("bigpad", 1, 3, 6, 6, 2, 2, 3, 3, 2),   # 2*pad > Y-1: output stays H x W
    ("nopad", 1, 3, 7, 6, 0, 2, 3, 3, 2),    # 2*pad < Y-1: output stays H x W
]


def dense_same_conv(x, K, pad):
    """H x W output, tap (y, x) reads In[h+y-pad, w+x-pad], zero outside
    (Cuda_kernels/cp4Conv2dForward.cu:92-103)."""
    Y, X = K.shape[2], K.shape[3]
    xp = F.pad(x, (pad, X - 1 - pad, pad, Y - 1 - pad))
    return F.conv2d(xp, K)


# Layer geometry cases (stride, zeros before the image, output plane), expected
# values from torch float64 conv2d(stride) on the explicitly padded input and its
# autograd: name, N, C, H, W, T, Y, X, R, (sh, sw), (pad_top, pad_left), (out_h, out_w)
def tf_same(H, W, Y, X, sh, sw):
    """padding="SAME" of the framework the reference's layers call
    (test/layers.py:264-279): out = ceil(in / stride), total padding what the last
    window needs, the smaller half before the image."""
    ho, wo = -(-H // sh), -(-W // sw)
    th, tw = max((ho - 1) * sh + Y - H, 0), max((wo - 1) * sw + X - W, 0)
    return (th // 2, tw // 2), (ho, wo)


GEOM_CASES = [
    ("s2_same_even", 2, 3, 8, 8, 4, 3, 3, 3, (2, 2)) + tf_same(8, 8, 3, 3, 2, 2),      # pads 0 before, 1 after
    ("s2_same_odd", 1, 4, 9, 7, 3, 3, 3, 2, (2, 2)) + tf_same(9, 7, 3, 3, 2, 2),
    ("s2_sym_pad1", 2, 3, 8, 10, 4, 3, 3, 3, (2, 2), (1, 1), (4, 5)),                 # PyTorch padding=1
    ("s1_valid", 1, 3, 7, 6, 2, 3, 3, 2, (1, 1), (0, 0), (5, 4)),                     # "VALID": no padding
    ("s2_valid_5x5", 1, 2, 11, 12, 3, 5, 5, 2, (2, 2), (0, 0), (4, 4)),
    ("s21_rect", 2, 3, 9, 8, 2, 3, 3, 2, (2, 1), (1, 1), (5, 8)),                     # stride 2 down, 1 across
    ("s3_same_7x7", 1, 2, 13, 13, 2, 7, 7, 2, (3, 3)) + tf_same(13, 13, 7, 7, 3, 3),
    ("s1_full", 1, 2, 5, 5, 2, 3, 3, 2, (1, 1), (2, 2), (7, 7)),                      # output larger than the input
]


def geom_conv(x, K, stride, pads, out):
    (sh, sw), (pt, pl), (ho, wo) = stride, pads, out
    Y, X = K.shape[2], K.shape[3]
    H, W = x.shape[2], x.shape[3]
    pb = max(sh * (ho - 1) + Y - pt - H, 0)
    pr = max(sw * (wo - 1) + X - pl - W, 0)
    xp = F.pad(x, (pl, pr, pt, pb))
    return F.conv2d(xp, K, stride=(sh, sw))[:, :, :ho, :wo]


def geom_main():
    out = {}
    for name, N, C, H, W, T, Y, X, R, stride, pads, osz in GEOM_CASES:
        g = torch.Generator().manual_seed(sum(map(ord, name)))
        x = (torch.rand(N, C, H, W, generator=g, dtype=torch.float64) * 2 - 1)
        dy = torch.randn(N, T, *osz, generator=g, dtype=torch.float64)
        sd = 1.0 / np.sqrt(R * C)
        fac = [torch.randn(d, R, generator=g, dtype=torch.float64) * sd for d in (T, C, Y, X)]
        x, dy = x.float().double(), dy.float().double()
        fac = [f.float().double().requires_grad_(True) for f in fac]
        x.requires_grad_(True)
        K = torch.einsum("tr,cr,yr,xr->tcyx", *fac)
        y = geom_conv(x, K, stride, pads, osz)
        assert tuple(y.shape[2:]) == tuple(osz), (name, y.shape)
        (y * dy).sum().backward()
        out[name + ".shape"] = np.array([N, H, W, 0, T, C, Y, X, R], np.uint32)
        out[name + ".geometry"] = np.array([*stride, *pads, *osz], np.uint32)
        out[name + ".x"] = x.detach().numpy().astype(np.float32)
        out[name + ".dy"] = dy.numpy().astype(np.float32)
        for k, f in zip(("FK", "FC", "FH", "FW"), fac):
            out[f"{name}.{k}"] = f.detach().numpy().astype(np.float32)
            out[f"{name}.d{k}"] = f.grad.numpy().astype(np.float32)
        out[name + ".y"] = y.detach().numpy().astype(np.float32)
        out[name + ".dx"] = x.grad.numpy().astype(np.float32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cp4_golden_geometry.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


def main():
    out = {}
    for name, N, C, H, W, pad, T, Y, X, R in CASES:
        g = torch.Generator().manual_seed(sum(map(ord, name)))
        x = (torch.rand(N, C, H, W, generator=g, dtype=torch.float64) * 2 - 1)
        dy = torch.randn(N, T, H, W, generator=g, dtype=torch.float64)
        sd = 1.0 / np.sqrt(R * C)
        fac = [torch.randn(d, R, generator=g, dtype=torch.float64) * sd
               for d in (T, C, Y, X)]
        # round inputs to fp32 first so the stored inputs are exactly what is convolved
        x, dy = x.float().double(), dy.float().double()
        fac = [f.float().double().requires_grad_(True) for f in fac]
        x.requires_grad_(True)
        FK, FC, FH, FW = fac
        K = torch.einsum("tr,cr,yr,xr->tcyx", FK, FC, FH, FW)
        y = dense_same_conv(x, K, pad)
        (y * dy).sum().backward()
        out[name + ".shape"] = np.array([N, H, W, pad, T, C, Y, X, R], np.uint32)
        out[name + ".x"] = x.detach().numpy().astype(np.float32)
        out[name + ".dy"] = dy.numpy().astype(np.float32)
        for k, f in zip(("FK", "FC", "FH", "FW"), fac):
            out[f"{name}.{k}"] = f.detach().numpy().astype(np.float32)
            out[f"{name}.d{k}"] = f.grad.numpy().astype(np.float32)
        out[name + ".y"] = y.detach().numpy().astype(np.float32)
        # true adjoint of the forward map (equals the reference's backward-data
        # formula exactly when 2*pad == Y-1)
        out[name + ".dx_adjoint"] = x.grad.numpy().astype(np.float32)
        # the reference's backward-data formula for any pad
        # (Cuda_kernels/cp4Conv2dBackwardData.cu:79-87,98-108): same-size
        # correlation of dy with the spatially flipped, channel-transposed kernel
        Kb = K.detach().flip(2, 3).transpose(0, 1).contiguous()
        out[name + ".dx"] = dense_same_conv(dy, Kb, pad).numpy().astype(np.float32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cp4_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
    geom_main()
