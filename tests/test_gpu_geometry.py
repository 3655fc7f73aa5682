"""Layers with a stride, explicit padding or an output plane of their own
(cp4_conv2d_forward_ex and its two gradients) through the C ABI: the strides
and "SAME" / "VALID" padding of the reference's Python layer
(test/layers.py:264-279).

Checked against the committed geometry golden vectors (torch float64
conv2d(stride) + autograd, tests/golden/make_golden.py), against the CPU
oracle's strided restatement (pinned to those vectors in tests/test_oracle.py)
on shapes that take the matrix-core kernel, and against float64 autograd of the
dense strided convolution for the gradients at those sizes.  Bars: forward and
input gradient max|a-b| <= 1e-4 max|b| and |a-b| <= 1e-5 + 1e-4|b|; factor
gradients 1e-3.
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

GEOM = np.load(os.path.join(os.path.dirname(__file__), "golden", "cp4_golden_geometry.npz"))
GEOM_CASES = sorted({k.split(".")[0] for k in GEOM.files})
FACTORS = ("FK", "FC", "FH", "FW")


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def close_activation(got, want, what):
    scale = float(np.abs(want).max())
    err = np.abs(got - want)
    assert err.max() <= 1e-4 * scale, f"{what}: normalised {err.max() / scale:.2e}"
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(want)), f"{what}: elementwise {err.max():.2e}"


def close_gradient(got, want, what):
    scale = float(np.abs(want).max())
    err = np.abs(got - want)
    assert err.max() <= 1e-3 * scale, f"{what}: normalised {err.max() / scale:.2e}"


@pytest.mark.parametrize("name", GEOM_CASES)
def test_geometry_golden_all_passes(cp4, name):
    g = {k: GEOM[f"{name}.{k}"] for k in ("x", "dy", "y", "dx", "dFK", "dFC", "dFH", "dFW") + FACTORS}
    geom = cp4.Geometry(*[int(v) for v in GEOM[name + ".geometry"]])
    f = [dev(g[k]) for k in FACTORS]
    x, dy = dev(g["x"]), dev(g["dy"])
    y = cp4.conv2d_forward_ex(x, *f, geom)
    close_activation(y.cpu().numpy(), g["y"], f"{name} forward")
    dx = cp4.conv2d_backward_data_ex(dy, x.shape[2:], *f, geom)
    close_activation(dx.cpu().numpy(), g["dx"], f"{name} backward-data")
    grads = cp4.conv2d_backward_filter_ex(x, dy, *f, geom)
    for got, k in zip(grads, FACTORS):
        close_gradient(got.cpu().numpy(), g["d" + k], f"{name} d{k}")
    cp4.device_status()


def dense_reference(x, dy, fac, geom):
    """float64 autograd of the dense strided convolution on the recomposed filter."""
    xd = x.double().cpu().requires_grad_()
    fd = [t.double().cpu().requires_grad_() for t in fac]
    K = torch.einsum("tr,cr,yr,xr->tcyx", *fd)
    Y, X = K.shape[2:]
    H, W = xd.shape[2:]
    pb = max(geom.stride_h * (geom.out_h - 1) + Y - geom.pad_top - H, 0)
    pr = max(geom.stride_w * (geom.out_w - 1) + X - geom.pad_left - W, 0)
    xp = F.pad(xd, (geom.pad_left, pr, geom.pad_top, pb))
    y = F.conv2d(xp, K, stride=(geom.stride_h, geom.stride_w))[:, :, :geom.out_h, :geom.out_w]
    (y * dy.double().cpu()).sum().backward()
    return y.detach().numpy(), xd.grad.numpy(), [t.grad.numpy() for t in fd]


# N, C, H, W, T, Y, R, stride, padding: shapes the producer / consumer kernel's strided build takes
MATRIX_CASES = [
    (2, 32, 28, 28, 64, 3, 16, 2, "same"),
    (2, 64, 27, 29, 32, 3, 32, 2, "same"),          # odd sizes, odd output width
    (1, 48, 30, 30, 96, 5, 16, 2, "same"),
    (2, 32, 24, 24, 32, 3, 8, (2, 1), 1),           # stride 2 down, 1 across
    (2, 64, 16, 16, 64, 1, 16, 2, "valid"),         # 1x1 projection shortcut
    (1, 32, 20, 22, 40, 3, 24, 1, "valid"),         # stride 1, output smaller than the input
    (1, 32, 12, 12, 32, 3, 16, 1, 2),               # output larger than the input
    (1, 40, 33, 33, 72, 7, 16, 3, "same"),
    (2, 300, 14, 14, 64, 3, 16, 2, "same"),         # factor fragments in LDS
    (1, 32, 31, 45, 48, 5, 16, (3, 2), 2),          # unequal strides, 5x5
    (2, 32, 150, 40, 32, 3, 12, 2, "same"),         # many strips (both sweep directions)
    (1, 64, 96, 96, 64, 3, 4, (1, 2), 1),           # stride across only; whole-group consumers
    # passes of the strided build over channel slices and rank tiles
    (2, 1024, 14, 14, 96, 1, 16, 2, "same"),        # downsampling 1x1 layer, two slices of 512 channels
    (2, 64, 14, 14, 1000, 1, 24, 2, "same"),        # its adjoint contracts the 1000 output channels
    (2, 32, 20, 20, 48, 3, 48, 2, "same"),          # 48 ranks: two rank tiles, forward and adjoint
    (2, 48, 13, 13, 64, 3, 40, 1, "same"),          # stride 1, the reference's own layer: the plain passes
]


@pytest.mark.parametrize("dims", MATRIX_CASES, ids=lambda d: "x".join(map(str, d)))
def test_geometry_matrix_core_shapes(cp4, oracle, dims):
    N, C, H, W, T, Y, R, stride, padding = dims
    gen = torch.Generator(device="cuda").manual_seed(sum(map(ord, str(dims))))
    x = torch.rand((N, C, H, W), device="cuda", generator=gen) * 2 - 1
    fac = [torch.randn((d, R), device="cuda", generator=gen) * (R * C * Y * Y) ** -0.25
           for d in (T, C, Y, Y)]
    s = cp4.capi.shape_for(x.shape, *fac, 0)
    geom = cp4.geometry(s, stride, padding)
    y = cp4.conv2d_forward_ex(x, *fac, geom)
    want = oracle.forward_geom(x.cpu().numpy(), *[t.cpu().numpy() for t in fac],
                               oracle.Geometry(geom.stride_h, geom.stride_w, geom.pad_top,
                                               geom.pad_left, geom.out_h, geom.out_w))
    close_activation(y.cpu().numpy(), want, "forward vs oracle")
    dy = torch.randn(y.shape, device="cuda", generator=gen)
    yd, dxd, gd = dense_reference(x, dy, fac, geom)
    close_activation(y.cpu().numpy(), yd.astype(np.float32), "forward vs dense")
    dx = cp4.conv2d_backward_data_ex(dy, (H, W), *fac, geom)
    close_activation(dx.cpu().numpy(), dxd.astype(np.float32), "backward-data")
    grads = cp4.conv2d_backward_filter_ex(x, dy, *fac, geom)
    for got, wnt, k in zip(grads, gd, FACTORS):
        close_gradient(got.cpu().numpy(), wnt.astype(np.float32), "d" + k)
    # bias and activation on the strided output
    bias = torch.randn(T, device="cuda", generator=gen) * 0.1
    # (fused into the stores: the accumulators start at the bias, so the sum is
    # rounded in another order than y + bias)
    yb = cp4.conv2d_forward_ex(x, *fac, geom, bias=bias, activation="relu")
    wb = torch.relu(y + bias[None, :, None, None])
    assert float((yb - wb).abs().max()) <= 1e-5 * float(wb.abs().max())
    assert torch.equal(yb == 0, wb == 0) or float(wb[(yb == 0) != (wb == 0)].abs().max()) <= 1e-5
    cp4.device_status()


@pytest.mark.parametrize("dims", [(2, 32, 22, 26, 48, 3, 5, 12, (2, 3), (1, 2)),
                                  (1, 16, 30, 30, 32, 9, 9, 8, (2, 2), (4, 4)),
                                  (2, 48, 17, 19, 16, 2, 4, 40, (3, 2), (0, 1)),
                                  # unequal zeros before the image on the stride-1 canvas route
                                  # (stride 1; an odd channel count; more than 64 ranks)
                                  (2, 80, 22, 48, 4, 3, 3, 40, (1, 1), (1, 0)),
                                  (3, 48, 17, 6, 33, 3, 3, 2, (2, 2), (2, 1)),
                                  (1, 32, 30, 21, 32, 5, 5, 70, (2, 3), (0, 3))],
                         ids=lambda d: "x".join(map(str, d)))
def test_strided_factor_gradients_other_filters(cp4, dims):
    """Rectangular, even and 9x9 filters with a stride (the factor gradients run the
    strided matrix-core pass with its general tap kernel; forward and input gradient
    the general kernels), and layers with unequal zeros above and left of the image on
    the route over a stride-1 canvas.  Against float64 autograd of the dense strided
    convolution."""
    N, C, H, W, T, Y, X, R, (sh, sw), (pt, pl) = dims
    gen = torch.Generator(device="cuda").manual_seed(sum(map(ord, str(dims))))
    x = torch.rand((N, C, H, W), device="cuda", generator=gen) * 2 - 1
    fac = [torch.randn((d, R), device="cuda", generator=gen) * (R * C * Y * X) ** -0.25
           for d in (T, C, Y, X)]
    oh, ow = (H + 2 * pt - Y) // sh + 1, (W + 2 * pl - X) // sw + 1
    geom = cp4.Geometry(sh, sw, pt, pl, oh, ow)
    y = cp4.conv2d_forward_ex(x, *fac, geom)
    dy = torch.randn(y.shape, device="cuda", generator=gen)
    yd, dxd, gd = dense_reference(x, dy, fac, geom)
    close_activation(y.cpu().numpy(), yd.astype(np.float32), "forward")
    dx = cp4.conv2d_backward_data_ex(dy, (H, W), *fac, geom)
    close_activation(dx.cpu().numpy(), dxd.astype(np.float32), "backward-data")
    grads = cp4.conv2d_backward_filter_ex(x, dy, *fac, geom)
    for got, wnt, k in zip(grads, gd, FACTORS):
        close_gradient(got.cpu().numpy(), wnt.astype(np.float32), "d" + k)
    again = cp4.conv2d_backward_filter_ex(x, dy, *fac, geom)
    for a, b in zip(grads, again):
        assert torch.equal(a, b)                    # fixed summation order
    cp4.device_status()


def test_stride_two_at_the_headline_shape(cp4, oracle):
    """C3's shape at stride 2: against the oracle, and against every second row and
    column of the stride-1 layer for the padding that makes the two coincide."""
    from paralleltnnlayers_amd.configs import WORKLOADS, make_inputs
    w = WORKLOADS["C3"]
    a = make_inputs(w, seed=0)
    x = dev(a["x"])
    f = [dev(a[k]) for k in FACTORS]
    s = cp4.capi.shape_for(x.shape, *f, 0)
    geom = cp4.geometry(s, 2, "same")               # 56 -> 28: no zeros before, one row after
    assert (geom.pad_top, geom.out_h) == (0, 28)
    y = cp4.conv2d_forward_ex(x, *f, geom)
    og = oracle.Geometry(2, 2, geom.pad_top, geom.pad_left, 28, 28)
    want = oracle.forward_geom(a["x"], a["FK"], a["FC"], a["FH"], a["FW"], og)
    close_activation(y.cpu().numpy(), want, "stride 2, framework SAME")
    sym = cp4.geometry(s, 2, 1)                     # one zero on every side: windows at 2o - 1
    y2 = cp4.conv2d_forward_ex(x, *f, sym)
    full = cp4.conv2d_forward(x, *f, pad=1)
    ref = full[:, :, ::2, ::2]
    assert float((y2 - ref).abs().max()) <= 1e-5 * float(ref.abs().max())
    cp4.device_status()


def test_same_padding_layer_matches_the_framework_rule(cp4):
    """padding="same" at stride 2 on an even size through autograd: the windows of
    the reference's framework start at 2o (zeros only after the image)."""
    from paralleltnnlayers_amd import torch_ops
    gen = torch.Generator(device="cuda").manual_seed(3)
    mk = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    N, C, H, W, T, Y, R = 2, 32, 16, 18, 48, 3, 8
    x = mk(N, C, H, W).requires_grad_()
    fac = [(mk(d, R) / R ** 0.25).requires_grad_() for d in (T, C, Y, Y)]
    bias = mk(T).requires_grad_()
    y = torch_ops.cp4_conv2d(x, *fac, 1, bias=bias, activation="relu", stride=2, padding="same")
    assert tuple(y.shape) == (N, T, 8, 9)
    dy = mk(*y.shape)
    y.backward(dy)
    xd = x.detach().double().requires_grad_()
    fd = [t.detach().double().requires_grad_() for t in fac]
    bd = bias.detach().double().requires_grad_()
    K = torch.einsum("tr,cr,yr,xr->tcyx", *fd)
    yd = torch.relu(F.conv2d(F.pad(xd, (0, 1, 0, 1)), K, stride=2) + bd[None, :, None, None])
    yd.backward(dy.double())
    assert (y.detach().double() - yd.detach()).abs().max() <= 1e-4 * yd.detach().abs().max()
    for name, got, want in zip(("dx", "dFK", "dFC", "dFH", "dFW", "dbias"),
                               [x.grad] + [t.grad for t in fac] + [bias.grad],
                               [xd.grad] + [t.grad for t in fd] + [bd.grad]):
        tol = 1e-4 if name == "dx" else 1e-3
        assert (got.double() - want).abs().max() <= tol * want.abs().max(), name
