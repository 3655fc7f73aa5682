"""The 3-factor CP sibling op (pointwise K0 [C,R], depthwise K1 [Y,X,R], pointwise
K2 [R,T]; the reference's Conv2dCpFusedNchw, Kernels/cp_fused_nchw.cc:6-30) through
the C ABI: forward against the CPU oracle's restatement of the reference's Python
layer, to the forward bar (1e-5 + 1e-4*|b| elementwise, 1e-4 normalised); the expanded
CP4 factors bit-exactly against their definition; input and factor gradients against
PyTorch float64 autograd of the dense convolution on the einsum kernel (1e-4 / 1e-3
normalised, the backward-data / backward-filter bars)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


def operands(dims, uniform=False):
    N, C, H, W, Y, R, T = dims
    rng = np.random.default_rng(sum(dims))
    draw = (lambda *s: rng.uniform(size=s)) if uniform else (lambda *s: rng.standard_normal(s))
    x = draw(N, C, H, W).astype(np.float32)
    K0 = (draw(C, R) / np.sqrt(C)).astype(np.float32)
    K1 = (draw(Y, Y, R) / Y).astype(np.float32)
    K2 = (draw(R, T) / np.sqrt(R)).astype(np.float32)
    return x, K0, K1, K2


# (N, C, H, W, Y, R, T)
SHAPES = [
    (1, 16, 32, 32, 3, 6, 16),     # the reference's only shape (test/test_conv2d_cp.py:12-15)
    (4, 64, 28, 28, 3, 10, 64),    # expanded rank 30: producer / consumer kernel
    (2, 128, 28, 28, 3, 16, 96),   # expanded rank 48: two rank passes
    (2, 32, 15, 17, 5, 6, 40),     # 5x5, odd plane, expanded rank 30
    (1, 24, 14, 14, 3, 24, 24),    # expanded rank 72: general kernel
    (3, 5, 9, 9, 1, 3, 7),         # 1x1 depthwise filter
]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_cp3_forward_matches_oracle(cp4, oracle, dims):
    x, K0, K1, K2 = operands(dims, uniform=dims == SHAPES[0])
    pad = dims[4] // 2
    want = oracle.cp3_forward(x, K0, K1, K2, pad)
    got = host(cp4.cp3_conv2d_forward(dev(x), dev(K0), dev(K1), dev(K2), pad=pad))
    err = np.abs(got - want)
    assert (err <= 1e-5 + 1e-4 * np.abs(want)).all(), err.max()
    assert err.max() <= 1e-4 * np.abs(want).max()


# shapes on the 2-D-tap build of the producer / consumer kernel (R <= 32, 3x3 or 1x1)
NATIVE = [
    (2, 64, 28, 28, 3, 16, 64),    # split consumer roles (R <= 16, at most 4 channel blocks)
    (2, 256, 56, 56, 3, 32, 256),  # full rank tile, registers-resident factor slice
    (3, 40, 13, 13, 3, 21, 72),    # odd plane, ragged channels and ranks
    (1, 320, 14, 14, 3, 12, 300),  # factor fragments in LDS
    (2, 16, 20, 20, 1, 8, 24),     # 1x1, one-chunk producers
    (2, 64, 20, 20, 3, 40, 48),    # 40 ranks: two passes of the 2-D-tap build with y +=
    (1, 1024, 10, 10, 3, 12, 32),  # 1024 input channels: two channel slices
]


@pytest.mark.parametrize("dims", NATIVE, ids=lambda d: "x".join(map(str, d)))
def test_cp3_native_taps_agree_with_expanded_factors(cp4, oracle, dims):
    """Forward and input gradient of the one-pass kernel against the same passes run on
    the expanded CP4 factors (whose kernels the oracle pins), to the forward bar; the
    forward of the smaller shapes also against the oracle directly."""
    x, K0, K1, K2 = operands(dims)
    N, C, H, W, Y, R, T = dims
    pad = Y // 2
    dK = [dev(a) for a in (K0, K1, K2)]
    fac = cp4.cp3_expand_factors(*dK)
    y = host(cp4.cp3_conv2d_forward(dev(x), *dK, pad=pad))
    y_ref = host(cp4.conv2d_forward(dev(x), *fac, pad=pad))
    assert np.abs(y - y_ref).max() <= 1e-5 * np.abs(y_ref).max()
    if N * C * H * W * R <= 2 ** 24:
        want = oracle.cp3_forward(x, K0, K1, K2, pad)
        err = np.abs(y - want)
        assert (err <= 1e-5 + 1e-4 * np.abs(want)).all() and err.max() <= 1e-4 * np.abs(want).max()
    dy = np.random.default_rng(5).standard_normal((N, T, H, W)).astype(np.float32)
    dx = host(cp4.cp3_conv2d_backward_data(dev(dy), *dK, pad=pad))
    dx_ref = host(cp4.conv2d_backward_data(dev(dy), *fac, pad=pad))
    assert np.abs(dx - dx_ref).max() <= 1e-5 * np.abs(dx_ref).max()
    # adjoint identity ("same" padding): <dy, conv(x)> = <conv^T(dy), x>
    lhs = float((dy.astype(np.float64) * y).sum()); rhs = float((dx.astype(np.float64) * x).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), np.sqrt(float((dy ** 2).sum()) * float((y ** 2).sum())) * 1e-2)


def test_cp3_expanded_factors_exact(cp4):
    _, K0, K1, K2 = operands((1, 7, 4, 4, 3, 5, 9))
    FK, FC, FH, FW = (host(t) for t in cp4.cp3_expand_factors(dev(K0), dev(K1), dev(K2)))
    Y, X, R = K1.shape
    for i in range(Y):
        cols = slice(i * R, (i + 1) * R)
        np.testing.assert_array_equal(FK[:, cols], K2.T)
        np.testing.assert_array_equal(FC[:, cols], K0)
        np.testing.assert_array_equal(FW[:, cols], K1[i])
        np.testing.assert_array_equal(FH[:, cols], np.eye(Y, dtype=np.float32)[:, i:i + 1].repeat(R, 1))


@pytest.mark.parametrize("dims", [(2, 16, 12, 12, 3, 6, 16), (2, 64, 14, 14, 3, 16, 32),
                                  (1, 8, 10, 11, 5, 4, 12)],
                         ids=lambda d: "x".join(map(str, d)))
def test_cp3_autograd_matches_float64_dense(cp4, dims):
    from paralleltnnlayers_amd.torch_ops import cp3_conv2d
    x, K0, K1, K2 = operands(dims)
    pad = dims[4] // 2
    leaves = [dev(a).requires_grad_() for a in (x, K0, K1, K2)]
    y = cp3_conv2d(*leaves, pad)
    dy = torch.randn(y.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(3))
    y.backward(dy)

    ref = [torch.from_numpy(a).double().requires_grad_() for a in (x, K0, K1, K2)]
    dense = torch.einsum("cr,ijr,rt->tcij", ref[1], ref[2], ref[3])
    yr = F.conv2d(ref[0], dense, padding=pad)
    yr.backward(dy.cpu().double())
    assert (host(y.detach()) - yr.detach().numpy()).__abs__().max() <= 1e-4 * yr.abs().max().item()
    for name, got, want, tol in zip(("dx", "dK0", "dK1", "dK2"), leaves, ref,
                                    (1e-4, 1e-3, 1e-3, 1e-3)):
        g, w = host(got.grad), want.grad.numpy()
        assert g.shape == w.shape, name
        assert np.abs(g - w).max() <= tol * np.abs(w).max(), name


def test_cp3_rejects_small_workspace(cp4):
    import ctypes
    x, K0, K1, K2 = (dev(a) for a in operands((1, 4, 6, 6, 3, 2, 4)))
    s = cp4.cp3_shape_for(x.shape, K0, K1, K2, 1)
    y = torch.empty((1, 4, 6, 6), device="cuda")
    ws = torch.empty(16, device="cuda", dtype=torch.uint8)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = cp4.lib().cp3_conv2d_forward(ctypes.byref(s), p(x), p(K0), p(K1), p(K2), p(y), p(ws), 16,
                                      None)
    assert rc == 4      # CP4_ERR_WORKSPACE


def test_cp3_layer_trains(cp4):
    """A few SGD steps on the layer reduce a regression loss: forward, input gradient and
    folded factor gradients fit together."""
    from paralleltnnlayers_amd.torch_ops import CP3Conv2d
    torch.manual_seed(0)
    layer = CP3Conv2d(32, 48, 3, rank=12)
    teacher = CP3Conv2d(32, 48, 3, rank=12)
    x = torch.randn(4, 32, 16, 16, device="cuda")
    with torch.no_grad():
        target = teacher(x)
    opt = torch.optim.SGD(layer.parameters(), lr=0.05)
    losses = []
    for _ in range(30):
        opt.zero_grad()
        loss = ((layer(x) - target) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < 0.7 * losses[0], losses[::6]


@pytest.mark.parametrize("dims", SHAPES + [(4, 64, 56, 56, 3, 16, 64), (2, 32, 12, 12, 3, 40, 48)],
                         ids=lambda d: "x".join(map(str, d)))
def test_cp3_backward_filter_entry_point(cp4, dims):
    """cp3_conv2d_backward_filter (K1 applied as it is where the matrix-core pass takes
    the shape, the rank-Y*R rewriting elsewhere) against the rewriting spelled out
    through the C ABI - cp3_expand_factors, the CP4 pass, cp3_fold_gradients - and
    against float64 autograd of the dense convolution."""
    x, K0, K1, K2 = operands(dims)
    pad = dims[4] // 2
    xd, k0, k1, k2 = (dev(a) for a in (x, K0, K1, K2))
    dy = torch.randn((dims[0], dims[6], dims[2], dims[3]), device="cuda",
                     generator=torch.Generator("cuda").manual_seed(5))
    got = cp4.cp3_conv2d_backward_filter(xd, dy, k0, k1, k2, pad=pad)
    FK, FC, FH, FW = cp4.cp3_expand_factors(k0, k1, k2)
    dFK, dFC, _, dFW = cp4.conv2d_backward_filter(xd, dy, FK, FC, FH, FW, pad=pad)
    via = cp4.cp3_fold_gradients(dFK, dFC, dFW, K1.shape[0])
    ref = [torch.from_numpy(a).double().requires_grad_() for a in (x, K0, K1, K2)]
    dense = torch.einsum("cr,ijr,rt->tcij", ref[1], ref[2], ref[3])
    (F.conv2d(ref[0], dense, padding=pad) * dy.cpu().double()).sum().backward()
    for name, g, v, r in zip(("dK0", "dK1", "dK2"), got, via, ref[1:]):
        w = r.grad.numpy()
        assert np.abs(host(g) - w).max() <= 1e-3 * np.abs(w).max(), name + " vs float64"
        assert np.abs(host(g) - host(v)).max() <= 1e-4 * np.abs(w).max(), name + " vs rewriting"
    # bit-reproducible: no floating-point atomics on either path
    again = cp4.cp3_conv2d_backward_filter(xd, dy, k0, k1, k2, pad=pad)
    for a, b in zip(got, again):
        assert torch.equal(a, b)
