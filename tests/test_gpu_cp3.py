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
