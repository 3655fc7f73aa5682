"""Forward with the fused bias / activation epilogue (cp4_conv2d_forward_bias_act)
against the CPU oracle's forward followed by the epilogue's closed form
y = max(conv + bias[t], 0): through the producer / consumer kernel's epilogue
build where that kernel runs the shape, and through the other variants followed
by the in-place epilogue kernel elsewhere.  Tolerance: the forward bar
(1e-5 + 1e-4*|b| elementwise, 1e-4 normalised)."""
import numpy as np
import pytest
import torch

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


# (N, C, H, W, pad, T, Y, R)
SHAPES = [
    (2, 64, 28, 28, 1, 64, 3, 16),     # producer / consumer kernel, cached output factor
    (1, 256, 56, 56, 1, 256, 3, 32),   # one image of the ResNet-stage workload
    (2, 32, 15, 17, 2, 72, 5, 8),      # odd width, output channels not a multiple of 32
    (1, 320, 14, 14, 1, 300, 3, 32),   # factor in LDS, more channel blocks than consumer waves
    (3, 5, 9, 9, 1, 7, 3, 3),          # general kernel + in-place epilogue
    (2, 64, 14, 14, 1, 64, 3, 48),     # rank above 32: strip kernel + in-place epilogue
    (1, 24, 20, 224, 1, 40, 3, 16),    # wide plane: the tiled build, which carries the epilogue too
    (2, 64, 30, 150, 1, 64, 3, 4),     # wide plane, whole pixel groups per consumer wave
    (2, 3, 70, 130, 1, 1, 3, 16),      # three channels to one: the recomposed-filter kernel's own epilogue
    (1, 4, 33, 47, 2, 12, 5, 8),       # ... with two groups of output channels, ragged tiles
    (2, 16, 28, 28, 1, 40, 3, 8),      # small layer: the light kernel's own epilogue
    (1, 32, 20, 30, 2, 64, 5, 16),     # ... 5x5, two blocks of output channels
]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("mode", ["bias", "relu", "bias+relu"])
def test_epilogue_matches_oracle(cp4, oracle, dims, mode):
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / np.sqrt(R) for d in (T, C, Y, Y)]
    conv = oracle.forward(x, *fac, pad)
    bias = (rng.standard_normal(T) * np.abs(conv).mean()).astype(np.float32)
    want = conv + (bias[None, :, None, None] if "bias" in mode else 0.0)
    if "relu" in mode:
        want = np.maximum(want, 0.0)
    got = cp4.conv2d_forward_bias_act(dev(x), *[dev(f) for f in fac],
                                      bias=dev(bias) if "bias" in mode else None,
                                      activation="relu" if "relu" in mode else None, pad=pad)
    # the bar is relative to the pre-activation magnitude: ReLU zeroes may not hide errors
    pre = conv + (bias[None, :, None, None] if "bias" in mode else 0.0)
    err = np.abs(host(got) - want)
    assert err.max() <= 1e-4 * np.abs(pre).max()
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(pre))
    if "relu" in mode:
        assert host(got).min() >= 0.0 and (host(got) == 0).mean() > 0.2


def test_no_epilogue_is_the_plain_forward(cp4):
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(2, 64, 20, 20, device="cuda", generator=g)
    fac = [torch.randn(d, 16, device="cuda", generator=g) / 2 for d in (64, 64, 3, 3)]
    a = cp4.conv2d_forward_bias_act(x, *fac, bias=None, activation=None, pad=1)
    b = cp4.conv2d_forward(x, *fac, pad=1)
    assert torch.equal(a, b)


def test_unknown_activation_is_refused(cp4):
    import ctypes
    x = torch.randn(1, 8, 6, 6, device="cuda")
    fac = [torch.randn(d, 4, device="cuda") for d in (8, 8, 3, 3)]
    y = torch.empty(1, 8, 6, 6, device="cuda")
    s = cp4.capi.shape_for(x.shape, *fac, 1)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = cp4.lib().cp4_conv2d_forward_bias_act(ctypes.byref(s), p(x), *[p(f) for f in fac],
                                                None, 7, p(y), None)
    assert rc == cp4.capi.ERR_UNSUPPORTED


def test_autograd_with_bias_and_relu():
    from paralleltnnlayers_amd import torch_ops
    g = torch.Generator(device="cuda").manual_seed(9)
    mk = lambda *s: torch.randn(*s, device="cuda", generator=g)
    N, C, H, W, T, Y, R = 2, 16, 12, 14, 24, 3, 8
    x = mk(N, C, H, W).requires_grad_()
    fac = [(mk(d, R) / R ** 0.25).requires_grad_() for d in (T, C, Y, Y)]
    bias = mk(T).requires_grad_()
    dy = mk(N, T, H, W)
    y = torch_ops.cp4_conv2d(x, *fac, 1, bias, "relu")
    y.backward(dy)
    got = [x.grad, *[f.grad for f in fac], bias.grad]
    xd = x.detach().double().requires_grad_()
    fd = [f.detach().double().requires_grad_() for f in fac]
    bd = bias.detach().double().requires_grad_()
    K = torch.einsum("tr,cr,yr,xr->tcyx", *fd)
    yd = torch.relu(torch.nn.functional.conv2d(xd, K, bd, padding=1))
    yd.backward(dy.double())
    want = [xd.grad, *[f.grad for f in fd], bd.grad]
    assert (y.detach().double() - yd.detach()).abs().max() <= 1e-4 * yd.detach().abs().max()
    for name, a, b in zip(("dx", "dFK", "dFC", "dFH", "dFW", "dbias"), got, want):
        tol = 1e-4 if name == "dx" else 1e-3
        assert (a.double() - b).abs().max() <= tol * b.abs().max(), name
