"""The autograd binding (replacement of the reference's TF custom-op boundary,
Kernels/cp4_conv_nchw.cc:6-108) against PyTorch's own dense convolution on the
recomposed filter: forward values and all five gradients."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import paralleltnnlayers_amd as p
    p.lib()
    from paralleltnnlayers_amd import torch_ops
    return torch_ops


def recomposed(FK, FC, FH, FW):
    return torch.einsum("tr,cr,yr,xr->tcyx", FK, FC, FH, FW)


@pytest.mark.parametrize("dims", [(2, 16, 12, 14, 24, 3, 8), (1, 64, 20, 20, 64, 5, 16),
                                  (3, 5, 9, 9, 7, 1, 3)],
                         ids=lambda d: "x".join(map(str, d)))
def test_gradients_match_dense_autograd(ops, dims):
    N, C, H, W, T, Y, R = dims
    g = torch.Generator(device="cuda").manual_seed(sum(dims))
    mk = lambda *s: torch.randn(*s, device="cuda", generator=g)
    x = mk(N, C, H, W).requires_grad_()
    fac = [(mk(d, R) / R ** 0.25).requires_grad_() for d in (T, C, Y, Y)]
    dy = mk(N, T, H, W)
    y = ops.cp4_conv2d(x, *fac, Y // 2)
    y.backward(dy)
    got = [x.grad.clone()] + [f.grad.clone() for f in fac]

    # float64 dense reference through PyTorch autograd on the recomposed filter
    xd = x.detach().double().requires_grad_()
    fd = [f.detach().double().requires_grad_() for f in fac]
    yd = torch.nn.functional.conv2d(xd, recomposed(*fd), padding=Y // 2)
    yd.backward(dy.double())
    want = [xd.grad] + [f.grad for f in fd]
    assert (y.detach().double() - yd.detach()).abs().max() <= 1e-4 * yd.detach().abs().max()
    for name, a, b in zip(("dx", "dFK", "dFC", "dFH", "dFW"), got, want):
        tol = 1e-4 if name == "dx" else 1e-3
        assert (a.double() - b).abs().max() <= tol * b.abs().max(), name


def test_only_requested_gradients(ops):
    x = torch.randn(1, 8, 6, 6, device="cuda")
    fac = [torch.randn(d, 4, device="cuda") for d in (8, 8, 3, 3)]
    fac[0].requires_grad_()
    ops.cp4_conv2d(x, *fac, 1).sum().backward()
    assert fac[0].grad is not None and all(f.grad is None for f in fac[1:]) and x.grad is None


def test_padding_other_than_same_gives_the_smaller_output(ops):
    """pad = 0 with a 3x3 filter: the layer's output is (H - 2) x (W - 2), as a dense
    convolution's, and differentiable (the geometry entry points)."""
    x = torch.randn(1, 8, 6, 6, device="cuda", requires_grad=True)
    fac = [torch.randn(d, 4, device="cuda", requires_grad=True) for d in (8, 8, 3, 3)]
    y = ops.cp4_conv2d(x, *fac, 0)
    want = torch.nn.functional.conv2d(x.detach(), recomposed(*[f.detach() for f in fac]))
    assert y.shape == want.shape == (1, 8, 4, 4)
    assert (y.detach() - want).abs().max() <= 1e-4 * want.abs().max()
    y.sum().backward()
    assert x.grad is not None and all(f.grad is not None for f in fac)


def test_layer_trains(ops):
    """A few SGD steps on a CP4Conv2d layer lower a regression loss: forward,
    both backward passes and the optimizer see consistent tensors."""
    torch.manual_seed(0)
    layer = ops.CP4Conv2d(16, 16, 3, rank=8)
    target = ops.CP4Conv2d(16, 16, 3, rank=8)
    x = torch.randn(4, 16, 10, 10, device="cuda")
    with torch.no_grad():
        want = target(x)
    opt = torch.optim.SGD(layer.parameters(), lr=0.05)
    losses = []
    for _ in range(30):
        opt.zero_grad()
        loss = ((layer(x) - want) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < 0.7 * losses[0]
    K = layer.dense_filter()
    assert K.shape == (16, 16, 3, 3)
    dense = torch.nn.functional.conv2d(x, K, padding=1)
    assert (layer(x).detach() - dense).abs().max() <= 1e-4 * dense.abs().max()


def test_strided_layer_matches_dense_strided_conv(ops):
    """stride 2 = every second row and column of the stride-1 result, which for
    "same" padding is PyTorch's strided convolution with the recomposed filter;
    the gradients flow through the subsampling."""
    g = torch.Generator(device="cuda").manual_seed(11)
    mk = lambda *s: torch.randn(*s, device="cuda", generator=g)
    N, C, H, W, T, Y, R = 2, 16, 13, 16, 24, 3, 8
    x = mk(N, C, H, W).requires_grad_()
    fac = [(mk(d, R) / R ** 0.25).requires_grad_() for d in (T, C, Y, Y)]
    y = ops.cp4_conv2d(x, *fac, 1, stride=2)
    dy = mk(*y.shape)
    y.backward(dy)
    xd = x.detach().double().requires_grad_()
    fd = [f.detach().double().requires_grad_() for f in fac]
    yd = torch.nn.functional.conv2d(xd, recomposed(*fd), padding=1, stride=2)
    assert yd.shape == y.shape
    yd.backward(dy.double())
    assert (y.detach().double() - yd.detach()).abs().max() <= 1e-4 * yd.detach().abs().max()
    for name, a, b in zip(("dx", "dFK", "dFC", "dFH", "dFW"), [x.grad] + [f.grad for f in fac],
                          [xd.grad] + [f.grad for f in fd]):
        tol = 1e-4 if name == "dx" else 1e-3
        assert (a.double() - b).abs().max() <= tol * b.abs().max(), name


def test_bfloat16_activations_through_autograd(ops):
    """bfloat16 x: forward, input gradient and factor gradients run the library's
    bfloat16-activation entry points; compared with float64 autograd on the same
    (bfloat16-representable) inputs within the bfloat16 rounding of y, dx and dy."""
    g = torch.Generator(device="cuda").manual_seed(21)
    mk = lambda *s: torch.randn(*s, device="cuda", generator=g)
    N, C, H, W, T, Y, R = 2, 32, 12, 16, 48, 3, 8
    x = mk(N, C, H, W).to(torch.bfloat16).requires_grad_()
    fac = [(mk(d, R) / R ** 0.25).requires_grad_() for d in (T, C, Y, Y)]
    y = ops.cp4_conv2d(x, *fac, 1)
    assert y.dtype == torch.bfloat16
    dy = mk(N, T, H, W).to(torch.bfloat16)
    y.backward(dy)
    assert x.grad.dtype == torch.bfloat16 and fac[0].grad.dtype == torch.float32
    xd = x.detach().double().requires_grad_()
    fd = [f.detach().double().requires_grad_() for f in fac]
    yd = torch.nn.functional.conv2d(xd, recomposed(*fd), padding=1)
    yd.backward(dy.double())
    assert (y.detach().double() - yd.detach()).abs().max() <= 2.0 ** -7 * yd.detach().abs().max()
    assert (x.grad.double() - xd.grad).abs().max() <= 2.0 ** -7 * xd.grad.abs().max()
    for name, a, b in zip(("dFK", "dFC", "dFH", "dFW"), [f.grad for f in fac], [f.grad for f in fd]):
        assert (a.double() - b).abs().max() <= 1e-3 * b.abs().max(), name
