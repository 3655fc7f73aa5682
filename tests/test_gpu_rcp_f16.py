"""The reshaped-CP sibling op (Kernels/rcp_fused_nchw.cc:6-12) and the
half-precision (float16) activation entry points, through the C ABI.

rCP: forward against the oracle's restatement of the reference's test
(test/test_conv2d_rcp.py:38-41; pinned to torch's dense conv2d in
tests/test_oracle.py) at the reference's own shape and others, input gradient
through the adjoint identity, all gradients against float64 autograd of the
dense convolution on einsum('axr,byr,hwr->hwabxy').

float16: against the fp32 oracle on the same float16-representable inputs, within
the one rounding of the stored result (2^-11 relative) plus the forward bar.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

from paralleltnnlayers_amd.configs import WORKLOADS, make_inputs  # noqa: E402


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


# N, S0, S1, T0, T1, H, W, Y, R
RCP_CASES = [
    (1, 4, 4, 4, 4, 32, 32, 3, 11),       # the reference's op: 1 x (4,4) x 32 x 32, rank 11
    (2, 2, 3, 3, 2, 9, 11, 3, 4),
    (3, 4, 8, 2, 5, 14, 14, 5, 6),        # 32 -> 10 channels, 5x5
    (1, 3, 3, 5, 5, 20, 24, 1, 7),        # 1x1 filter, 25 output channels (four groups of 8)
    (2, 12, 12, 6, 4, 14, 18, 3, 5),      # 144 -> 24 channels at 3x3: the filter's weights stream
                                          # through LDS by channel chunk (forward)
    (1, 4, 5, 16, 10, 12, 12, 3, 4),      # 20 -> 160 channels: the same for the input gradient
    (1, 8, 8, 8, 8, 10, 10, 5, 3),        # 64 -> 64 at 5x5: both
]


@pytest.mark.parametrize("dims", RCP_CASES, ids=lambda d: "x".join(map(str, d)))
def test_rcp_all_passes(cp4, oracle, dims):
    N, S0, S1, T0, T1, H, W, Y, R = dims
    gen = torch.Generator(device="cuda").manual_seed(sum(dims))
    x = torch.rand((N, S0 * S1, H, W), device="cuda", generator=gen)
    K0 = torch.rand((S0, T0, R), device="cuda", generator=gen)
    K1 = torch.rand((S1, T1, R), device="cuda", generator=gen)
    KC = torch.randn((Y, Y, R), device="cuda", generator=gen) / R
    pad = Y // 2
    y = cp4.rcp_conv2d_forward(x, K0, K1, KC, pad=pad)
    want = oracle.rcp_forward(x.cpu().numpy(), K0.cpu().numpy(), K1.cpu().numpy(), KC.cpu().numpy(), pad)
    err = np.abs(y.cpu().numpy() - want)
    assert err.max() <= 1e-4 * np.abs(want).max()
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(want))
    # gradients: float64 autograd of the dense convolution the reference's test builds
    dy = torch.randn(y.shape, device="cuda", generator=gen)
    xd = x.double().cpu().requires_grad_()
    kd = [t.double().cpu().requires_grad_() for t in (K0, K1, KC)]
    Kd = torch.einsum("axr,byr,hwr->hwabxy", *kd).reshape(Y, Y, S0 * S1, T0 * T1).permute(3, 2, 0, 1)
    yd = F.conv2d(xd, Kd, padding=pad)
    (yd * dy.double().cpu()).sum().backward()
    dx = cp4.rcp_conv2d_backward_data(dy, K0, K1, KC, pad=pad)
    assert (dx.double().cpu() - xd.grad).abs().max() <= 1e-4 * xd.grad.abs().max()
    # adjoint identity <y, dy> = <x, dx>
    lhs, rhs = float((y.double() * dy.double()).sum()), float((x.double() * dx.double()).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs), 1.0)
    for got, ref, name in zip(cp4.rcp_conv2d_backward_filter(x, dy, K0, K1, KC, pad=pad), kd,
                              ("dK0", "dK1", "dKC")):
        assert (got.double().cpu() - ref.grad).abs().max() <= 1e-3 * ref.grad.abs().max(), name


def test_rcp_autograd_layer(cp4):
    from paralleltnnlayers_amd import torch_ops
    gen = torch.Generator(device="cuda").manual_seed(9)
    x = torch.rand((2, 16, 12, 12), device="cuda", generator=gen).requires_grad_()
    ks = [torch.rand((4, 4, 5), device="cuda", generator=gen).requires_grad_() for _ in range(2)]
    kc = (torch.randn((3, 3, 5), device="cuda", generator=gen) / 5).requires_grad_()
    y = torch_ops.rcp_conv2d(x, ks[0], ks[1], kc, 1)
    y.square().sum().backward()
    assert x.grad is not None and all(k.grad is not None for k in ks) and kc.grad is not None
    xd = x.detach().double().requires_grad_()
    kd = [k.detach().double().requires_grad_() for k in ks + [kc]]
    Kd = torch.einsum("axr,byr,hwr->hwabxy", *kd).reshape(3, 3, 16, 16).permute(3, 2, 0, 1)
    F.conv2d(xd, Kd, padding=1).square().sum().backward()
    assert (x.grad.double() - xd.grad).abs().max() <= 1e-3 * xd.grad.abs().max()
    for got, ref in zip(ks + [kc], kd):
        assert (got.grad.double() - ref.grad).abs().max() <= 1e-3 * ref.grad.abs().max()


def test_rcp_argument_errors(cp4):
    import ctypes
    L = cp4.lib()
    s = cp4.capi.Shape(N=1, H=8, W=8, pad=1, T=16, C=16, Y=3, X=3, Rank=4)
    one = ctypes.c_void_p(256)
    bad = cp4.capi.RcpDims(4, 4, 4, 3)                       # T0*T1 != T
    assert L.rcp_conv2d_forward(ctypes.byref(s), ctypes.byref(bad), one, one, one, one, one, one,
                                1 << 20, None) == cp4.capi.ERR_SHAPE
    ok = cp4.capi.RcpDims(4, 4, 4, 4)
    assert L.rcp_conv2d_forward(ctypes.byref(s), ctypes.byref(ok), one, one, one, one, one, one,
                                16, None) == cp4.capi.ERR_WORKSPACE


# ---- float16 activations -------------------------------------------------------
@pytest.mark.parametrize("name", ["C1", "C2", "C4"])
def test_float16_forward_and_backward_data(cp4, oracle, name):
    w = WORKLOADS[name]
    a = make_inputs(w, seed=0)
    f = [torch.from_numpy(a[k]).cuda() for k in ("FK", "FC", "FH", "FW")]
    fa = [a[k] for k in ("FK", "FC", "FH", "FW")]
    x16 = torch.from_numpy(a["x"]).cuda().half()
    dy16 = torch.from_numpy(a["dy"]).cuda().half()
    s = cp4.capi.shape_for(x16.shape, *f, w.pad)
    assert cp4.bf16_supported(s)

    def within_one_rounding(got16, want, what):
        got = got16.float().cpu().numpy()
        scale = np.abs(want).max()
        err = np.abs(got - want)
        bound = 2.0 ** -11 * np.abs(want) * 1.01 + 1e-4 * scale * 2.0 ** -11 + 1e-4 * np.abs(want) + 1e-7
        assert np.all(err <= bound), f"{what}: {err.max():.3e}"
        assert err.max() <= (2.0 ** -11 + 1e-4) * scale

    y = cp4.conv2d_forward_f16(x16, *f, pad=w.pad)
    assert y.dtype == torch.float16
    within_one_rounding(y, oracle.forward(x16.float().cpu().numpy(), *fa, w.pad), "forward")
    dx = cp4.conv2d_backward_data_f16(dy16, *f, pad=w.pad)
    within_one_rounding(dx, oracle.backward_data(dy16.float().cpu().numpy(), *fa, w.pad), "backward-data")
    # bias and ReLU in the same launch
    bias = torch.randn(w.T, device="cuda") * 0.01
    yb = cp4.conv2d_forward_f16(x16, *f, bias=bias, activation="relu", pad=w.pad)
    ref = torch.relu(torch.from_numpy(oracle.forward(x16.float().cpu().numpy(), *fa, w.pad)).cuda()
                     + bias[None, :, None, None])
    within_one_rounding(yb, ref.cpu().numpy(), "bias + relu")
    cp4.device_status()


def test_float16_through_autograd(cp4):
    from paralleltnnlayers_amd import torch_ops
    gen = torch.Generator(device="cuda").manual_seed(21)
    mk = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    N, C, H, W, T, Y, R = 2, 32, 12, 16, 48, 3, 8
    x = mk(N, C, H, W).half().requires_grad_()
    fac = [(mk(d, R) / R ** 0.25).requires_grad_() for d in (T, C, Y, Y)]
    y = torch_ops.cp4_conv2d(x, *fac, 1)
    assert y.dtype == torch.float16
    dy = mk(N, T, H, W).half()
    y.backward(dy)
    assert x.grad.dtype == torch.float16 and fac[0].grad.dtype == torch.float32
    xd = x.detach().double().requires_grad_()
    fd = [f.detach().double().requires_grad_() for f in fac]
    yd = F.conv2d(xd, torch.einsum("tr,cr,yr,xr->tcyx", *fd), padding=1)
    yd.backward(dy.double())
    assert (y.detach().double() - yd.detach()).abs().max() <= 2.0 ** -10 * yd.detach().abs().max()
    assert (x.grad.double() - xd.grad).abs().max() <= 2.0 ** -10 * xd.grad.abs().max()
    for name, got, want in zip(("dFK", "dFC", "dFH", "dFW"), fac, fd):
        assert (got.grad.double() - want.grad).abs().max() <= 1e-3 * want.grad.abs().max(), name
