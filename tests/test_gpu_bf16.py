"""bfloat16 activations in memory (cp4_conv2d_forward_bf16 /
cp4_conv2d_backward_data_bf16): fp32 factors and arithmetic, one rounding at the
store.  The oracle runs in fp32 on the same bf16-representable inputs; the
result may differ from it by the final rounding to bfloat16 (half a unit in the
last place: 2^-8 relative) plus the fp32 bar of the pass."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


def bf16_values(rng, shape, relu=False):
    """float32 array whose values are exactly representable in bfloat16."""
    t = torch.from_numpy(rng.standard_normal(shape).astype(np.float32))
    if relu:
        t = torch.relu(t)
    return t.to(torch.bfloat16)


def assert_bf16_close(got_bf16, want_f32, what):
    got = got_bf16.float().cpu().numpy()
    scale = float(np.abs(want_f32).max())
    err = np.abs(got - want_f32)
    bound = 2.0 ** -8 * np.abs(want_f32) * 1.01 + 1e-4 * scale * 2.0 ** -8 + 1e-4 * np.abs(want_f32)
    assert np.all(err <= bound), f"{what}: max excess {(err - bound).max():.3e} (scale {scale:.3e})"


# (N, C, H, W, pad, T, Y, R)
SHAPES = [
    (2, 64, 28, 28, 1, 64, 3, 16),
    (1, 256, 56, 56, 1, 256, 3, 32),     # one image of the ResNet-stage workload
    (2, 32, 15, 17, 2, 72, 5, 8),        # odd width: element-wise stores
    (1, 320, 14, 14, 1, 304, 3, 32),     # factor in LDS, partly filled last channel block
    (3, 48, 9, 12, 3, 40, 7, 12),        # 7x7, channels padded to 64
    (2, 16, 32, 32, 0, 16, 1, 8),        # 1x1
]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_forward_and_backward_data_bf16(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = bf16_values(rng, (N, C, H, W), relu=True)
    dy = bf16_values(rng, (N, T, H, W))
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    f = [torch.from_numpy(v).cuda() for v in fac]
    s = cp4.capi.shape_for(x.shape, *f, pad)
    assert cp4.bf16_supported(s) and cp4.bf16_supported(s, backward_data=True)
    y = cp4.conv2d_forward_bf16(x.cuda(), *f, pad=pad)
    assert y.dtype == torch.bfloat16
    assert_bf16_close(y, oracle.forward(x.float().numpy(), *fac, pad), "forward")
    dx = cp4.conv2d_backward_data_bf16(dy.cuda(), *f, pad=pad)
    assert_bf16_close(dx, oracle.backward_data(dy.float().numpy(), *fac, pad), "backward-data")


def test_forward_bf16_epilogue(cp4, oracle):
    N, C, H, W, pad, T, Y, R = 2, 64, 20, 20, 1, 96, 3, 16
    rng = np.random.default_rng(7)
    x = bf16_values(rng, (N, C, H, W))
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    conv = oracle.forward(x.float().numpy(), *fac, pad)
    bias = (rng.standard_normal(T) * np.abs(conv).mean()).astype(np.float32)
    want = np.maximum(conv + bias[None, :, None, None], 0.0)
    y = cp4.conv2d_forward_bf16(x.cuda(), *[torch.from_numpy(v).cuda() for v in fac],
                                bias=torch.from_numpy(bias).cuda(), activation="relu", pad=pad)
    got = y.float().cpu().numpy()
    pre = np.abs(conv + bias[None, :, None, None])
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * 1.01 * pre + 2e-4 * pre + 1e-6)
    assert got.min() >= 0.0 and (got == 0).mean() > 0.2


def test_bf16_matches_fp32_kernel_then_rounding(cp4):
    """Same inputs through the fp32 entry point, rounded afterwards: the two
    differ at most where the fp32 results straddle a rounding boundary."""
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(2, 128, 28, 28, device="cuda", generator=g).to(torch.bfloat16)
    fac = [torch.randn(d, 32, device="cuda", generator=g) / 4 for d in (128, 128, 3, 3)]
    a = cp4.conv2d_forward_bf16(x, *fac, pad=1).float()
    b = cp4.conv2d_forward(x.float(), *fac, pad=1).to(torch.bfloat16).float()
    differ = (a != b).float().mean().item()
    assert differ < 1e-3
    assert (a - b).abs().max().item() <= 2.0 ** -7 * b.abs().max().item()


# even rows: producers load pixel pairs; plane lengths of an odd and an even number
# of 32-pixel blocks, one strip and several (odd strips sweep backwards)
PAIR_SHAPES = [
    (2, 64, 40, 22, 1, 64, 3, 16),
    (1, 128, 13, 30, 1, 96, 3, 32),
    (3, 32, 9, 34, 2, 40, 5, 8),
    (2, 16, 57, 12, 0, 16, 1, 4),
    (1, 320, 21, 18, 1, 64, 3, 24),      # factor in LDS
]


@pytest.mark.parametrize("dims", PAIR_SHAPES, ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("half", [False, True], ids=["bf16", "f16"])
def test_pixel_pair_producers_match_the_element_path(cp4, oracle, dims, half):
    """With an even row length the producers of the 16-bit builds load two pixels
    per lane.  An x that starts two bytes off a 4-byte boundary takes the
    element-by-element path instead: same products in the same order, so the two
    results are bit-identical, and both meet the oracle's bar."""
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    dt = torch.float16 if half else torch.bfloat16
    x = torch.from_numpy(rng.standard_normal((N, C, H, W)).astype(np.float32)).to(dt)
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    f = [torch.from_numpy(v).cuda() for v in fac]
    fwd = cp4.conv2d_forward_f16 if half else cp4.conv2d_forward_bf16
    buf = torch.zeros(x.numel() + 2, dtype=dt, device="cuda")
    aligned = buf[:x.numel()].view(x.shape)
    shifted = buf[1:1 + x.numel()].view(x.shape)
    assert aligned.data_ptr() % 4 == 0 and shifted.data_ptr() % 4 == 2
    aligned.copy_(x)
    ya = fwd(aligned, *f, pad=pad).clone()
    shifted.copy_(x)
    ys = fwd(shifted, *f, pad=pad)
    assert torch.equal(ya, ys)
    want = oracle.forward(x.float().numpy(), *fac, pad)
    got = ya.float().cpu().numpy()
    ulp = 2.0 ** -11 if half else 2.0 ** -8
    scale = float(np.abs(want).max())
    assert np.all(np.abs(got - want) <= ulp * 1.01 * np.abs(want) + 1e-4 * np.abs(want) + 1e-5 * scale)


def test_bf16_unsupported_shapes_are_refused(cp4):
    x = torch.randn(1, 8, 6, 6, device="cuda").to(torch.bfloat16)
    fac = [torch.randn(d, 40, device="cuda") for d in (8, 8, 3, 3)]     # rank 40 > 32
    s = cp4.capi.shape_for(x.shape, *fac, 1)
    assert not cp4.bf16_supported(s)
    with pytest.raises(cp4.Cp4Error) as e:
        cp4.conv2d_forward_bf16(x, *fac, pad=1)
    assert e.value.status == cp4.capi.ERR_UNSUPPORTED


def assert_gradient_close(got, want, what):
    scale = float(np.abs(want).max())
    err = np.abs(got - want)
    assert np.all(err <= 1e-3 * np.abs(want) + 1e-4 * scale), f"{what}: elementwise {err.max():.3e}"
    assert err.max() <= 1e-3 * scale, f"{what}: normalised {err.max() / scale:.3e}"


# (N, C, H, W, pad, T, Y, R): channel counts multiples of 16
FILTER_SHAPES = [
    (2, 64, 28, 28, 1, 64, 3, 16),
    (1, 256, 56, 56, 1, 256, 3, 32),
    (1, 320, 14, 14, 1, 304, 3, 32),
    (2, 16, 32, 32, 0, 16, 1, 8),
    (4, 32, 7, 7, 1, 48, 3, 8),          # odd plane: element-wise staging
    (8, 256, 14, 14, 1, 256, 3, 64),     # two rank tiles, the backward-filter workload's shape
    (3, 48, 9, 10, 2, 80, 5, 20),        # plane not a multiple of 4 pixels
]


@pytest.mark.parametrize("dims", FILTER_SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_backward_filter_bf16(cp4, oracle, dims):
    """x and dy bfloat16 in memory, gradients fp32: the same bar as the fp32 pass
    (the arithmetic is the same exact-product, fp32-accumulate one)."""
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims) + 1)
    x = bf16_values(rng, (N, C, H, W))
    dy = bf16_values(rng, (N, T, H, W))
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    f = [torch.from_numpy(v).cuda() for v in fac]
    got = cp4.conv2d_backward_filter_bf16(x.cuda(), dy.cuda(), *f, pad=pad)
    want = oracle.backward_filter(x.float().numpy(), dy.float().numpy(), *fac, pad)
    for g, wnt, name in zip(got, want, ("dFK", "dFC", "dFH", "dFW")):
        assert g.dtype == torch.float32
        assert_gradient_close(g.cpu().numpy(), wnt, name)
    # bit-identical to the fp32 entry point on the widened inputs? not required: the
    # fp32 path splits its activations into three parts whose lower two are zero here,
    # so the sums agree to rounding order
    ref = cp4.conv2d_backward_filter(x.float().cuda(), dy.float().cuda(), *f, pad=pad)
    for g, r in zip(got, ref):
        assert (g - r).abs().max().item() <= 1e-5 * r.abs().max().item()


@pytest.mark.parametrize("dims", FILTER_SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_backward_filter_f16(cp4, oracle, dims):
    """x and dy IEEE half in memory, gradients fp32: a half value is two bf16 parts, so
    the products stay exact and the bar is the fp32 pass's."""
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims) + 2)
    x = torch.from_numpy(rng.standard_normal((N, C, H, W)).astype(np.float32)).half()
    dy = torch.from_numpy(rng.standard_normal((N, T, H, W)).astype(np.float32)).half()
    x[0, 0, 0, 0] = 6.1e-5          # a value near the bottom of the normal range, and a subnormal
    dy[0, 0, 0, 1] = 3.0e-7
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    f = [torch.from_numpy(v).cuda() for v in fac]
    got = cp4.conv2d_backward_filter_f16(x.cuda(), dy.cuda(), *f, pad=pad)
    want = oracle.backward_filter(x.float().numpy(), dy.float().numpy(), *fac, pad)
    for g, wnt, name in zip(got, want, ("dFK", "dFC", "dFH", "dFW")):
        assert g.dtype == torch.float32
        assert_gradient_close(g.cpu().numpy(), wnt, name)
    ref = cp4.conv2d_backward_filter(x.float().cuda(), dy.float().cuda(), *f, pad=pad)
    for g, r in zip(got, ref):
        assert (g - r).abs().max().item() <= 1e-5 * r.abs().max().item()


def test_backward_filter_bf16_unsupported(cp4):
    x = torch.randn(1, 24, 6, 6, device="cuda").to(torch.bfloat16)      # 24 channels: not a multiple of 16
    dy = torch.randn(1, 16, 6, 6, device="cuda").to(torch.bfloat16)
    fac = [torch.randn(d, 4, device="cuda") for d in (16, 24, 3, 3)]
    with pytest.raises(cp4.Cp4Error) as e:
        cp4.conv2d_backward_filter_bf16(x, dy, *fac, pad=1)
    assert e.value.status == cp4.capi.ERR_UNSUPPORTED
