"""The few-channel tiled kernel (variant `mfma_bf16x3_few`: persistent small workgroups over
2-D tiles, taps and output contraction in registers; up to 64 input channels and 16 ranks,
planes of any width) against the CPU oracle, forward and backward-data (reference:
Cuda_kernels/cp4Conv2dForward.cu:84-133, cp4Conv2dBackwardData.cu:57-108), through the C ABI.
Tolerance: the forward bar, |a-b| <= 1e-5 + 1e-4*|b| elementwise and max|a-b| <= 1e-4*max|b|."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NAME = "mfma_bf16x3_few"


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


def variant_index(cp4):
    return {n: v for v, n, _ in cp4.forward_variants()}[NAME]


def close(got, want, what=""):
    err = np.abs(got - want)
    assert err.max() <= 1e-4 * np.abs(want).max(), f"{what}: normalised {err.max() / np.abs(want).max():.2e}"
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(want)), f"{what}: elementwise {err.max():.2e}"


def layer(dims):
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = (rng.random((N, C, H, W)) * 2 - 1).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) * np.float32((R * C * Y * Y) ** -0.25)
           for d in (T, C, Y, Y)]
    return x, dy, fac


# (N, C, H, W, pad, T, Y, R)
SHAPES = [
    (1, 16, 32, 32, 1, 16, 3, 8),      # workload C1
    (2, 16, 40, 70, 1, 16, 3, 16),     # a column tile past the right edge
    (3, 5, 13, 15, 1, 7, 3, 3),        # odd rows: single-pixel stores; ragged channels and ranks
    (2, 32, 33, 130, 2, 40, 5, 16),    # 5x5, two channel chunks, two output-channel blocks
    (1, 64, 20, 64, 0, 70, 1, 12),     # 1x1, four channel chunks, three output-channel blocks
    (2, 3, 64, 200, 1, 1, 3, 16),      # three channels to one
    (1, 16, 9, 300, 0, 16, 3, 5),      # no padding: the last rows and columns read zeros
    (2, 48, 17, 31, 2, 33, 3, 9),      # pad beyond (Y - 1) / 2
    (1, 8, 100, 20, 1, 8, 5, 16),      # tall narrow plane
    (4, 16, 7, 7, 1, 16, 3, 1),        # rank 1, planes smaller than a tile
    (2, 16, 130, 257, 1, 16, 3, 16),   # odd width on a wide plane, several tiles per workgroup
]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_few_forward_and_backward_data(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, R = dims
    x, dy, fac = layer(dims)
    f = [dev(v) for v in fac]
    v = variant_index(cp4)
    want = oracle.forward(x, *fac, pad)
    s = cp4.capi.shape_for(x.shape, *f, pad)
    cp4.tune_clear()
    try:
        # the kernel's own tile, then tiles of every width with eight and with four waves
        # (schedule 0 / 2), one of them taller than the plane
        for th, tw, schedule in ((0, 0, 1), (1, 64, 2), (2, 32, 0), (4, 64, 2), (8, 64, 0),
                                 (3, 128, 2), (16, 32, 0), (5, 64, 0)):
            try:
                cp4.set_tuned_choice(s, v, th, tw, schedule)
            except cp4.Cp4Error as e:               # this tile does not fit the LDS (5x5, 64 channels)
                assert e.status == cp4.capi.ERR_UNSUPPORTED and (th, tw) != (0, 0)
                continue
            close(host(cp4.conv2d_forward(dev(x), *f, pad=pad)), want, f"forward, tile {th}x{tw}")
        cp4.tune_clear()
        if T <= 64:     # backward-data contracts the output channels first
            cp4.set_tuned_choice(s, v, backward_data=True)
            assert cp4.default_variant(s, backward_data=True) == NAME
            dx = cp4.conv2d_backward_data(dev(dy), *f, pad=pad)
            close(host(dx), oracle.backward_data(dy, *fac, pad), "backward-data")
    finally:
        cp4.tune_clear()
    cp4.device_status()


def test_few_with_bias_and_relu(cp4, oracle):
    dims = (2, 16, 50, 90, 1, 24, 3, 16)
    x, dy, fac = layer(dims)
    f = [dev(v) for v in fac]
    b = np.linspace(-0.2, 0.2, 24).astype(np.float32)
    s = cp4.capi.shape_for(x.shape, *f, 1)
    cp4.tune_clear()
    try:
        cp4.set_tuned_choice(s, variant_index(cp4))
        y = cp4.conv2d_forward_bias_act(dev(x), *f, dev(b), "relu", pad=1)
    finally:
        cp4.tune_clear()
    close(host(y), np.maximum(oracle.forward(x, *fac, 1) + b[None, :, None, None], 0), "bias + relu")
    cp4.device_status()


def test_few_is_the_default_on_large_planes_with_few_channels(cp4):
    def shape(N, C, H, W, T, R, Y=3):
        return cp4.capi.Shape(N=N, H=H, W=W, pad=Y // 2, T=T, C=C, Y=Y, X=Y, Rank=R)
    cp4.tune_clear()
    assert cp4.default_variant(shape(16, 16, 512, 512, 16, 16)) == NAME       # the reference's all_scales row
    assert cp4.default_variant(shape(32, 16, 56, 56, 16, 16)) == NAME
    assert cp4.default_variant(shape(4, 32, 256, 256, 32, 16)) == NAME
    assert cp4.default_variant(shape(16, 16, 512, 512, 16, 16), backward_data=True) == NAME
    assert cp4.default_variant(shape(128, 3, 512, 512, 1, 16)) == "dense_small_valu"   # the recomposed filter stays
    assert cp4.default_variant(shape(1, 16, 32, 32, 16, 8)) == "mfma_bf16x3_light"     # workload C1
    assert cp4.default_variant(shape(16, 64, 32, 32, 64, 16)) == "mfma_bf16x3_pipe"    # workload C2
    assert cp4.default_variant(shape(8, 64, 224, 224, 64, 16)) == "mfma_bf16x3_pipe"   # 64 input channels
    assert cp4.default_variant(shape(16, 16, 512, 512, 16, 32)) != NAME                # 32 ranks
    q = cp4.plan_query(shape(16, 16, 512, 512, 16, 16), "forward")
    assert q["variant"] == NAME and q["strip_rows"] >= 1 and 256 <= q["workgroups"] <= 1024


def test_few_refuses_what_it_cannot_run(cp4):
    g = torch.Generator(device="cuda").manual_seed(3)
    v = variant_index(cp4)
    for dims in [(1, 16, 8, 8, 3, 16, 7, 8),       # 7x7
                 (1, 16, 8, 8, 1, 16, 3, 17),      # 17 ranks
                 (1, 80, 8, 8, 1, 16, 3, 8)]:      # more than 64 input channels
        N, C, H, W, pad, T, Y, R = dims
        x = torch.randn(N, C, H, W, device="cuda", generator=g)
        f = [torch.randn(d, R, device="cuda", generator=g) / 4 for d in (T, C, Y, Y)]
        with pytest.raises(cp4.Cp4Error) as ei:
            cp4.conv2d_forward(x, *f, pad=pad, variant=v)
        assert ei.value.status == cp4.capi.ERR_UNSUPPORTED
        assert cp4.conv2d_forward(x, *f, pad=pad).shape == (N, T, H, W)
