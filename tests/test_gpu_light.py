"""The light kernel (variant `mfma_bf16x3_light`: three short phases in small workgroups,
the default for small problems with few channels) against the CPU oracle, forward and
backward-data (reference: Cuda_kernels/cp4Conv2dForward.cu:84-133,
cp4Conv2dBackwardData.cu:57-108), through the C ABI with the variant entered as the
shape's tuned choice.  Tolerance: the forward bar, |a-b| <= 1e-5 + 1e-4*|b| elementwise
and max|a-b| <= 1e-4*max|b|."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NAME = "mfma_bf16x3_light"


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


def close(got, want):
    err = np.abs(got - want)
    assert err.max() <= 1e-4 * np.abs(want).max()
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(want))


# (N, C, H, W, pad, T, Y, R)
SHAPES = [
    (1, 16, 32, 32, 1, 16, 3, 8),      # workload C1
    (2, 24, 10, 14, 1, 40, 3, 5),      # ragged channel chunk, rank not a multiple of four
    (3, 16, 9, 6, 0, 8, 3, 3),         # no padding: the output's last rows and columns read zeros
    (2, 72, 17, 22, 2, 33, 5, 20),     # 5x5, two rank chunks, five channel chunks (ring refill)
    (1, 8, 5, 4, 0, 8, 1, 4),          # 1x1, half a channel chunk
    (2, 48, 40, 64, 1, 96, 3, 32),     # 32 ranks; more blocks than waves
    (1, 200, 13, 20, 1, 100, 3, 17),   # thirteen channel chunks
    (4, 16, 33, 18, 2, 16, 3, 7),      # pad beyond (Y - 1) / 2
    (1, 3, 12, 16, 1, 2, 3, 16),       # three channels to two
    (5, 32, 7, 2, 1, 32, 3, 16),       # two-pixel rows
]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_light_forward_and_backward_data(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / np.sqrt(R) for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    v = variant_index(cp4)
    y = cp4.conv2d_forward(dev(x), *f, pad=pad, variant=v)
    close(host(y), oracle.forward(x, *fac, pad))
    s = cp4.capi.shape_for(dy.shape, *f, pad)
    cp4.tune_clear()
    try:
        cp4.set_tuned_choice(s, v, backward_data=True)
        assert cp4.default_variant(s, backward_data=True) == NAME
        dx = cp4.conv2d_backward_data(dev(dy), *f, pad=pad)
    finally:
        cp4.tune_clear()
    close(host(dx), oracle.backward_data(dy, *fac, pad))
    cp4.device_status()


@pytest.mark.parametrize("th", [1, 2, 3, 5, 8])
def test_light_strip_heights(cp4, oracle, th):
    """Every strip height the planner may pick gives the same result (tuned tile rows)."""
    N, C, H, W, pad, T, Y, R = 3, 32, 19, 24, 1, 48, 3, 12
    rng = np.random.default_rng(th)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / np.sqrt(R) for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    s = cp4.capi.shape_for(x.shape, *f, pad)
    cp4.tune_clear()
    try:
        cp4.set_tuned_choice(s, variant_index(cp4), tile_rows=th)
        y = cp4.conv2d_forward(dev(x), *f, pad=pad)
    finally:
        cp4.tune_clear()
    close(host(y), oracle.forward(x, *fac, pad))


def test_light_is_the_default_for_small_layers_only(cp4):
    def shape(N, C, H, W, T, R, Y=3):
        return cp4.capi.Shape(N=N, H=H, W=W, pad=Y // 2, T=T, C=C, Y=Y, X=Y, Rank=R)
    cp4.tune_clear()
    assert cp4.default_variant(shape(1, 16, 32, 32, 16, 8)) == NAME            # workload C1
    assert cp4.default_variant(shape(8, 16, 56, 56, 16, 16)) == NAME
    assert cp4.default_variant(shape(16, 8, 32, 32, 8, 16)) == NAME            # not the recomposed filter
    assert cp4.default_variant(shape(16, 64, 32, 32, 64, 16)) == "mfma_bf16x3_pipe"   # workload C2
    assert cp4.default_variant(shape(32, 16, 56, 56, 16, 16)) == "mfma_bf16x3_few"    # 100,000 pixels
    assert cp4.default_variant(shape(8, 16, 56, 56, 16, 32)) == "mfma_bf16x3_pipe"    # 32 ranks


def test_light_refuses_what_it_cannot_run(cp4):
    """Odd row lengths (its stores are pixel pairs) and ranks beyond 32: CP4_ERR_UNSUPPORTED
    for the variant by number, while the default choice runs the shape elsewhere."""
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(1, 16, 9, 7, device="cuda", generator=g)
    f = [torch.randn(d, 8, device="cuda", generator=g) / 2 for d in (16, 16, 3, 3)]
    with pytest.raises(cp4.Cp4Error):
        cp4.conv2d_forward(x, *f, pad=1, variant=variant_index(cp4))
    assert cp4.conv2d_forward(x, *f, pad=1).shape == (1, 16, 9, 7)
    f40 = [torch.randn(d, 40, device="cuda", generator=g) / 2 for d in (16, 16, 3, 3)]
    x2 = torch.randn(1, 16, 8, 8, device="cuda", generator=g)
    with pytest.raises(cp4.Cp4Error):
        cp4.conv2d_forward(x2, *f40, pad=1, variant=variant_index(cp4))
