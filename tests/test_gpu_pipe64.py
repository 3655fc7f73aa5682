"""The single-pass kernel for ranks 33 - 64 (variant `mfma_bf16x3_pipe64`: the producer /
consumer strip kernel with a 64-rank plane kept as a ring in LDS) against the CPU oracle,
forward and backward-data (reference: Cuda_kernels/cp4Conv2dForward.cu:84-133,
cp4Conv2dBackwardData.cu:57-108), through the C ABI.  Tolerance: the forward bar,
|a-b| <= 1e-5 + 1e-4*|b| elementwise and max|a-b| <= 1e-4*max|b|."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NAME = "mfma_bf16x3_pipe64"


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


def layer(dims, seed=None):
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims) if seed is None else seed)
    x = (rng.random((N, C, H, W)) * 2 - 1).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) * np.float32((R * C * Y * Y) ** -0.25)
           for d in (T, C, Y, Y)]
    return x, dy, fac


# (N, C, H, W, pad, T, Y, R)
SHAPES = [
    (2, 64, 14, 14, 1, 64, 3, 64),       # workload C5's plane: the whole plane fits, nothing wraps
    (1, 32, 8, 8, 1, 32, 3, 40),         # 48-rank fragment tiles, one channel chunk per producer wave
    (2, 256, 28, 28, 1, 256, 3, 64),     # two chunks per producer wave
    (3, 100, 13, 15, 1, 70, 3, 33),      # odd rows and planes: single-pixel stores; ragged channels
    (2, 128, 9, 10, 0, 300, 1, 48),      # 1x1; more output-channel blocks than consumer waves
    (1, 200, 30, 31, 1, 96, 3, 57),      # ragged everything
    (2, 256, 56, 56, 1, 256, 3, 64),     # the plane is a ring: strips taller than the LDS holds
    (2, 16, 20, 64, 0, 40, 3, 64),       # pad 0 with a 3x3 filter
    (1, 256, 7, 7, 1, 512, 3, 64),       # output channels in slices (one strip on an idle chip)
    (2, 3, 17, 17, 2, 8, 3, 36),         # three channels, pad beyond (Y - 1) / 2
    (1, 64, 100, 20, 1, 64, 3, 48),      # tall narrow plane
    (1, 48, 40, 100, 1, 32, 3, 64),      # rows of more than three blocks: the widest ring a 64-rank plane allows
]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_pipe64_forward_and_backward_data(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, R = dims
    x, dy, fac = layer(dims)
    f = [dev(v) for v in fac]
    v = variant_index(cp4)
    y = cp4.conv2d_forward(dev(x), *f, pad=pad, variant=v)
    close(host(y), oracle.forward(x, *fac, pad), "forward")
    cp4.device_status()
    if T > 256:        # backward-data contracts the output channels first: beyond the kernel's 256
        return
    s = cp4.capi.shape_for(x.shape, *f, pad)
    cp4.tune_clear()
    try:
        cp4.set_tuned_choice(s, v, backward_data=True)
        assert cp4.default_variant(s, backward_data=True) == NAME
        dx = cp4.conv2d_backward_data(dev(dy), *f, pad=pad)
    finally:
        cp4.tune_clear()
    close(host(dx), oracle.backward_data(dy, *fac, pad), "backward-data")
    cp4.device_status()


# Strip heights entered as a tuned choice, with three and with two fragment tiles
# (schedule 1 / 0).  On the 56-pixel plane the 64-rank ring holds 10 - 13 blocks of 32
# cells, so strips from five rows on wrap it; heights that do not divide the 56 rows leave
# a shorter last strip, which sweeps bottom-up when its index is odd (5, 6, 10, 16, 20).
@pytest.mark.parametrize("R", [64, 48])
def test_pipe64_strip_heights_on_a_ring(cp4, oracle, R):
    dims = (2, 64, 56, 56, 1, 96, 3, R)
    N, C, H, W, pad, T, Y, _ = dims
    x, dy, fac = layer(dims)
    f = [dev(v) for v in fac]
    want = oracle.forward(x, *fac, pad)
    s = cp4.capi.shape_for(x.shape, *f, pad)
    v = variant_index(cp4)
    ran = 0
    cp4.tune_clear()
    try:
        for th in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 28, 56):
            for schedule in (1, 0):
                try:
                    cp4.set_tuned_choice(s, v, th, 0, schedule)
                except cp4.Cp4Error as e:           # this strip does not fit the LDS
                    assert e.status == cp4.capi.ERR_UNSUPPORTED
                    continue
                y = cp4.conv2d_forward(dev(x), *f, pad=pad)
                st, detail = cp4.device_status_detail()
                assert st == cp4.capi.OK, f"strip of {th} rows, schedule {schedule}: {detail}"
                close(host(y), want, f"strip of {th} rows, schedule {schedule}")
                ran += 1
    finally:
        cp4.tune_clear()
    assert ran >= 20


# More than 64 ranks or 256 input channels: the kernel once per (tile of 64 ranks, slice of up
# to 256 channels) with y += after the first pass, the 32-rank build for a last tile of up to 32.
PASSES = [
    (2, 320, 20, 20, 1, 64, 3, 64),      # two channel slices of one rank tile
    (2, 64, 28, 28, 1, 96, 3, 96),       # 64 ranks, then 32 on the 32-rank build
    (1, 600, 12, 12, 1, 48, 3, 100),     # tiles of 64 and 36 ranks x three slices of 208 channels
    (1, 1024, 7, 7, 0, 32, 1, 129),      # 1x1: two tiles x four slices, a last rank in two slices of 512
    (2, 128, 56, 56, 1, 128, 3, 128),    # two tiles on a wrapped ring
]


@pytest.mark.parametrize("dims", PASSES, ids=lambda d: "x".join(map(str, d)))
def test_pipe64_in_passes(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, R = dims
    x, dy, fac = layer(dims)
    f = [dev(v) for v in fac]
    v = {n: i for i, n, _ in cp4.forward_variants()}[NAME + "_passes"]
    y = cp4.conv2d_forward(dev(x), *f, pad=pad, variant=v)
    close(host(y), oracle.forward(x, *fac, pad), "forward")
    s = cp4.capi.shape_for(x.shape, *f, pad)
    cp4.tune_clear()
    try:
        try:
            cp4.set_tuned_choice(s, v, backward_data=True)
        except cp4.Cp4Error as e:       # up to 64 ranks and 256 output channels: a single pass
            assert e.status == cp4.capi.ERR_UNSUPPORTED and R <= 64 and T <= 256
        dx = cp4.conv2d_backward_data(dev(dy), *f, pad=pad)
    finally:
        cp4.tune_clear()
    close(host(dx), oracle.backward_data(dy, *fac, pad), "backward-data")
    cp4.device_status()


def test_pipe64_is_the_default_for_33_to_64_ranks(cp4):
    def shape(N, C, H, W, T, R, Y=3):
        return cp4.capi.Shape(N=N, H=H, W=W, pad=Y // 2, T=T, C=C, Y=Y, X=Y, Rank=R)
    cp4.tune_clear()
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 64)) == NAME
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 48)) == NAME
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 33)) == NAME
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 64), backward_data=True) == NAME
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 64, Y=1)) == NAME
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 32)) == "mfma_bf16x3_pipe"
    # 5x5 filters: passes of 32 ranks
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 64, Y=5)) == "mfma_bf16x3_pipe_rank_passes"
    # tiles of 64 ranks beyond 64 ranks, slices of 256 channels beyond 256 channels
    assert cp4.default_variant(shape(32, 256, 56, 56, 256, 128)) == NAME + "_passes"
    assert cp4.default_variant(shape(32, 512, 28, 28, 512, 64)) == NAME + "_passes"
    q = cp4.plan_query(shape(32, 256, 56, 56, 256, 64), "forward")
    assert q["variant"] == NAME and q["strip_rows"] >= 1 and q["workgroups"] >= 200


def test_pipe64_wait_timeout_is_reported(cp4, oracle):
    """The kernel's waits (producers behind the ring's readers, the eighths of a block,
    consumers behind blocks and arrivals) with the bound at one poll: the fault is
    reported, every wave ends, and the next launch is right again."""
    dims = (2, 128, 56, 56, 1, 64, 3, 64)
    x, dy, fac = layer(dims)
    f = [dev(v) for v in fac]
    v = variant_index(cp4)
    assert cp4.device_status_detail()[0] == cp4.capi.OK
    cp4.set_spin_limit(1)
    try:
        cp4.conv2d_forward(dev(x), *f, pad=1, variant=v)
        st, detail = cp4.device_status_detail()
    finally:
        cp4.set_spin_limit(0)
    assert st == cp4.capi.ERR_DEVICE and detail[0] != 0
    y = cp4.conv2d_forward(dev(x), *f, pad=1, variant=v)
    cp4.device_status()
    close(host(y), oracle.forward(x, *fac, 1), "after the fault")


def test_pipe64_refuses_what_it_cannot_run(cp4):
    g = torch.Generator(device="cuda").manual_seed(3)
    v = variant_index(cp4)
    for dims in [(1, 32, 8, 8, 2, 32, 5, 64),      # 5x5
                 (1, 32, 8, 8, 1, 32, 3, 32),      # 32 ranks: the 32-rank kernel's
                 (1, 32, 8, 8, 1, 32, 3, 65),      # 65 ranks
                 (1, 272, 8, 8, 1, 32, 3, 64)]:    # more than 256 input channels
        N, C, H, W, pad, T, Y, R = dims
        x = torch.randn(N, C, H, W, device="cuda", generator=g)
        f = [torch.randn(d, R, device="cuda", generator=g) / 4 for d in (T, C, Y, Y)]
        with pytest.raises(cp4.Cp4Error) as ei:
            cp4.conv2d_forward(x, *f, pad=pad, variant=v)
        assert ei.value.status == cp4.capi.ERR_UNSUPPORTED
        assert cp4.conv2d_forward(x, *f, pad=pad).shape == (N, T, H, W)
