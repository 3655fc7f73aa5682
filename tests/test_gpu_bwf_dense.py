"""Backward-filter variant 3 (`dense_gradient_tiles`: the dense filter gradient
dK[k,c,i,j] = sum dy[k,h,w] x[c,h+i-pad,w+j-pad] over tiles of pixels, with plain
multiply-adds or as a GEMM over the pixels on the matrix cores, then the chain rule onto the
four factors; up to 64 channels a side) against the CPU oracle's factor-by-factor gradients (reference: Cuda_kernels/cp4Conv2dBackwardFilter.cu:64-257), through the C ABI.
Tolerance: the backward-filter bar, |a-b| <= 1e-3*|b| + 1e-6*max|b| elementwise and
max|a-b| <= 1e-3*max|b|."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

FACTORS = ("FK", "FC", "FH", "FW")


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


def close(got, want, what):
    scale = float(np.abs(want).max())
    err = np.abs(got - want)
    assert np.all(err <= 1e-3 * np.abs(want) + 1e-6 * scale), f"{what}: elementwise {err.max():.3e}"
    assert err.max() <= 1e-3 * scale, f"{what}: normalised {err.max() / scale:.3e}"


# (N, C, H, W, pad, T, Y, R)
SHAPES = [
    (2, 3, 64, 200, 1, 1, 3, 16),      # the reference's sweep family: three channels to one
    (1, 16, 40, 70, 1, 16, 3, 16),     # 256 channel pairs; tiles past the right edge
    (3, 5, 13, 15, 1, 7, 3, 3),        # ragged channel blocks, odd planes
    (2, 8, 33, 130, 2, 8, 5, 16),      # 5x5
    (1, 12, 20, 64, 0, 20, 1, 12),     # 1x1
    (2, 3, 17, 17, 2, 8, 3, 36),       # pad beyond (Y - 1) / 2, more ranks than channels
    (1, 1, 100, 20, 1, 1, 3, 16),      # one channel each side
    (4, 16, 7, 7, 1, 16, 3, 1),        # planes smaller than a tile, rank 1
    (2, 4, 9, 300, 0, 2, 3, 5),        # no padding with a 3x3 filter
    (2, 8, 130, 257, 1, 8, 3, 8),      # several tiles per workgroup
    # the matrix-core tile kernel
    (2, 32, 31, 45, 1, 32, 3, 16),     # nine column blocks over two groups of waves; odd width: cell-by-cell loads
    (1, 40, 20, 36, 1, 40, 3, 8),      # two blocks of output channels, the second ragged
    (2, 24, 30, 32, 2, 24, 5, 8),      # 5x5, nineteen column blocks
    (1, 48, 17, 40, 0, 32, 1, 16),     # 1x1 with 80 channels in all: waves across more column blocks than there are
    (1, 64, 17, 40, 0, 64, 1, 16),     # 1x1 with 64 channels a side: 32 x 32 blocks, two blocks of output channels
    (1, 50, 20, 20, 1, 33, 3, 16),     # ragged on both sides
    (3, 16, 70, 132, 1, 16, 3, 16),    # several tiles per workgroup, 16-byte loads, tiles past both edges
    (2, 20, 40, 64, 0, 12, 3, 4),      # no padding with a 3x3 filter
    (1, 6, 9, 16, 2, 64, 3, 5),        # pad beyond (Y - 1) / 2; a plane smaller than a tile
    (1, 4, 800, 800, 1, 4, 3, 4),      # 640,000 pixels, four channels a side
    (2, 12, 64, 96, 1, 16, 5, 8),      # 16 x 16 blocks, 5x5: nineteen column blocks over four groups of waves
    (2, 16, 24, 40, 1, 32, 3, 8),      # 16 x 16 blocks, two blocks of output channels
    (1, 20, 30, 44, 1, 25, 3, 6),      # the same, ragged on both sides
    (2, 4, 1, 1, 0, 4, 1, 3),          # planes of one pixel
    (1, 3, 2, 3, 2, 2, 3, 2),          # planes narrower than four pixels, pad 2
    (300, 6, 5, 8, 1, 6, 3, 4),        # more images than workgroups
    (4, 3, 512, 512, 1, 1, 3, 16),     # three channels to one on a million pixels
    (1, 24, 701, 603, 1, 2, 3, 4),     # plain multiply-adds by choice (ten million cells), cell-by-cell loads (odd width)
]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_dense_gradient_tiles(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = (rng.random((N, C, H, W)) * 2 - 1).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) * np.float32((R * C) ** -0.25)
           for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    assert cp4.backward_filter_variants()[3] == "dense_gradient_tiles"
    wants = oracle.backward_filter(x, dy, *fac, pad)
    # the route's own tile kernel, then each of the two where it can run the shape
    # (0: plain multiply-adds, T * C <= 256; 1: matrix cores)
    try:
        for which in (-1, 0, 1):
            cp4.set_backward_filter_tile_kernel(which)
            first = None
            for rep in range(2):       # bit-reproducible: no atomics anywhere
                grads = cp4.conv2d_backward_filter(dev(x), dev(dy), *f, pad=pad, variant=3)
                got = [host(g) for g in grads]
                for g, w, k in zip(got, wants, FACTORS):
                    close(g, w, f"d{k}, tile kernel {which}")
                if first is None:
                    first = got
                else:
                    assert all(np.array_equal(a, b) for a, b in zip(first, got))
    finally:
        cp4.set_backward_filter_tile_kernel(-1)
    cp4.device_status()


def test_dense_gradient_is_the_default_for_few_channels(cp4):
    def shape(N, C, H, W, T, R, Y=3):
        return cp4.capi.Shape(N=N, H=H, W=W, pad=Y // 2, T=T, C=C, Y=Y, X=Y, Rank=R)
    cp4.tune_clear()
    name = "dense_gradient_tiles"
    assert cp4.plan_query(shape(128, 3, 512, 512, 1, 16), "backward_filter")["variant"] == name
    assert cp4.plan_query(shape(16, 16, 512, 512, 16, 16), "backward_filter")["variant"] == name
    assert cp4.plan_query(shape(8, 8, 256, 256, 8, 16), "backward_filter")["variant"] == name
    assert cp4.plan_query(shape(16, 32, 256, 256, 32, 16), "backward_filter")["variant"] == name
    assert cp4.plan_query(shape(16, 3, 112, 112, 64, 16), "backward_filter")["variant"] == name
    assert cp4.plan_query(shape(1, 16, 32, 32, 16, 8), "backward_filter")["variant"] != name   # workload C1
    # many channels, and workload C5: the matrix-core variants
    assert cp4.plan_query(shape(32, 256, 56, 56, 256, 32), "backward_filter")["variant"] != name
    assert cp4.plan_query(shape(64, 256, 14, 14, 256, 64), "backward_filter")["variant"] != name


def test_dense_gradient_unaligned_pointers(cp4, oracle):
    """x and dy four bytes off a 16-byte boundary: the tile kernel loads cell by cell."""
    dims = (2, 16, 24, 64, 1, 16, 3, 8)
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(11)
    x = (rng.random((N, C, H, W)) * 2 - 1).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / 2 for d in (T, C, Y, Y)]
    xb = torch.zeros(x.size + 1, device="cuda")
    db = torch.zeros(dy.size + 1, device="cuda")
    xd = xb[1:].view(x.shape)
    dd = db[1:].view(dy.shape)
    xd.copy_(dev(x))
    dd.copy_(dev(dy))
    assert xd.data_ptr() % 16 == 4 and dd.data_ptr() % 16 == 4
    grads = cp4.conv2d_backward_filter(xd, dd, *[dev(v) for v in fac], pad=pad, variant=3)
    for g, w, k in zip(grads, oracle.backward_filter(x, dy, *fac, pad), FACTORS):
        close(host(g), w, f"d{k}")
    cp4.device_status()


def test_dense_gradient_refuses_many_channels(cp4):
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(1, 128, 8, 8, device="cuda", generator=g)
    dy = torch.randn(1, 32, 8, 8, device="cuda", generator=g)
    f = [torch.randn(d, 8, device="cuda", generator=g) / 4 for d in (32, 128, 3, 3)]
    with pytest.raises(cp4.Cp4Error) as ei:
        cp4.conv2d_backward_filter(x, dy, *f, pad=1, variant=3)
    assert ei.value.status == cp4.capi.ERR_UNSUPPORTED
