"""GPU parity tests: the HIP path, called through the C ABI, against the CPU
oracle, the committed golden vectors and size-independent properties.

Tolerances (written out here as the bar for this path):
  forward / backward-data : |a-b| <= 1e-5 + 1e-4*|b| elementwise, and
                            max|a-b| <= 1e-4 * max|b| so that small-magnitude
                            outputs cannot pass vacuously;
  backward-filter         : |a-b| <= 1e-3*|b| + 1e-6*max|b| elementwise (the
                            floor only keeps entries that cancel to ~0 from
                            dividing by nothing), and max|a-b| <= 1e-3 * max|b|.
"""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from paralleltnnlayers_amd.configs import WORKLOADS, make_inputs  # noqa: E402

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "cp4_golden.npz"))
GOLD_CASES = sorted({k.split(".")[0] for k in GOLD.files})
FACTORS = ("FK", "FC", "FH", "FW")


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_activation_close(got, want, what=""):
    scale = float(np.abs(want).max())
    err = np.abs(got - want)
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(want)), f"{what}: elementwise, max err {err.max():.3e}"
    assert err.max() <= 1e-4 * scale, f"{what}: normalised {err.max() / scale:.3e} (scale {scale:.3e})"


def assert_gradient_close(got, want, what=""):
    scale = float(np.abs(want).max())
    err = np.abs(got - want)
    assert np.all(err <= 1e-3 * np.abs(want) + 1e-6 * scale), f"{what}: elementwise {err.max():.3e}"
    assert err.max() <= 1e-3 * scale, f"{what}: normalised {err.max() / scale:.3e}"


def gold(name):
    g = {k: GOLD[f"{name}.{k}"] for k in
         ("x", "dy", "y", "dx", "dFK", "dFC", "dFH", "dFW") + FACTORS}
    g["pad"] = int(GOLD[name + ".shape"][3])
    return g


def variants_for(cp4, x_shape, f, pad):
    s = cp4.capi.shape_for(x_shape, f["FK"], f["FC"], f["FH"], f["FW"], pad)
    return [v for v, _, ok in cp4.forward_variants(s) if ok]


def filter_variants(cp4, x, dy, f, pad):
    """Backward-filter variants that accept this shape: -1 (library's choice),
    0 (general) and, where they qualify, 1 (matrix cores, four launches),
    2 (matrix cores, tap step fused into the gradient GEMMs) and 3 (few channels: the
    dense filter gradient over tiles of pixels, then the chain rule)."""
    out = [-1, 0]
    for v in (1, 2, 3):
        try:
            cp4.conv2d_backward_filter(x, dy, *f, pad=pad, variant=v)
            out.append(v)
        except cp4.Cp4Error as e:
            assert e.status == cp4.capi.ERR_UNSUPPORTED
    return out


# ---------------------------------------------------------------- golden ----
@pytest.mark.parametrize("name", GOLD_CASES)
def test_golden_all_passes(cp4, name):
    g = gold(name)
    f = {k: dev(g[k]) for k in FACTORS}
    x, dy = dev(g["x"]), dev(g["dy"])
    for v in variants_for(cp4, x.shape, f, g["pad"]):
        y = host(cp4.conv2d_forward(x, *f.values(), pad=g["pad"], variant=v))
        assert_activation_close(y, g["y"], f"{name} forward variant {v}")
    dx = host(cp4.conv2d_backward_data(dy, *f.values(), pad=g["pad"]))
    assert_activation_close(dx, g["dx"], f"{name} backward-data")
    for variant in filter_variants(cp4, x, dy, list(f.values()), g["pad"]):
        grads = cp4.conv2d_backward_filter(x, dy, *f.values(), pad=g["pad"], variant=variant)
        for got, k in zip(grads, FACTORS):
            assert_gradient_close(host(got), g["d" + k], f"{name} d{k} variant {variant}")


# ------------------------------------------------- the five workloads -------
@pytest.fixture(scope="module", params=list(WORKLOADS))
def workload(request):
    w = WORKLOADS[request.param]
    return w, make_inputs(w, seed=0)


def test_workload_forward(cp4, oracle, workload):
    w, a = workload
    want = oracle.forward(a["x"], a["FK"], a["FC"], a["FH"], a["FW"], w.pad)
    f = {k: dev(a[k]) for k in FACTORS}
    x = dev(a["x"])
    vs = variants_for(cp4, x.shape, f, w.pad)
    assert vs
    for v in vs + [-1]:
        y = host(cp4.conv2d_forward(x, *f.values(), pad=w.pad, variant=v))
        assert_activation_close(y, want, f"{w.name} forward variant {v}")


def test_workload_backward_data(cp4, oracle, workload):
    w, a = workload
    want = oracle.backward_data(a["dy"], a["FK"], a["FC"], a["FH"], a["FW"], w.pad)
    f = [dev(a[k]) for k in FACTORS]
    dx = host(cp4.conv2d_backward_data(dev(a["dy"]), *f, pad=w.pad))
    assert_activation_close(dx, want, f"{w.name} backward-data")


def test_workload_backward_filter(cp4, oracle, workload):
    w, a = workload
    want = oracle.backward_filter(a["x"], a["dy"], a["FK"], a["FC"], a["FH"], a["FW"], w.pad)
    f = [dev(a[k]) for k in FACTORS]
    for variant in filter_variants(cp4, dev(a["x"]), dev(a["dy"]), f, w.pad):
        got = cp4.conv2d_backward_filter(dev(a["x"]), dev(a["dy"]), *f, pad=w.pad,
                                         variant=variant)
        for g, wnt, k in zip(got, want, FACTORS):
            assert_gradient_close(host(g), wnt, f"{w.name} d{k} variant {variant}")
        # bit-reproducible: no floating-point atomics anywhere in a variant's reductions
        again = cp4.conv2d_backward_filter(dev(a["x"]), dev(a["dy"]), *f, pad=w.pad,
                                           variant=variant)
        for g1, g2 in zip(got, again):
            assert torch.equal(g1, g2), f"{w.name} variant {variant} differs between two runs"


def test_workload_properties(cp4, workload):
    """Size-independent properties at full size: linearity in x and the
    adjoint identity <forward(x), dy> == <x, backward_data(dy)> (2*pad == Y-1
    for all five workloads)."""
    w, a = workload
    f = [dev(a[k]) for k in FACTORS]
    x, dy = dev(a["x"]), dev(a["dy"])
    z = torch.roll(x, shifts=(1, 3), dims=(2, 3)) * 0.5
    y = cp4.conv2d_forward(x, *f, pad=w.pad)
    yz = cp4.conv2d_forward(z, *f, pad=w.pad)
    ylin = cp4.conv2d_forward(2.0 * x - 3.0 * z, *f, pad=w.pad)
    assert_activation_close(host(ylin), host(2.0 * y - 3.0 * yz), f"{w.name} linearity")
    dx = cp4.conv2d_backward_data(dy, *f, pad=w.pad)
    lhs = float((y.double() * dy.double()).sum())
    rhs = float((x.double() * dx.double()).sum())
    norm = float(y.double().norm() * dy.double().norm())
    assert abs(lhs - rhs) <= 1e-5 * norm, (lhs, rhs, norm)
    assert norm > 0 and float(y.abs().max()) > 0


# ------------------------------------------------------------ edge cases ----
EDGE = [
    # N, C, H, W, pad, T, Y, X, R
    (1, 48, 55, 55, 5, 256, 11, 11, 16),  # the reference's single-kernel test case
    (2, 3, 37, 41, 1, 5, 3, 3, 6),        # ragged tile edges, rank not a power of two
    (1, 1, 1, 1, 0, 1, 1, 1, 1),          # everything equal to one
    (3, 7, 5, 67, 2, 9, 5, 5, 1),         # rank 1, wide and short
    (1, 4, 9, 9, 0, 4, 3, 3, 4),          # no padding: output still H x W
    (1, 4, 9, 9, 3, 4, 3, 3, 4),          # pad larger than the filter radius
    (2, 5, 8, 8, 1, 3, 2, 2, 3),          # even filter
    (1, 6, 10, 12, 1, 4, 3, 5, 5),        # rectangular filter (the reference only warns)
    (1, 2, 20, 20, 8, 2, 17, 17, 2),      # largest filter of the reference's sweeps
    (4, 40, 16, 16, 1, 72, 3, 3, 48),     # rank above the register block
    (2, 16, 12, 12, 1, 32, 3, 3, 16),     # MFMA-eligible rank, small image
    # shapes the producer/consumer strip kernels accept (channels a multiple of
    # 64, even width), sized so that an image needs several strips
    (2, 64, 40, 50, 1, 40, 3, 3, 7),      # ragged last strip, partial output-channel block
    (1, 128, 33, 38, 2, 128, 5, 5, 32),   # 5x5, both passes eligible, odd strip count
    (1, 192, 30, 26, 3, 64, 7, 7, 16),    # 7x7, three chunks per channel quarter
    (2, 256, 57, 18, 0, 32, 3, 3, 20),    # no padding, tall image
    (3, 64, 9, 120, 1, 64, 1, 1, 9),      # 1x1 filter, wide rows
    # odd widths on the matrix-core path (the reference's AlexNet layers 3-5,
    # Cuda_kernels/bench/tensors_alexnet.txt): per-pixel stores, 12 output blocks
    (1, 192, 13, 13, 1, 384, 3, 3, 16),
    (1, 256, 27, 27, 1, 384, 3, 3, 8),
    (2, 64, 9, 11, 2, 40, 5, 5, 5),
    # channel counts that are multiples of 8 but not of 64 (padded channel quarters)
    (1, 48, 55, 55, 2, 256, 5, 5, 16),    # AlexNet layer 2
    (2, 24, 10, 12, 1, 16, 3, 3, 4),
    (1, 200, 9, 9, 1, 32, 3, 3, 7),
    # more than 256 input channels: factor fragments in LDS; odd width, odd chunk count
    (2, 512, 7, 7, 1, 64, 3, 3, 32),
    (1, 320, 14, 14, 1, 96, 3, 3, 16),
    (1, 384, 13, 13, 2, 384, 5, 5, 16),   # both passes above 256 channels
    # odd planes (7x7, 13x13, 27x27) on the matrix-core backward-filter path
    (4, 32, 7, 7, 1, 48, 3, 3, 8),
    (3, 64, 13, 13, 1, 32, 3, 3, 16),
    (2, 16, 27, 27, 2, 16, 5, 5, 4),
    # at most 16 ranks and 4 output-channel blocks: consumer waves in split roles
    (2, 64, 20, 22, 1, 80, 3, 3, 12),     # three channel blocks, the last partly filled
    (1, 32, 40, 40, 0, 128, 1, 1, 16),    # 1x1, four blocks
    (3, 16, 30, 34, 2, 96, 5, 5, 9),      # 5x5, several groups per strip
    (2, 64, 6, 288, 1, 128, 3, 3, 16),    # long rows: five groups per strip, fragment tiles reused
    (1, 32, 3, 576, 0, 64, 1, 1, 8),      # ten groups per strip
    # more than 16 ranks or more than 4 channel blocks, 1x1 / 3x3: wide role split (a
    # tap wave takes two rank quads, a contraction wave two channel blocks)
    (2, 64, 6, 288, 1, 160, 3, 3, 20),    # five blocks (one wave with two), ranks end inside quad 5
    (1, 128, 4, 320, 1, 256, 3, 3, 32),   # eight blocks, 32 ranks, five groups per strip
    (2, 32, 5, 200, 0, 200, 1, 1, 12),    # 1x1, seven blocks (the last partly filled), one rank chunk
    (1, 64, 13, 13, 1, 224, 3, 3, 24),    # odd plane: per-pixel stores, one group per strip
    (1, 320, 3, 210, 1, 72, 3, 3, 28),    # factor fragments in LDS, three blocks, four groups
    (2, 64, 10, 90, 2, 200, 5, 5, 12),    # 5x5 with up to 16 ranks: one quad per tap wave, seven blocks
    # wide planes: tiles of TH rows x Wt columns (producer/consumer kernel, tiled build)
    (1, 16, 9, 200, 1, 32, 3, 3, 8),      # four column tiles, the last one 8 columns wide
    (2, 24, 5, 131, 2, 16, 5, 5, 12),     # odd width across three tiles, 5x5
    (1, 64, 20, 300, 0, 64, 3, 3, 32),    # no padding, 32 ranks, ragged last row strip
    (1, 8, 3, 1000, 3, 8, 7, 7, 4),       # 7x7, very wide and short
    (2, 3, 40, 224, 1, 64, 3, 3, 16),     # three input channels, first-layer shape
    # many small planes (wave-per-plane tap kernel, one partial per image)
    (64, 32, 8, 8, 1, 48, 3, 3, 20),
    (70, 16, 6, 10, 2, 16, 5, 5, 40),     # two rank tiles, the second partly filled
    (64, 16, 14, 14, 0, 32, 1, 1, 8),     # 1x1 filter, no padding
    # few strips, many output channels: slices of output channels per strip
    (1, 96, 12, 12, 1, 200, 3, 3, 16),    # seven blocks in four slices, the last one of one ragged block
    (2, 320, 9, 10, 0, 130, 1, 1, 24),    # 1x1, factor fragments in LDS, five blocks in two slices
]


@pytest.mark.parametrize("dims", EDGE, ids=lambda d: "x".join(map(str, d)))
def test_edge_shapes(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, X, R = dims
    rng = np.random.default_rng(sum(dims))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / np.sqrt(R) for d in (T, C, Y, X)]
    f = [dev(v) for v in fac]
    fdict = dict(zip(FACTORS, f))
    want = oracle.forward(x, *fac, pad)
    for v in variants_for(cp4, x.shape, fdict, pad):
        y = host(cp4.conv2d_forward(dev(x), *f, pad=pad, variant=v))
        assert_activation_close(y, want, f"forward variant {v}")
    dx = host(cp4.conv2d_backward_data(dev(dy), *f, pad=pad))
    assert_activation_close(dx, oracle.backward_data(dy, *fac, pad), "backward-data")
    want_grads = oracle.backward_filter(x, dy, *fac, pad)
    for variant in filter_variants(cp4, dev(x), dev(dy), f, pad):
        got = cp4.conv2d_backward_filter(dev(x), dev(dy), *f, pad=pad, variant=variant)
        for g, wnt, k in zip(got, want_grads, FACTORS):
            assert_gradient_close(host(g), wnt, f"d{k} variant {variant}")


# (N, C, H, W, pad, T, Y, X, R): even and rectangular filters of up to 7 taps a side - the
# strided build of the producer / consumer kernel takes them as the next odd square window
WINDOWED = [
    (2, 32, 20, 24, 0, 48, 2, 2, 16),     # 2x2 in a 3x3 window, no zeros before the image
    (2, 32, 20, 24, 1, 48, 2, 2, 16),
    (1, 64, 17, 17, 1, 64, 4, 4, 32),     # 4x4 in 5x5, odd plane
    (2, 48, 14, 30, 3, 32, 1, 7, 16),     # 1x7: a one-row plane per output row
    (2, 48, 30, 14, 0, 32, 7, 1, 16),     # 7x1
    (1, 32, 28, 28, 1, 64, 3, 5, 24),     # 3x5
    (1, 32, 28, 28, 2, 64, 6, 6, 8),      # 6x6 in 7x7
    (2, 40, 13, 13, 1, 24, 3, 1, 48),     # two rank tiles: in passes
    (1, 900, 10, 10, 1, 32, 1, 3, 16),    # two channel slices
    (1, 16, 33, 35, 2, 16, 5, 2, 4),      # whole-group consumers
    (2, 32, 150, 12, 1, 32, 2, 4, 12),    # many strips, both sweep directions
]


@pytest.mark.parametrize("dims", WINDOWED, ids=lambda d: "x".join(map(str, d)))
def test_even_and_rectangular_filters(cp4, oracle, dims):
    N, C, H, W, pad, T, Y, X, R = dims
    rng = np.random.default_rng(sum(dims))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / np.sqrt(R) for d in (T, C, Y, X)]
    f = [dev(v) for v in fac]
    s = cp4.capi.shape_for(x.shape, *f, pad)
    assert cp4.default_variant(s) == "mfma_bf16x3_pipe_window"
    assert cp4.default_variant(s, backward_data=True) == "mfma_bf16x3_pipe_window"
    y = host(cp4.conv2d_forward(dev(x), *f, pad=pad))
    assert_activation_close(y, oracle.forward(x, *fac, pad), "forward")
    dx = host(cp4.conv2d_backward_data(dev(dy), *f, pad=pad))
    assert_activation_close(dx, oracle.backward_data(dy, *fac, pad), "backward-data")
    bias = rng.standard_normal(T).astype(np.float32)
    yb = host(cp4.conv2d_forward_bias_act(dev(x), *f, dev(bias), "relu", pad=pad))
    assert_activation_close(yb, np.maximum(y + bias[None, :, None, None], 0), "bias + relu")
    cp4.device_status()


# (N, C, H, W, pad, T, Y, R): channel counts the matrix-core backward-filter kernels do not
# take as they are
PADDED = [
    (2, 3, 12, 16, 1, 5, 3, 4),      # odd C and T on an even plane: one zero channel appended to each
    (3, 5, 9, 7, 1, 7, 3, 6),        # odd plane: padded to 16 channels
    (2, 3, 10, 10, 1, 1, 3, 70),     # three channels to one, more than 64 ranks: padding, then rank tiles
    (1, 3, 24, 40, 2, 16, 5, 16),    # only x is copied (T is even)
    (4, 16, 15, 15, 1, 20, 3, 8),    # odd plane, only dy is copied
]


@pytest.mark.parametrize("dims", PADDED, ids=lambda d: "x".join(map(str, d)))
def test_backward_filter_with_padded_channels(cp4, oracle, dims):
    """The library's choice runs these layers on the matrix cores, on copies of x / dy with
    zero channels appended (the general kernel takes 50 to 1000 times the forward pass on a
    first layer); a workspace off the 256-byte boundary falls back to the general kernel.
    Both against the oracle."""
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / np.sqrt(R) for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    want = oracle.backward_filter(x, dy, *fac, pad)
    s = cp4.capi.shape_for(x.shape, *f, pad)
    cp4.tune_clear()
    assert cp4.plan_query(s, "backward_filter")["variant"] != cp4.backward_filter_variants()[0]
    nbytes = cp4.backward_filter_workspace_bytes(s)
    buf = torch.empty(nbytes + 512, dtype=torch.uint8, device="cuda")
    off = (-buf.data_ptr()) % 256
    for shift, label in ((0, "padded route"), (16, "workspace off the boundary")):
        ws = buf[off + shift:off + shift + nbytes].view(torch.float32)
        got = cp4.conv2d_backward_filter(dev(x), dev(dy), *f, pad=pad, workspace=ws)
        for g, wnt, k in zip(got, want, FACTORS):
            assert_gradient_close(host(g), wnt, f"d{k} {label}")
    again = cp4.conv2d_backward_filter(dev(x), dev(dy), *f, pad=pad)
    for g1, g2 in zip(got, again):
        assert g1.shape == g2.shape
    cp4.device_status()


def test_split_role_schedule_at_scale(cp4, oracle):
    """Twice as many workgroups as compute units, five 64-pixel groups per strip,
    at most 16 ranks and 4 channel blocks: tap waves and contraction waves of a
    workgroup run several groups apart and the fragment tiles are reused."""
    N, C, H, W, pad, T, Y, R = 64, 64, 8, 288, 1, 128, 3, 16
    rng = np.random.default_rng(99)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    want = oracle.forward(x, *fac, pad)
    xd = dev(x)
    for _ in range(3):      # a race would not show on every launch
        assert_activation_close(host(cp4.conv2d_forward(xd, *f, pad=pad)), want, "forward")


def test_wide_role_split_at_scale(cp4, oracle):
    """More workgroups than compute units, seven groups per strip, 32 ranks and 8
    channel blocks (the ResNet-stage shape at a small batch), forward and
    backward-data: the tap waves run up to three groups ahead of the contraction
    waves and the fragment tiles are reused."""
    N, C, H, W, pad, T, Y, R = 5, 256, 56, 56, 1, 256, 3, 32
    rng = np.random.default_rng(7)
    x = np.maximum(rng.standard_normal((N, C, H, W)), 0).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    want = oracle.forward(x, *fac, pad)
    want_dx = oracle.backward_data(dy, *fac, pad)
    xd, dyd = dev(x), dev(dy)
    for _ in range(3):      # a race would not show on every launch
        assert_activation_close(host(cp4.conv2d_forward(xd, *f, pad=pad)), want, "forward")
        assert_activation_close(host(cp4.conv2d_backward_data(dyd, *f, pad=pad)), want_dx,
                                "backward-data")


def test_whole_row_strips_on_a_wide_plane(cp4, oracle):
    """Rows of 224 pixels, 16 ranks, 128 channels: the library's choice is the
    whole-row strip variant (4-row strips, one round of workgroups; the LDS plane
    has the room because up to 16 ranks it holds half the rank rows); with 32
    ranks the same layer runs on tiles.  Forward, backward-data and the fused epilogue."""
    N, C, H, W, pad, T, Y = 32, 128, 28, 224, 1, 128, 3     # (enough rows for several per strip)
    rng = np.random.default_rng(224)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    for R, variant in ((16, "mfma_bf16x3_pipe"), (32, "mfma_bf16x3_pipe_tiled")):
        fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
        f = [dev(v) for v in fac]
        s = cp4.capi.shape_for(x.shape, *f, pad)
        assert cp4.default_variant(s) == variant
        assert cp4.default_variant(s, backward_data=True) == variant
        want = oracle.forward(x, *fac, pad)
        want_dx = oracle.backward_data(dy, *fac, pad)
        bias = rng.standard_normal(T).astype(np.float32)
        for _ in range(2):
            assert_activation_close(host(cp4.conv2d_forward(dev(x), *f, pad=pad)), want, "forward")
            assert_activation_close(host(cp4.conv2d_backward_data(dev(dy), *f, pad=pad)), want_dx,
                                    "backward-data")
        yb = host(cp4.conv2d_forward_bias_act(dev(x), *f, bias=dev(bias), activation="relu", pad=pad))
        assert_activation_close(yb, np.maximum(want + bias[None, :, None, None], 0), "bias + relu")


@pytest.mark.parametrize("dims", [(2, 64, 28, 28, 64, 3, 16), (2, 256, 28, 28, 256, 3, 32),
                                  (2, 128, 14, 14, 128, 5, 16), (3, 5, 9, 9, 7, 3, 3),
                                  (2, 48, 13, 13, 48, 3, 40)],
                         ids=lambda d: "x".join(map(str, d)))
def test_pointers_aligned_to_four_bytes_only(cp4, dims):
    """The C ABI takes any float pointer: operands that start 4 bytes into an allocation
    (no 8- or 16-byte alignment) give the results of the aligned call - bit-identical for
    forward and backward-data, within fp32 summation order for the factor gradients."""
    N, C, H, W, T, Y, R = dims
    pad = Y // 2
    gen = torch.Generator(device="cuda").manual_seed(sum(dims))
    mk = lambda *s: torch.randn(*s, device="cuda", generator=gen)

    def shifted(t):
        buf = torch.empty(t.numel() + 1, device="cuda")
        view = buf[1:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 8 == 4
        return view

    x, dy = mk(N, C, H, W), mk(N, T, H, W)
    fac = [mk(d, R) for d in (T, C, Y, Y)]
    y = cp4.conv2d_forward(x, *fac, pad=pad)
    dx = cp4.conv2d_backward_data(dy, *fac, pad=pad)
    grads = cp4.conv2d_backward_filter(x, dy, *fac, pad=pad)
    xs, dys, facs = shifted(x), shifted(dy), [shifted(f) for f in fac]
    ys = cp4.conv2d_forward(xs, *facs, pad=pad, out=shifted(torch.zeros_like(y)))
    dxs = cp4.conv2d_backward_data(dys, *facs, pad=pad, out=shifted(torch.zeros_like(dx)))
    gs = cp4.conv2d_backward_filter(xs, dys, *facs, pad=pad)
    torch.cuda.synchronize()
    assert torch.equal(ys, y) or (ys - y).abs().max() <= 1e-6 * y.abs().max()
    assert torch.equal(dxs, dx) or (dxs - dx).abs().max() <= 1e-6 * dx.abs().max()
    for a, b in zip(gs, grads):
        assert (a - b).abs().max() <= 2e-6 * b.abs().max()


def test_reference_single_case_against_dense_conv(cp4):
    """Cuda_kernels/test/test_cp4Conv.cpp.cu:14-44: CP4 forward vs a dense conv
    of the recomposed kernel, all-positive U(0,1] inputs, compared with the
    reference's own relative-error counter at 1e-5 ... here 2e-5 because the
    dense comparator is torch's conv2d in fp32 rather than cuDNN."""
    n, c, hw, pad, t, f, r = 1, 48, 55, 5, 256, 11, 16
    x = cp4.random_uniform((n, c, hw, hw), 1234)
    FK, FC, FH, FW = (cp4.random_uniform((d, r), 1234 + i)
                      for i, d in enumerate((t, c, f, f)))
    K = cp4.recompose(FK, FC, FH, FW)
    y = cp4.conv2d_forward(x, FK, FC, FH, FW, pad=pad)
    ref = torch.nn.functional.conv2d(x.double(), K.double(), padding=pad).float()
    assert tuple(y.shape) == (n, t, hw, hw)
    assert cp4.count_exceeding(y, ref, 2e-5) == 0


def test_empty_batch(cp4):
    f = [torch.ones((d, 2), device="cuda") for d in (3, 4, 3, 3)]
    x = torch.empty((0, 4, 5, 5), device="cuda")
    assert cp4.conv2d_forward(x, *f, pad=1).shape == (0, 3, 5, 5)
    dy = torch.empty((0, 3, 5, 5), device="cuda")
    assert cp4.conv2d_backward_data(dy, *f, pad=1).shape == (0, 4, 5, 5)
    for g in cp4.conv2d_backward_filter(x, dy, *f, pad=1):
        assert float(host(g).max()) == 0.0 and float(host(g).min()) == 0.0


def test_dense_filter_gradient(cp4, oracle):
    g = gold("five5x5")
    x, dy = dev(g["x"]), dev(g["dy"])
    want = oracle.backward_filter_full(g["x"], g["dy"], 5, 5, g["pad"])
    dK = cp4.conv2d_backward_filter_full(x, dy, 5, 5, pad=g["pad"])
    assert_gradient_close(host(dK), want, "dK")
    # accumulate flag: the reference adds into the caller's buffer
    acc = cp4.conv2d_backward_filter_full(x, dy, 5, 5, pad=g["pad"], out=dK.clone())
    assert_gradient_close(host(acc), 2 * want, "dK accumulate")


# -------------------------------------------------------------- utilities ---
def test_recompose_and_allclose_like_reference(cp4, oracle):
    """Cuda_kernels/test/test_Utils.cpp.cu:10-51."""
    K0, K1 = cp4.random_uniform((16, 6), 1), cp4.random_uniform((16, 6), 2)
    K2, K3 = cp4.random_uniform((3, 6), 3), cp4.random_uniform((3, 6), 4)
    U = cp4.random_uniform((1, 16, 32, 32), 5)
    assert float(U.min()) > 0 and float(U.max()) <= 1.0
    assert torch.equal(U, cp4.random_uniform((1, 16, 32, 32), 5))
    assert not torch.equal(U, cp4.random_uniform((1, 16, 32, 32), 6))
    K = cp4.recompose(K0, K1, K2, K3)
    assert tuple(K.shape) == (16, 16, 3, 3) and K.numel() == 2304
    want = oracle.recompose(*(host(k) for k in (K0, K1, K2, K3)))
    np.testing.assert_allclose(host(K), want, rtol=1e-5)
    V = cp4.conv2d_forward(U, K0, K1, K2, K3, pad=1)
    V2 = cp4.conv2d_forward(U, K0, K1, K2, K3, pad=1)
    assert tuple(V.shape) == (1, 16, 32, 32) and bool((V != 0).all())
    assert cp4.count_exceeding(V, V2, 1e-5) == 0
    V[0, 0, 0, 0] *= 2
    assert cp4.count_exceeding(V, V2, 1e-1) == 1
    a = torch.tensor([0.0, 0.0, 1.0, float("nan")], device="cuda")
    b = torch.tensor([0.05, 0.0, 1.0, 1.0], device="cuda")
    assert cp4.count_exceeding(a, b, 1e-1) == 1      # NaN counts, 0.05 abs passes
    assert cp4.count_exceeding(a, b, 1e-2) == 2
    assert cp4.count_exceeding(a, b, 1e-2) == oracle.count_exceeding(
        host(a)[:3], host(b)[:3], 1e-2) + 1


def test_timed_launch_and_tuner(cp4):
    w = WORKLOADS["C2"]
    a = make_inputs(w)
    f = [dev(a[k]) for k in FACTORS]
    x = dev(a["x"])
    y = torch.empty((w.N, w.T, w.H, w.W), device="cuda")
    us = cp4.time_forward(x, *f, y, w.pad, warmup=1, profcount=5)
    assert 0 < us < 1e6
    best, best_us = cp4.tune_forward(x, *f, y, w.pad, warmup=1, profcount=5)
    names = dict((v, n) for v, n, _ in cp4.forward_variants())
    assert best in names and best_us > 0
    y2 = cp4.conv2d_forward(x, *f, pad=w.pad)          # uses the tuned choice
    y3 = cp4.conv2d_forward(x, *f, pad=w.pad, variant=best)
    assert torch.equal(y2, y3)
    cp4.lib().cp4_tune_clear()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        y4 = cp4.conv2d_forward(x, *f, pad=w.pad, variant=best)   # explicit non-default stream
    s.synchronize()
    assert torch.equal(y3, y4)


def test_tuner_table_round_trip(cp4, tmp_path):
    """The tuner's table written to a file and entered again (a later process): the
    same choices come back, variants by name."""
    w = WORKLOADS["C1"]
    a = make_inputs(w)
    f = [dev(a[k]) for k in FACTORS]
    x = dev(a["x"])
    s = cp4.capi.shape_for(x.shape, *f, w.pad)
    names = [n for _, n, _ in cp4.forward_variants()]
    try:
        cp4.tune_clear()
        cp4.set_tuned_choice(s, names.index("mfma_bf16x3_pipe"), 2, 0, 0)
        cp4.set_tuned_choice(s, names.index("general_valu"), 0, 0, 1, backward_data=True)
        # the backward-filter tuner's own table travels in the same file
        best, _ = cp4.tune_backward_filter(x, dev(a["dy"]), *f, w.pad, warmup=1, profcount=3)
        fnames = cp4.backward_filter_variants()
        assert fnames == ["general_valu", "mfma_four_launches", "mfma_fused_taps",
                          "dense_gradient_tiles"]
        ftable = cp4.tuned_filter_table()
        assert len(ftable) == 1 and ftable[0]["variant"] == fnames[best]
        table = cp4.tuned_table()
        assert len(table) == 2 and {e["variant"] for e in table} == {"mfma_bf16x3_pipe", "general_valu"}
        path = str(tmp_path / "tuned.json")
        cp4.save_tuned(path)
        cp4.tune_clear()
        assert cp4.tuned_table() == [] and cp4.tuned_filter_table() == []
        assert cp4.load_tuned(path) == 3
        assert cp4.tuned_table() == table
        assert cp4.tuned_filter_table() == ftable
        assert cp4.tuned_choice(s) == {"variant": names.index("mfma_bf16x3_pipe"), "tile_rows": 2,
                                       "tile_cols": 0, "role_split": 0}
        assert cp4.tuned_choice(s, backward_data=True)["variant"] == names.index("general_valu")
    finally:
        cp4.tune_clear()


# N, C, H, W, T, Y, R: few ranks and channels, planes of many blocks (whole-block
# producers; consumer waves that take whole pixel groups each)
FEW_CHANNEL_CASES = [
    (2, 64, 96, 96, 64, 3, 16),
    (2, 32, 112, 112, 32, 3, 4),        # whole groups by the kernel's own rule
    (1, 48, 224, 224, 40, 3, 9),        # ragged channels, three rank quads, wide plane (tiles)
    (2, 20, 64, 80, 64, 5, 16),
    (3, 16, 72, 72, 24, 3, 1),
    (1, 64, 130, 70, 33, 1, 12),
]


@pytest.mark.parametrize("dims", FEW_CHANNEL_CASES, ids=lambda d: "x".join(map(str, d)))
def test_consumer_schedules_at_few_channels(cp4, oracle, dims):
    """Every consumer schedule (the kernel's rule, no role split, whole groups per
    wave) of every producer / consumer variant that takes the shape, entered through
    the tuner's table, against the oracle; forward and backward-data."""
    N, C, H, W, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    a = {"x": rng.standard_normal((N, C, H, W), dtype=np.float32),
         "dy": rng.standard_normal((N, T, H, W), dtype=np.float32)}
    for k, d in (("FK", T), ("FC", C), ("FH", Y), ("FW", Y)):
        a[k] = rng.standard_normal((d, R), dtype=np.float32) * np.float32((R * C * Y * Y) ** -0.25)
    fa = [a[k] for k in FACTORS]
    f = [dev(a[k]) for k in FACTORS]
    x, dy = dev(a["x"]), dev(a["dy"])
    pad = (Y - 1) // 2
    want_y = oracle.forward(a["x"], *fa, pad)
    want_dx = oracle.backward_data(a["dy"], *fa, pad)
    s = cp4.capi.shape_for(x.shape, *f, pad)
    ran = 0
    try:
        for v, name, ok in cp4.forward_variants(s):
            if not ok or "pipe" not in name:
                continue
            for schedule in (1, 0, 2):
                for th in (0, 3):
                    cols = 64 if (th and "tiled" in name) else 0
                    for bwd in (False, True):
                        try:
                            cp4.set_tuned_choice(s, v, th, cols, schedule, backward_data=bwd)
                        except cp4.Cp4Error as e:      # this tile does not fit this variant
                            assert e.status == cp4.capi.ERR_UNSUPPORTED
                            continue
                        got = (cp4.conv2d_backward_data(dy, *f, pad=pad) if bwd
                               else cp4.conv2d_forward(x, *f, pad=pad))
                        assert_activation_close(host(got), want_dx if bwd else want_y,
                                             f"{name} schedule {schedule} th {th} bwd {bwd}")
                        ran += 1
    finally:
        cp4.tune_clear()
    cp4.device_status()
    assert ran >= 6


# ------------------------------------------------ ranks beyond a kernel's tile ----
@pytest.mark.parametrize("R", [33, 48, 64, 65, 96, 128, 200])
def test_ranks_beyond_one_tile(cp4, oracle, R):
    """Ranks above 32 (forward / backward-data: passes of 32 ranks on the producer /
    consumer kernel) and above 64 (backward-filter: the matrix-core pass per tile of 64
    ranks): all three passes, every variant that takes the shape, against the oracle."""
    rng = np.random.default_rng(R)
    N, C, H, W, T, Y = 2, 64, 28, 28, 96, 3
    a = {"x": rng.standard_normal((N, C, H, W), dtype=np.float32),
         "dy": rng.standard_normal((N, T, H, W), dtype=np.float32)}
    for k, d in (("FK", T), ("FC", C), ("FH", Y), ("FW", Y)):
        a[k] = rng.standard_normal((d, R), dtype=np.float32) * np.float32((R * C) ** -0.25)
    f = {k: dev(a[k]) for k in FACTORS}
    fa = [a[k] for k in FACTORS]
    x, dy = dev(a["x"]), dev(a["dy"])
    want = oracle.forward(a["x"], *fa, 1)
    names = dict((v, n) for v, n, _ in cp4.forward_variants())
    vs = variants_for(cp4, x.shape, f, 1)
    assert any(names[v] == "mfma_bf16x3_pipe_rank_passes" for v in vs)
    for v in vs:
        assert_activation_close(host(cp4.conv2d_forward(x, *f.values(), pad=1, variant=v)), want,
                                f"R={R} forward {names[v]}")
    assert_activation_close(host(cp4.conv2d_backward_data(dy, *f.values(), pad=1)),
                            oracle.backward_data(a["dy"], *fa, 1), f"R={R} backward-data")
    wants = oracle.backward_filter(a["x"], a["dy"], *fa, 1)
    fv = filter_variants(cp4, x, dy, list(f.values()), 1)
    assert 1 in fv, "the matrix-core backward-filter must take every rank here"
    for variant in fv:
        grads = cp4.conv2d_backward_filter(x, dy, *f.values(), pad=1, variant=variant)
        for g, wnt, k in zip(grads, wants, FACTORS):
            assert_gradient_close(host(g), wnt, f"R={R} d{k} variant {variant}")
    cp4.device_status()


# (N, C, H, W, pad, T, Y, R): more than 768 channels on the side a pass contracts first
WIDE_CHANNELS = [
    (2, 1024, 14, 14, 1, 96, 3, 16),     # forward: two slices of 512 input channels
    (1, 800, 9, 12, 0, 64, 1, 8),        # 1x1, slices of 400 channels; backward-data is a single pass
    (2, 64, 10, 10, 1, 1000, 3, 24),     # backward-data: 1000 output channels are its input side
    (1, 1600, 7, 8, 1, 32, 3, 40),       # three slices x two rank tiles
    (2, 1024, 7, 7, 1, 1360, 3, 24),     # odd plane: backward-filter contracts slice by slice
]


@pytest.mark.parametrize("dims", WIDE_CHANNELS, ids=lambda d: "x".join(map(str, d)))
def test_channels_beyond_one_slice(cp4, oracle, dims):
    """The producer / consumer kernel holds 768 input channels: wider layers run it once per
    channel slice (and rank tile) with y +=, forward and backward-data, instead of the
    general kernel.  Against the oracle; the library's choice must not be the general kernel."""
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) * np.float32((R * max(C, T)) ** -0.25)
           for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    s = cp4.capi.shape_for(x.shape, *f, pad)
    cp4.tune_clear()
    assert cp4.default_variant(s) != "general_valu"
    assert cp4.default_variant(s, backward_data=True) != "general_valu"
    want = oracle.forward(x, *fac, pad)
    assert_activation_close(host(cp4.conv2d_forward(dev(x), *f, pad=pad)), want, "forward")
    if C > 768:     # the variant by number as well (a small layer's default may be another)
        v = {n: i for i, n, _ in cp4.forward_variants()}["mfma_bf16x3_pipe_rank_passes"]
        assert_activation_close(host(cp4.conv2d_forward(dev(x), *f, pad=pad, variant=v)), want,
                                "forward, channel passes")
    assert_activation_close(host(cp4.conv2d_backward_data(dev(dy), *f, pad=pad)),
                            oracle.backward_data(dy, *fac, pad), "backward-data")
    # backward-filter: the contraction's factor tile in slices (even planes: inside the fp32
    # kernel; odd planes with channel counts that are multiples of 16: one launch per slice)
    assert cp4.plan_query(s, "backward_filter")["variant"] != cp4.backward_filter_variants()[0]
    grads = cp4.conv2d_backward_filter(dev(x), dev(dy), *f, pad=pad)
    for g, wnt, k in zip(grads, oracle.backward_filter(x, dy, *fac, pad), FACTORS):
        assert_gradient_close(host(g), wnt, f"d{k}")
    cp4.device_status()

