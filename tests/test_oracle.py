"""CPU tests that pin the oracle (no GPU, no HIP library).

The oracle's two restatements (literal loop nests / unfused factor-by-factor
sequence) are checked against: the committed golden vectors (torch float64
dense conv + autograd on the recomposed kernel), torch's CPU conv2d directly,
closed forms, the adjoint identity and linearity -- each chosen so that a
dropped term, wrong sign/index or transposed operand fails.
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "cp4_golden.npz"))
CASES = sorted({k.split(".")[0] for k in GOLD.files})


def gold(name):
    N, H, W, pad, T, C, Y, X, R = (int(v) for v in GOLD[name + ".shape"])
    g = {k: GOLD[f"{name}.{k}"] for k in
         ("x", "dy", "FK", "FC", "FH", "FW", "y", "dx", "dx_adjoint",
          "dFK", "dFC", "dFH", "dFW")}
    g["pad"] = pad
    return g


def close(a, b, rtol, atol=0.0):
    scale = np.abs(b).max()
    np.testing.assert_allclose(a, b, rtol=rtol, atol=atol + rtol * scale * 1e-2)
    assert np.abs(a - b).max() <= rtol * max(scale, 1e-30)


@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("direct", [True, False])
def test_forward_golden(oracle, name, direct):
    g = gold(name)
    if direct and name == "config1":
        pytest.skip("literal loops only on tiny cases")
    y = oracle.forward(g["x"], g["FK"], g["FC"], g["FH"], g["FW"], g["pad"], direct)
    close(y, g["y"], 2e-5)


@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("direct", [True, False])
def test_backward_data_golden(oracle, name, direct):
    g = gold(name)
    if direct and name == "config1":
        pytest.skip("literal loops only on tiny cases")
    dx = oracle.backward_data(g["dy"], g["FK"], g["FC"], g["FH"], g["FW"], g["pad"], direct)
    close(dx, g["dx"], 2e-5)
    Y = g["FH"].shape[0]
    if 2 * g["pad"] == Y - 1:
        # the reference's flipped-tap formula is the exact adjoint here
        close(dx, g["dx_adjoint"], 2e-5)


@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("direct", [True, False])
def test_backward_filter_golden(oracle, name, direct):
    g = gold(name)
    if direct and name in ("config1", "ragged"):
        pytest.skip("literal 8-deep loops only on tiny cases")
    grads = oracle.backward_filter(g["x"], g["dy"], g["FK"], g["FC"], g["FH"],
                                   g["FW"], g["pad"], direct)
    for got, k in zip(grads, ("dFK", "dFC", "dFH", "dFW")):
        close(got, g[k], 5e-5)


def test_filter_factor_direct_accumulates(oracle):
    """The reference's per-factor functions add into the caller's buffer
    (Cuda_kernels/cp4Conv2dBackwardFilter.cu:99,150,200,249)."""
    import ctypes
    g = gold("tiny3x3")
    s = oracle.shape_of(g["x"].shape, g["FK"], g["FC"], g["FH"], g["FW"], g["pad"])
    out = np.full_like(g["FK"], 3.0)
    oracle.lib().cp4o_backward_filter_factor_direct(
        ctypes.byref(s), 0, oracle._fp(out), oracle._fp(g["x"]), oracle._fp(g["dy"]),
        oracle._fp(g["FK"]), oracle._fp(g["FC"]), oracle._fp(g["FH"]), oracle._fp(g["FW"]))
    close(out - 3.0, g["dFK"], 1e-4, atol=1e-6)


def test_dense_filter_gradient_chain_rule(oracle):
    """dFK[t,r] = sum_{c,y,x} dK[t,c,y,x] FC[c,r] FH[y,r] FW[x,r] ties the dense
    gradient (cp4Conv2dBackwardFilter.cu:23-59) to the factor gradients, and
    torch autograd on a dense conv pins the dense gradient itself."""
    g = gold("five5x5")
    Y, X = g["FH"].shape[0], g["FW"].shape[0]
    dK = oracle.backward_filter_full(g["x"], g["dy"], Y, X, g["pad"])
    x = torch.from_numpy(g["x"]).double()
    K = torch.zeros(dK.shape, dtype=torch.float64, requires_grad=True)
    y = F.conv2d(x, K, padding=g["pad"])
    (y * torch.from_numpy(g["dy"]).double()).sum().backward()
    close(dK, K.grad.numpy(), 2e-5)
    dFK = np.einsum("tcyx,cr,yr,xr->tr", dK.astype(np.float64), g["FC"], g["FH"], g["FW"])
    close(dFK, g["dFK"], 5e-5)
    dFW = np.einsum("tcyx,tr,cr,yr->xr", dK.astype(np.float64), g["FK"], g["FC"], g["FH"])
    close(dFW, g["dFW"], 5e-5)


def test_recompose_matches_einsum(oracle):
    g = gold("ragged")
    K = oracle.recompose(g["FK"], g["FC"], g["FH"], g["FW"])
    ref = np.einsum("tr,cr,yr,xr->tcyx", *(g[k].astype(np.float64)
                                           for k in ("FK", "FC", "FH", "FW")))
    assert K.shape == ref.shape
    close(K, ref, 1e-5)


def test_recompose_shape_like_reference_test(oracle):
    """Cuda_kernels/test/test_Utils.cpp.cu:25-31: (16,6),(16,6),(3,6),(3,6) -> 16x16x3x3."""
    rng = np.random.default_rng(0)
    K = oracle.recompose(*(rng.random((d, 6), np.float32) for d in (16, 16, 3, 3)))
    assert K.shape == (16, 16, 3, 3) and K.size == 2304


def test_forward_vs_torch_conv_reference_single_case(oracle):
    """The shape of the reference's 'Single Convolution Kernel test'
    (Cuda_kernels/test/test_cp4Conv.cpp.cu:16-22) with its all-positive U(0,1]
    inputs, against torch's dense conv on the recomposed kernel."""
    rng = np.random.default_rng(1234)
    n, c, hw, pad, t, f, r = 1, 48, 55, 5, 256, 11, 16
    x = 1.0 - rng.random((n, c, hw, hw), np.float32)
    FK, FC, FH, FW = (1.0 - rng.random((d, r), np.float32) for d in (t, c, f, f))
    y = oracle.forward(x, FK, FC, FH, FW, pad)
    K = np.einsum("tr,cr,yr,xr->tcyx", *(a.astype(np.float64) for a in (FK, FC, FH, FW)))
    ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(K), padding=pad).numpy()
    assert y.shape == (n, t, hw, hw)
    assert oracle.count_exceeding(y, ref.astype(np.float32), 1e-4) == 0


def test_all_ones_closed_form(oracle):
    """All-ones factors and a constant image: an interior pixel equals
    R*C*Y*X*const, a corner pixel R*C*(Y-pad)*(X-pad)*const."""
    N, C, H, W, pad, T, Y, X, R = 1, 3, 8, 9, 1, 2, 3, 3, 4
    x = np.full((N, C, H, W), 0.5, np.float32)
    ones = [np.ones((d, R), np.float32) for d in (T, C, Y, X)]
    for direct in (True, False):
        y = oracle.forward(x, *ones, pad, direct)
        assert np.allclose(y[0, :, 1:-1, 1:-1], R * C * Y * X * 0.5)
        assert np.allclose(y[0, :, 0, 0], R * C * (Y - pad) * (X - pad) * 0.5)
        assert np.allclose(y[0, :, 0, 3], R * C * (Y - pad) * X * 0.5)


def test_asymmetric_taps_not_flipped(oracle):
    """Cross-correlation, not convolution: a single tap at (y=0, x=2) of a 3x3
    filter with pad 1 reads In[h-1, w+1]."""
    x = np.zeros((1, 1, 5, 5), np.float32)
    x[0, 0, 2, 3] = 1.0
    FK = FC = np.ones((1, 1), np.float32)
    FH = np.array([[1.0], [0.0], [0.0]], np.float32)
    FW = np.array([[0.0], [0.0], [1.0]], np.float32)
    for direct in (True, False):
        y = oracle.forward(x, FK, FC, FH, FW, 1, direct)
        exp = np.zeros_like(y)
        exp[0, 0, 3, 2] = 1.0       # h-1 == 2, w+1 == 3
        assert np.array_equal(y, exp)
        # backward-data sends the impulse the other way
        dx = oracle.backward_data(x, FK, FC, FH, FW, 1, direct)
        exp = np.zeros_like(dx)
        exp[0, 0, 1, 4] = 1.0
        assert np.array_equal(dx, exp)


@pytest.mark.parametrize("seed", range(4))
def test_unfused_equals_direct_random_shapes(oracle, seed):
    rng = np.random.default_rng(seed)
    N, C, T, R = (int(rng.integers(1, 5)) for _ in range(4))
    H, W = int(rng.integers(3, 9)), int(rng.integers(3, 9))
    Y = X = int(rng.choice([1, 3, 5]))
    pad = int(rng.integers(0, 3))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) for d in (T, C, Y, X)]
    close(oracle.forward(x, *fac, pad), oracle.forward(x, *fac, pad, True), 1e-5)
    close(oracle.backward_data(dy, *fac, pad), oracle.backward_data(dy, *fac, pad, True), 1e-5)
    for a, b in zip(oracle.backward_filter(x, dy, *fac, pad),
                    oracle.backward_filter(x, dy, *fac, pad, True)):
        close(a, b, 1e-4)


def test_adjoint_identity_same_padding(oracle):
    """<y, dy> == <x, dx> when 2*pad == Y-1 (backward-data is the adjoint)."""
    rng = np.random.default_rng(7)
    N, C, H, W, pad, T, Y, X, R = 2, 6, 10, 12, 2, 5, 5, 5, 3
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) for d in (T, C, Y, X)]
    y = oracle.forward(x, *fac, pad).astype(np.float64)
    dx = oracle.backward_data(dy, *fac, pad).astype(np.float64)
    lhs, rhs = (y * dy).sum(), (x * dx).sum()
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs))
    # and the factor gradients are directional derivatives of <y, dy>
    grads = oracle.backward_filter(x, dy, *fac, pad)
    for i, gname in enumerate(("FK", "FC", "FH", "FW")):
        d = rng.standard_normal(fac[i].shape).astype(np.float32)
        eps = 1e-2
        fp = [f.copy() for f in fac]; fm = [f.copy() for f in fac]
        fp[i] = fac[i] + eps * d; fm[i] = fac[i] - eps * d
        num = ((oracle.forward(x, *fp, pad).astype(np.float64) * dy).sum()
               - (oracle.forward(x, *fm, pad).astype(np.float64) * dy).sum()) / (2 * eps)
        ana = (grads[i].astype(np.float64) * d).sum()
        assert abs(num - ana) <= 2e-3 * max(abs(num), abs(ana)), gname


def test_rank_additivity(oracle):
    g = gold("ragged")
    R = g["FK"].shape[1]
    total = np.zeros_like(g["y"], dtype=np.float64)
    for r in range(R):
        total += oracle.forward(g["x"], *(g[k][:, r:r + 1] for k in ("FK", "FC", "FH", "FW")),
                                g["pad"])
    close(total, g["y"], 2e-5)


def test_count_exceeding_semantics(oracle):
    """Cuda_kernels/Utils.cu:151-155 and the reference's use in
    test/test_Utils.cpp.cu:45-51."""
    a = np.array([1.0, 2.0, 0.0, 0.0, -4.0], np.float32)
    assert oracle.count_exceeding(a, a, 1e-5) == 0
    b = a.copy(); b[0] *= 2                     # rel err max(1/1, 1/2) = 1
    assert oracle.count_exceeding(a, b, 1e-1) == 1
    b = a.copy(); b[2] = 0.05                   # a == 0 -> absolute error
    assert oracle.count_exceeding(a, b, 1e-1) == 0
    assert oracle.count_exceeding(a, b, 1e-2) == 1


# ---- 3-factor CP sibling op ------------------------------------------------------

@pytest.mark.parametrize("shape", [(1, 16, 32, 32, 3, 6, 16),     # test/test_conv2d_cp.py:12-15
                                   (2, 5, 9, 7, 5, 4, 3),
                                   (1, 3, 6, 6, 1, 2, 4)])
def test_cp3_forward_vs_torch_dense_conv(oracle, shape):
    """The reference's own check (test/test_conv2d_cp.py:20,27-31): the CP layer equals
    the dense convolution with kernel einsum over the three factors."""
    N, C, H, W, Y, R, T = shape
    rng = np.random.default_rng(7)
    x = rng.uniform(size=(N, C, H, W)).astype(np.float32)
    K0 = rng.uniform(size=(C, R)).astype(np.float32)
    K1 = rng.uniform(size=(Y, Y, R)).astype(np.float32)
    K2 = rng.uniform(size=(R, T)).astype(np.float32)
    dense = np.einsum("cr,ijr,rt->tcij", K0.astype(np.float64), K1.astype(np.float64),
                      K2.astype(np.float64))
    want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(dense), padding=Y // 2).numpy()
    close(oracle.cp3_forward(x, K0, K1, K2, Y // 2), want, 1e-5)


def test_cp3_depthwise_tap_orientation(oracle):
    """A single tap at (row 0, column 2) of a 3x3 depthwise filter reads the pixel one row
    up and one column right: fails on a transposed or flipped K1."""
    x = np.arange(25, dtype=np.float32).reshape(1, 1, 5, 5)
    K1 = np.zeros((3, 3, 1), np.float32)
    K1[0, 2, 0] = 1.0
    y = oracle.cp3_forward(x, np.ones((1, 1), np.float32), K1, np.ones((1, 1), np.float32), 1)
    want = np.zeros((5, 5), np.float32)
    want[1:, :4] = x[0, 0, :4, 1:]
    np.testing.assert_array_equal(y[0, 0], want)


# ---- layer geometry: stride, explicit padding, an output plane of its own ----
GEOM = np.load(os.path.join(os.path.dirname(__file__), "golden", "cp4_golden_geometry.npz"))
GEOM_CASES = sorted({k.split(".")[0] for k in GEOM.files})


def geom_gold(oracle, name):
    g = {k: GEOM[f"{name}.{k}"] for k in
         ("x", "dy", "FK", "FC", "FH", "FW", "y", "dx", "dFK", "dFC", "dFH", "dFW")}
    g["geometry"] = oracle.Geometry(*[int(v) for v in GEOM[name + ".geometry"]])
    return g


@pytest.mark.parametrize("name", GEOM_CASES)
def test_geometry_forward_golden(oracle, name):
    g = geom_gold(oracle, name)
    f = [g[k] for k in ("FK", "FC", "FH", "FW")]
    close(oracle.forward_geom(g["x"], *f, g["geometry"], direct=True), g["y"], 2e-5)
    close(oracle.forward_geom(g["x"], *f, g["geometry"], direct=False), g["y"], 2e-5)


@pytest.mark.parametrize("name", GEOM_CASES)
def test_geometry_backward_golden(oracle, name):
    g = geom_gold(oracle, name)
    f = [g[k] for k in ("FK", "FC", "FH", "FW")]
    dx = oracle.backward_data_geom(g["dy"], g["x"].shape[2:], *f, g["geometry"])
    close(dx, g["dx"], 2e-5)
    grads = oracle.backward_filter_geom(g["x"], g["dy"], *f, g["geometry"])
    for got, k in zip(grads, ("dFK", "dFC", "dFH", "dFW")):
        close(got, g[k], 1e-4)


def test_geometry_same_padding_formula(oracle):
    """The framework's SAME rule on an even size: 8 -> 4 at stride 2 with a 3x3
    filter pads 0 before and 1 after, so window o starts at input row 2o; the
    symmetric padding=1 of a same-named PyTorch layer starts it at 2o - 1."""
    g = oracle.geometry_same(8, 8, 3, 3, 2)
    assert (g.pad_top, g.pad_left, g.out_h, g.out_w) == (0, 0, 4, 4)
    g = oracle.geometry_same(9, 7, 3, 3, 2)
    assert (g.pad_top, g.pad_left, g.out_h, g.out_w) == (1, 1, 5, 4)
    g = oracle.geometry_same(13, 13, 7, 7, 3)
    assert (g.pad_top, g.out_h) == (3, 5)
    g = oracle.geometry_valid(11, 12, 5, 5, 2)
    assert (g.pad_top, g.out_h, g.out_w) == (0, 4, 4)
    # an impulse at input row 2, column 2 under SAME / stride 2 / 3x3 on 8x8: output
    # (1, 1) sees it through tap (0, 0), output (0, 0) through tap (2, 2)
    x = np.zeros((1, 1, 8, 8), np.float32)
    x[0, 0, 2, 2] = 1.0
    FK = np.ones((1, 1), np.float32)
    FC = np.ones((1, 1), np.float32)
    FH = np.array([[1.0], [10.0], [100.0]], np.float32)
    FW = np.array([[1.0], [2.0], [3.0]], np.float32)
    y = oracle.forward_geom(x, FK, FC, FH, FW, oracle.geometry_same(8, 8, 3, 3, 2), direct=True)
    assert y[0, 0, 1, 1] == 1.0 and y[0, 0, 0, 0] == 300.0 and y[0, 0, 1, 0] == 3.0 \
        and y[0, 0, 0, 1] == 100.0


def test_geometry_reduces_to_the_reference_case(oracle):
    """Stride 1, pad zeros before, an H x W output: the reference's own operator."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 6, 7)).astype(np.float32)
    dy = rng.standard_normal((2, 4, 6, 7)).astype(np.float32)
    f = [rng.standard_normal((d, 3)).astype(np.float32) for d in (4, 3, 3, 3)]
    g = oracle.Geometry(1, 1, 1, 1, 6, 7)
    close(oracle.forward_geom(x, *f, g, direct=True), oracle.forward(x, *f, 1, direct=True), 1e-6)
    close(oracle.backward_data_geom(dy, (6, 7), *f, g), oracle.backward_data(dy, *f, 1, direct=True), 1e-6)
    for a, b in zip(oracle.backward_filter_geom(x, dy, *f, g),
                    oracle.backward_filter(x, dy, *f, 1, direct=True)):
        close(a, b, 1e-6)


# ---- reshaped-CP sibling op ---------------------------------------------------
@pytest.mark.parametrize("dims", [(1, 4, 4, 4, 4, 8, 8, 3, 11), (2, 2, 3, 3, 2, 6, 7, 3, 4),
                                  (1, 3, 2, 2, 5, 5, 6, 5, 3)],
                         ids=lambda d: "x".join(map(str, d)))
def test_rcp_forward_matches_the_dense_einsum(oracle, dims):
    """The reference's own check of its reshaped-CP op (test/test_conv2d_rcp.py:38-45):
    a SAME convolution with einsum('axr,byr,hwr->hwabxy') reshaped to [h,w,in,out]."""
    N, S0, S1, T0, T1, H, W, Y, R = dims
    g = torch.Generator().manual_seed(sum(dims))
    x = torch.rand(N, S0 * S1, H, W, generator=g, dtype=torch.float64)
    K0 = torch.rand(S0, T0, R, generator=g, dtype=torch.float64)
    K1 = torch.rand(S1, T1, R, generator=g, dtype=torch.float64)
    KC = torch.randn(Y, Y, R, generator=g, dtype=torch.float64)
    K = torch.einsum("axr,byr,hwr->hwabxy", K0, K1, KC).reshape(Y, Y, S0 * S1, T0 * T1)
    want = F.conv2d(x, K.permute(3, 2, 0, 1), padding=Y // 2).numpy()
    got = oracle.rcp_forward(x.numpy(), K0.numpy(), K1.numpy(), KC.numpy(), Y // 2)
    close(got, want.astype(np.float32), 2e-5)
    # an impulse in channel (a, b) = (1, 0) reaches output channel (x, y) through
    # K0[1, x] K1[0, y] only: pins the row-major channel pairing
    if S0 > 1:
        xi = np.zeros((1, S0 * S1, H, W), np.float32)
        xi[0, 1 * S1 + 0, H // 2, W // 2] = 1.0
        yi = oracle.rcp_forward(xi, K0.numpy(), K1.numpy(), KC.numpy(), Y // 2)
        t = (T0 - 1) * T1 + (T1 - 1)
        centre = float((K0[1, T0 - 1] * K1[0, T1 - 1] * KC[Y // 2, Y // 2]).sum())
        assert abs(yi[0, t, H // 2, W // 2] - centre) <= 1e-5 * max(abs(centre), 1.0)
