"""Seeded random layers through the three passes, every forward variant that takes
the shape and both backward-filter variants, against the CPU oracle: filter sizes
1-7, the three paddings the reference's shapes use (same, none, full), channel
counts that are not multiples of the kernels' blocks, ranks on both sides of the
32- and 64-rank tiles, rows from 2 to 300 pixels."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

FACTORS = ("FK", "FC", "FH", "FW")


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def draw(seed):
    rng = np.random.default_rng(1000 + seed)
    Y = int(rng.choice([1, 3, 3, 3, 5, 7]))
    pad = int(rng.choice([Y // 2, Y // 2, Y // 2, 0, Y - 1]))
    C = int(rng.choice([3, 5, 8, 16, 24, 32, 33, 48, 64, 96, 128, 200, 256, 320]))
    T = int(rng.choice([1, 7, 8, 16, 32, 40, 64, 80, 128, 160, 256, 300]))
    R = int(rng.choice([1, 2, 4, 8, 12, 16, 17, 24, 32, 33, 48, 64, 70]))
    wide = rng.random() < 0.3
    H = int(rng.integers(1, 24 if wide else 40))
    W = int(rng.integers(100, 300)) if wide else int(rng.integers(2, 70))
    N = int(rng.integers(1, 5))
    if N * (C + T) * H * W > 4e6:
        N = 1
    if (C + T) * H * W > 4e6:
        H = max(1, H // 4)
    return rng, (N, C, H, W, pad, T, Y, R)


@pytest.mark.parametrize("seed", range(24))
def test_random_layer(cp4, oracle, seed):
    rng, (N, C, H, W, pad, T, Y, R) = draw(seed)
    what = f"N{N} C{C} {H}x{W} pad{pad} T{T} {Y}x{Y} R{R}"
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]

    def close(got, want, tol, name):
        err = float(np.abs(got.cpu().numpy() - want).max() / max(np.abs(want).max(), 1e-30))
        assert err <= tol, f"{what}: {name} {err:.2e}"

    want = oracle.forward(x, *fac, pad)
    s = cp4.capi.shape_for(x.shape, *f, pad)
    assert cp4.default_variant(s) is not None
    close(cp4.conv2d_forward(dev(x), *f, pad=pad), want, 1e-4, "forward, library's choice")
    for v, name, ok in cp4.forward_variants(s):
        if ok:
            close(cp4.conv2d_forward(dev(x), *f, pad=pad, variant=v), want, 1e-4, "forward " + name)
    close(cp4.conv2d_backward_data(dev(dy), *f, pad=pad), oracle.backward_data(dy, *fac, pad), 1e-4,
          "backward-data")
    grads = oracle.backward_filter(x, dy, *fac, pad)
    for variant in (-1, 0, 1, 2):
        try:
            got = cp4.conv2d_backward_filter(dev(x), dev(dy), *f, pad=pad, variant=variant)
        except cp4.Cp4Error as e:           # a matrix-core variant that does not take the shape
            assert variant > 0 and e.status == cp4.capi.ERR_UNSUPPORTED
            continue
        for g, wnt, k in zip(got, grads, FACTORS):
            close(g, wnt, 1e-3, f"d{k} (backward-filter variant {variant})")
    cp4.device_status()
