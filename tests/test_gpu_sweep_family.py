"""The reference's "Extended" forward test on its six sweep lists
(Cuda_kernels/test/test_cp4Conv.cpp.cu:105-171 runs every row of
bench/tensors_{all_scales,batch_size,channel_depth,filter_count,filter_size,image_size}.txt
against the vendor library's dense convolution on the recomposed filter).

The rows are typed in below as the grids those files spell out (N C H W pad T Y X
Rank); no file of the reference is read.  Each row runs through the C ABI with
the library's own choice of kernel and is checked

  * against the CPU oracle where that finishes in about a second, and
  * against MIOpen's dense convolution on the recomposed filter - the
    reference's own method; the comparator is pinned to the oracle in
    tests/test_gpu_dense.py - for the rows beyond that (batches of 512 x 512
    images, planes of 1024 x 1024 and more),

to the forward bar: max |a - b| <= 1e-4 * max |b| and |a - b| <= 1e-5 + 1e-4 |b|
for all but one element in a thousand (the reference's AllClose counts
exceedances the same way, Utils.cu:143-180).  Inputs follow the reference's test
(uniform in (0, 1], as its random_fill gives); factors are scaled so that outputs
stay of order one.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RANKS = (1, 2, 4, 8, 16)


def rows_all_scales():
    # tensors_all_scales.txt: channels, filters and the image edge double together
    out = [(n, c, e, e, 1, c, 3, 3, 1) for n, c, e in
           ((1, 1, 32), (2, 2, 64), (3, 4, 128), (4, 8, 256), (5, 16, 512), (5, 32, 1024))]
    for r in RANKS[1:]:
        out += [(c, c, e, e, 1, c, 3, 3, r) for c, e in ((1, 32), (2, 64), (4, 128), (8, 256), (16, 512))]
    return out


def rows_batch_size():
    return [(n, 3, 512, 512, 1, 1, 3, 3, r) for r in RANKS for n in (1, 2, 4, 8, 16, 32, 64, 128)]


def rows_channel_depth():
    return [(1, c, 512, 512, 1, 1, 3, 3, r) for r in RANKS for c in (1, 2, 3, 4, 8, 16, 32, 64, 128)]


def rows_filter_count():
    return [(1, 3, 512, 512, 1, t, 3, 3, r) for r in RANKS for t in (1, 2, 4, 8, 16, 32, 64, 128)]


def rows_filter_size():
    return [(1, 3, 512, 512, (y - 1) // 2, 1, y, y, r) for r in RANKS for y in range(3, 18, 2)]


def rows_image_size():
    return [(1, 3, e, e, 1, 1, 3, 3, r) for r in RANKS for e in (32, 64, 128, 256, 512, 1024, 2048, 4096)]


LISTS = {"all_scales": rows_all_scales, "batch_size": rows_batch_size,
         "channel_depth": rows_channel_depth, "filter_count": rows_filter_count,
         "filter_size": rows_filter_size, "image_size": rows_image_size}


def test_the_lists_have_the_reference_row_counts():
    assert {k: len(f()) for k, f in LISTS.items()} == {
        "all_scales": 26, "batch_size": 40, "channel_depth": 45, "filter_count": 40,
        "filter_size": 40, "image_size": 40}


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


@pytest.fixture(scope="module")
def dense():
    from paralleltnnlayers_amd import dense as d
    d.lib()
    return d


def oracle_is_quick(row):
    N, C, H, W, pad, T, Y, X, R = row
    per_image = H * W * R * (C + T + Y + X)         # multiply-adds of the unfused sequence
    return per_image <= 6e8 and N * per_image <= 3e9 and R * H * W <= 1 << 25


def check_row(cp4, oracle, dense, row, seed):
    N, C, H, W, pad, T, Y, X, R = row
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = 1.0 - torch.rand((N, C, H, W), device="cuda", generator=g)          # (0, 1]
    scale = (R * C * Y * X) ** -0.25
    f = [(torch.randn((d, R), device="cuda", generator=g) * scale).contiguous() for d in (T, C, Y, X)]
    y = cp4.conv2d_forward(x, *f, pad=pad)
    if oracle_is_quick(row):
        want = torch.from_numpy(oracle.forward(x.cpu().numpy(), *[t.cpu().numpy() for t in f], pad)).cuda()
        how = "oracle"
    else:
        want = dense.conv2d_forward(x, cp4.recompose(*f), pad)
        how = "dense comparator"
    top = float(want.abs().max())
    assert top > 0
    err = (y - want).abs()
    assert float(err.max()) <= 1e-4 * top, f"{row} vs {how}: normalised {float(err.max()) / top:.2e}"
    bad = int((err > 1e-5 + 1e-4 * want.abs()).sum())
    assert bad == 0, f"{row} vs {how}: {bad} of {y.numel()} elements beyond the bar"
    return how


@pytest.mark.parametrize("name", list(LISTS))
def test_sweep_list_forward(cp4, oracle, dense, name):
    used = {"oracle": 0, "dense comparator": 0}
    for i, row in enumerate(LISTS[name]()):
        used[check_row(cp4, oracle, dense, row, seed=1000 + i)] += 1
    cp4.device_status()
    assert used["oracle"] >= len(LISTS[name]()) // 2      # the comparator only for the big rows
