"""The dense comparator (MIOpen behind include/cp4/dense.h) against the oracle,
and the CP4 kernels against the comparator — the reference's own test method
(Cuda_kernels/test/test_cp4Conv.cpp.cu:14-101: cuDNN on the recomposed filter
vs the fused CP4 kernels, AllClose 1e-5 / 1e-4)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


@pytest.fixture(scope="module")
def dense():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from paralleltnnlayers_amd import dense as d
    d.lib()
    return d


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


# N, C, H, W, pad, T, Y, R  (2*pad = Y-1: the comparator's H x W output)
CASES = [
    (1, 48, 55, 55, 5, 256, 11, 16),   # the reference's single-kernel test case
    (2, 64, 28, 28, 1, 32, 3, 16),
    (3, 16, 17, 20, 2, 24, 5, 8),
    (2, 8, 9, 9, 0, 8, 1, 4),
]


@pytest.mark.parametrize("dims", CASES, ids=lambda d: "x".join(map(str, d)))
def test_dense_comparator_and_cp4(cp4, oracle, dense, dims):
    N, C, H, W, pad, T, Y, R = dims
    rng = np.random.default_rng(sum(dims))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, T, H, W)).astype(np.float32)
    fac = [rng.standard_normal((d, R)).astype(np.float32) / np.sqrt(R) for d in (T, C, Y, Y)]
    f = [dev(v) for v in fac]
    K = cp4.recompose(*f)                               # [T,C,Y,X] on the device

    # dense library vs the CPU oracle of the CP4 formula (independent of our kernels)
    y_dense = dense.conv2d_forward(dev(x), K, pad).cpu().numpy()
    y_want = oracle.forward(x, *fac, pad)
    scale = np.abs(y_want).max()
    assert np.abs(y_dense - y_want).max() <= 1e-4 * scale
    dx_dense = dense.conv2d_backward_data(dev(dy), K, pad).cpu().numpy()
    dx_want = oracle.backward_data(dy, *fac, pad)       # 2*pad = Y-1: the adjoint
    assert np.abs(dx_dense - dx_want).max() <= 1e-4 * np.abs(dx_want).max()
    dK_dense = dense.conv2d_backward_filter(dev(x), dev(dy), Y, Y, pad).cpu().numpy()
    dK_want = oracle.backward_filter_full(x, dy, Y, Y, pad)
    assert np.abs(dK_dense - dK_want).max() <= 1e-3 * np.abs(dK_want).max()

    # our kernels vs the dense library, as the reference's tests compare them
    y_cp4 = cp4.conv2d_forward(dev(x), *f, pad=pad)
    assert cp4.count_exceeding(y_cp4, dev(y_dense), 1e-3) <= y_cp4.numel() // 1000
    assert (y_cp4.cpu().numpy() - y_dense).__abs__().max() <= 1e-4 * scale
    dx_cp4 = cp4.conv2d_backward_data(dev(dy), *f, pad=pad).cpu().numpy()
    assert np.abs(dx_cp4 - dx_dense).max() <= 1e-4 * np.abs(dx_dense).max()
    dK_cp4 = cp4.conv2d_backward_filter_full(dev(x), dev(dy), Y, Y, pad=pad).cpu().numpy()
    assert np.abs(dK_cp4 - dK_dense).max() <= 1e-3 * np.abs(dK_dense).max()


def test_dense_rejects_non_same_padding(cp4, dense):
    x = torch.zeros((1, 4, 8, 8), device="cuda")
    K = torch.zeros((4, 4, 3, 3), device="cuda")
    with pytest.raises(cp4.Cp4Error) as e:
        dense.conv2d_forward(x, K, pad=0)
    assert e.value.status == 2 and "2*pad" in str(e.value)


def test_dense_timing_loop(cp4, dense):
    x = torch.randn((4, 32, 28, 28), device="cuda")
    K = torch.randn((32, 32, 3, 3), device="cuda")
    y = torch.empty((4, 32, 28, 28), device="cuda")
    us = dense.time_forward(x, K, y, pad=1, warmup=2, profcount=10)
    assert 0.5 < us < 5e4
    want = torch.nn.functional.conv2d(x, K, padding=1)
    assert (y - want).abs().max() <= 1e-3 * want.abs().max()


def test_bench_time_driver_dense_column(tmp_path):
    """cp4_bench_time prints the vendor library's time in the first data column
    (Cuda_kernels/bench/BenchBothTime.cu:84-98)."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "paralleltnnlayers_amd", "csrc", "cp4_bench_time")
    if not os.path.exists(exe):
        pytest.skip("host binaries not built")
    shapes = tmp_path / "tensors.txt"
    shapes.write_text("# N C H W pad T Y X\n2 16 14 14 1 16 3 3\n1 8 9 9 0 8 3 3\n")
    out = subprocess.run([exe, str(shapes)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    rows = [l for l in out.stdout.strip().splitlines()[1:]]
    assert len(rows) == 2
    first = rows[0].split(",")
    assert len(first) == 7 and float(first[1]) > 0         # dense column is a time
    assert rows[1].split(",")[1].strip() == "nan"          # pad 0 with a 3x3 filter
