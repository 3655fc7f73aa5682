"""The C++ operator API (Tensor, namespace CP, reference-signature launchers):
the library loads and exports the reference's entry points (CPU), and the C++
test executable passes on a GPU."""
import ctypes
import os
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                    "paralleltnnlayers_amd", "csrc")

# Itanium-mangled names of the reference's free functions with their original
# signatures (Cuda_kernels/cp4Conv2dForward.cuh:7-14, cp4Conv2dBackwardData.cuh:7-14,
# cp4Conv2dBackwardFilter.cuh:7-47, cp4Conv2d.cuh:30-31, Utils.cuh:9).
SYMBOLS = [
    "_Z22cp4_conv2d_forward_gpu12tensor_shapePKfS1_S1_S1_S1_Pfj",
    "_Z28cp4_conv2d_backward_data_gpu12tensor_shapePKfS1_S1_S1_S1_Pfj",
    "_Z35cp4_conv2d_backward_filter_full_gpu12tensor_shapePfPKfS2_j",
    "_Z32cp4_conv2d_backward_filter_t_gpu12tensor_shapePfPKfS2_S2_S2_S2_j",
    "_Z32cp4_conv2d_backward_filter_c_gpu12tensor_shapePfPKfS2_S2_S2_S2_j",
    "_Z32cp4_conv2d_backward_filter_y_gpu12tensor_shapePfPKfS2_S2_S2_S2_j",
    "_Z32cp4_conv2d_backward_filter_x_gpu12tensor_shapePfPKfS2_S2_S2_S2_j",
    "_ZN2CP15run_convolutionE12tensor_shapej",
    "_Z11random_fillSt16initializer_listIjE",
    "_ZN6TensorC1ESt16initializer_listIjE",
    "_ZNK6Tensor4sizeEv",
]


@pytest.fixture(scope="module")
def host_lib():
    from paralleltnnlayers_amd import capi
    capi.lib()  # libcp4conv.so first, globally, so the dependency resolves anywhere
    ctypes.CDLL(capi.library_path(), mode=ctypes.RTLD_GLOBAL)
    return ctypes.CDLL(os.path.join(CSRC, "libcp4host.so"))


@pytest.mark.parametrize("name", SYMBOLS)
def test_reference_entry_points_exported(host_lib, name):
    assert getattr(host_lib, name) is not None


def test_host_executables_built():
    for exe in ("cp4_bench_time", "cp4_bench_mem", "cp4_conv2d_forward", "cp4_host_tests"):
        assert os.access(os.path.join(CSRC, exe), os.X_OK), exe
    # usage error path of the bench driver needs no GPU
    r = subprocess.run([os.path.join(CSRC, "cp4_bench_time")], capture_output=True, text=True)
    assert r.returncode == 1 and "USAGE" in r.stderr


@pytest.mark.gpu
def test_cpp_host_api_suite():
    r = subprocess.run([os.path.join(CSRC, "cp4_host_tests")], capture_output=True, text=True,
                       timeout=100, cwd=CSRC)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "host API tests passed" in r.stdout


@pytest.mark.gpu
def test_bench_driver_csv(tmp_path):
    """CSV layout of the reference's timing driver
    (Cuda_kernels/bench/BenchBothTime.cu:49, 86-101)."""
    shapes = tmp_path / "shapes.txt"
    shapes.write_text("# N C H W pad T Y X\n1 192 13 13 1 256 3 3\n1 192 13 13 1 256 3 3\n"
                      "1  48 55 55 2 256 5 5\n")
    r = subprocess.run([os.path.join(CSRC, "cp4_bench_time"), str(shapes)], capture_output=True,
                       text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0] == "N C H W pad T Y X, cuDNN, Rank 1, Rank 2, Rank 4, Rank 8, Rank 16"
    assert len(lines) == 3 and lines[1].startswith("1 192 13 13 1 256 3 3, ")
    assert float(lines[1].split(",")[1]) > 0          # the vendor library's dense time
    assert all(float(v) > 0 for v in lines[2].split(", ")[2:])
    r = subprocess.run([os.path.join(CSRC, "cp4_bench_mem"), str(shapes)], capture_output=True,
                       text=True, timeout=100)
    kib = [int(v) for v in r.stdout.strip().splitlines()[1].split(", ")[1:]]
    assert kib[1] == 4 * (256 * 169 + 192 * 169 + 1 * (256 + 192 + 3 + 3)) // 1024
