"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and rejects bad arguments before touching a device."""
import ctypes
import os
import random
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    from paralleltnnlayers_amd import capi
    return capi.lib()


def declared_functions(header="capi.h"):
    text = open(os.path.join(ROOT, "include", "cp4", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cp[34]_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_three_passes():
    names = declared_functions()
    for n in ("cp4_conv2d_forward", "cp4_conv2d_backward_data",
              "cp4_conv2d_backward_filter", "cp4_conv2d_backward_filter_full",
              "cp4_time_forward", "cp4_tune_forward", "cp4_device_malloc"):
        assert n in names
    assert len(names) >= 30


@pytest.mark.parametrize("name", declared_functions())
def test_symbol_exported(L, name):
    assert getattr(L, name) is not None


@pytest.mark.parametrize("name", declared_functions("dense.h"))
def test_dense_symbol_exported(name):
    """libcp4dense.so (MIOpen comparator) loads without a GPU and exports what
    include/cp4/dense.h declares."""
    from paralleltnnlayers_amd import dense
    assert getattr(dense.lib(), name) is not None


def test_dense_argument_errors_need_no_device():
    from paralleltnnlayers_amd import capi, dense
    D = dense.lib()
    one = ctypes.c_void_p(16)   # never dereferenced: checks fail first
    assert D.cp4_dense_conv2d_forward(None, one, one, one, None) == capi.ERR_NULL_POINTER
    valid = capi.Shape(N=1, H=4, W=4, pad=0, T=2, C=2, Y=3, X=3, Rank=0)
    assert D.cp4_dense_conv2d_forward(ctypes.byref(valid), one, one, one, None) == capi.ERR_SHAPE
    assert b"2*pad" in D.cp4_dense_last_error_message()


def test_shape_struct_matches_reference_order():
    from paralleltnnlayers_amd.capi import Shape
    assert [f for f, _ in Shape._fields_] == ["N", "H", "W", "pad", "T", "C", "Y", "X", "Rank"]
    assert ctypes.sizeof(Shape) == 36


def test_argument_errors_need_no_device(L):
    from paralleltnnlayers_amd import capi
    good = capi.Shape(N=1, H=4, W=4, pad=1, T=2, C=2, Y=3, X=3, Rank=2)
    one = ctypes.c_void_p(16)   # never dereferenced: checks fail first
    assert L.cp4_conv2d_forward(None, one, one, one, one, one, one, None) == capi.ERR_NULL_POINTER
    assert L.cp4_conv2d_forward(ctypes.byref(good), None, one, one, one, one, one, None) \
        == capi.ERR_NULL_POINTER
    assert b"NULL" in L.cp4_last_error_message()
    for field in ("H", "W", "T", "C", "Y", "X", "Rank"):
        bad = capi.Shape(N=1, H=4, W=4, pad=1, T=2, C=2, Y=3, X=3, Rank=2)
        setattr(bad, field, 0)
        assert L.cp4_conv2d_forward(ctypes.byref(bad), one, one, one, one, one, one, None) \
            == capi.ERR_SHAPE, field
        assert L.cp4_conv2d_backward_data(ctypes.byref(bad), one, one, one, one, one, one, None) \
            == capi.ERR_SHAPE, field
    huge = capi.Shape(N=1, H=1 << 16, W=1 << 16, pad=1, T=2, C=2, Y=3, X=3, Rank=2)
    assert L.cp4_conv2d_forward(ctypes.byref(huge), one, one, one, one, one, one, None) \
        == capi.ERR_SHAPE
    # empty batch is a valid no-op and needs no pointers
    empty = capi.Shape(N=0, H=4, W=4, pad=1, T=2, C=2, Y=3, X=3, Rank=2)
    assert L.cp4_conv2d_forward(ctypes.byref(empty), None, None, None, None, None, None, None) \
        == capi.OK
    assert L.cp4_conv2d_backward_data(ctypes.byref(empty), None, None, None, None, None, None,
                                      None) == capi.OK
    # backward-filter: workspace too small is reported before any launch
    need = L.cp4_conv2d_backward_filter_workspace_bytes(ctypes.byref(good))
    assert need > 0
    args = [one] * 10
    assert L.cp4_conv2d_backward_filter(ctypes.byref(good), *args, one, need - 1, None) \
        == capi.ERR_WORKSPACE
    assert L.cp4_conv2d_backward_filter(ctypes.byref(good), *args, None, need, None) \
        == capi.ERR_WORKSPACE
    # variant index out of range
    assert L.cp4_forward_variant_supported(ctypes.byref(good), 99) == capi.ERR_UNSUPPORTED
    assert L.cp4_forward_variant_supported(ctypes.byref(good), 0) == capi.OK
    us = ctypes.c_float()
    assert L.cp4_time_forward(ctypes.byref(good), one, one, one, one, one, one, 0, 0,
                              ctypes.byref(us), None) == capi.ERR_SHAPE


def test_default_variant_on_wide_planes(L):
    """The variant choice needs no GPU (the planners assume 256 compute units when
    no device is current).  Rows beyond 128 pixels: whole-row strips where their
    plan keeps a few rows (up to 16 ranks the LDS plane holds half the rank rows),
    tiles where strips would be a row or two; a tuned entry overrides both."""
    from paralleltnnlayers_amd import capi

    def shape(N, C, H, W, T, R, Y=3):
        return capi.Shape(N=N, H=H, W=W, pad=Y // 2, T=T, C=C, Y=Y, X=Y, Rank=R)
    capi.tune_clear()
    assert capi.default_variant(shape(32, 256, 56, 56, 256, 32)) == "mfma_bf16x3_pipe"
    assert capi.default_variant(shape(8, 64, 224, 224, 64, 16)) == "mfma_bf16x3_pipe"
    assert capi.default_variant(shape(8, 64, 224, 224, 64, 32)) == "mfma_bf16x3_pipe_tiled"
    assert capi.default_variant(shape(2, 64, 512, 512, 64, 16)) == "mfma_bf16x3_pipe_tiled"
    assert capi.default_variant(shape(8, 48, 150, 300, 48, 16)) == "mfma_bf16x3_pipe_tiled"
    # up to 32 input and 64 output channels, 16 ranks, from 60,000 pixels on: the few-channel kernel
    assert capi.default_variant(shape(8, 32, 150, 300, 32, 16)) == "mfma_bf16x3_few"
    assert capi.default_variant(shape(16, 16, 512, 512, 16, 16)) == "mfma_bf16x3_few"
    assert capi.default_variant(shape(16, 256, 160, 160, 256, 16)) == "mfma_bf16x3_pipe"
    assert capi.default_variant(shape(1, 3, 512, 512, 1, 16)) == "dense_small_valu"
    # small layers with few channels: the light kernel (workload C1), not beyond its bounds
    assert capi.default_variant(shape(1, 16, 32, 32, 16, 8)) == "mfma_bf16x3_light"
    assert capi.default_variant(shape(16, 64, 32, 32, 64, 16)) == "mfma_bf16x3_pipe"
    assert capi.default_variant(shape(32, 16, 56, 56, 16, 16)) == "mfma_bf16x3_few"
    assert capi.default_variant(shape(8, 64, 224, 224, 64, 16), backward_data=True) \
        == "mfma_bf16x3_pipe"
    s = shape(8, 64, 224, 224, 64, 16)
    tiled = [v for v, n, _ in capi.forward_variants() if n == "mfma_bf16x3_pipe_tiled"][0]
    capi.set_tuned_choice(s, tiled, 14, 64, 1)
    assert capi.default_variant(s) == "mfma_bf16x3_pipe_tiled"
    capi.tune_clear()
    assert capi.default_variant(s) == "mfma_bf16x3_pipe"
    assert capi.default_variant(capi.Shape(N=1, H=0, W=8, pad=1, T=4, C=4, Y=3, X=3, Rank=2)) is None


def test_plan_query_names_what_a_launch_runs(L):
    """The plan report needs no GPU: the headline forward runs eight-row strips, 224 workgroups in one
    wave, its backward-filter takes the four-launch variant, a small layer's the
    three-launch one; an invalid pass is a shape error."""
    from paralleltnnlayers_amd import capi
    capi.tune_clear()
    s = capi.Shape(N=32, H=56, W=56, pad=1, T=256, C=256, Y=3, X=3, Rank=32)
    p = capi.plan_query(s, "forward")
    assert p == {"variant": "mfma_bf16x3_pipe", "strip_rows": 8, "workgroups": 224}
    assert capi.plan_query(s, "backward_data")["variant"] == "mfma_bf16x3_pipe"
    # one image leaves 28 strips: the 16 blocks of output channels are cut into 8 slices
    one = capi.Shape(N=1, H=28, W=28, pad=1, T=512, C=512, Y=3, X=3, Rank=16)
    assert capi.plan_query(one, "forward") == {"variant": "mfma_bf16x3_pipe", "strip_rows": 1,
                                               "workgroups": 224}
    names = capi.backward_filter_variants()
    assert capi.plan_query(s, "backward_filter")["variant"] == names[1]
    small = capi.Shape(N=8, H=28, W=28, pad=1, T=64, C=64, Y=3, X=3, Rank=16)
    assert capi.plan_query(small, "backward_filter")["variant"] == names[2]
    capi.set_tuned_filter_choice(small, 1)
    assert capi.plan_query(small, "backward_filter")["variant"] == names[1]
    capi.tune_clear()
    # few channels on both sides: the dense gradient over tiles and the chain rule, with plain
    # multiply-adds (three channels to one) or on the matrix cores; not workload C1's 1024 pixels
    for dims in ((128, 3, 512, 512, 1), (16, 16, 512, 512, 16), (16, 32, 256, 256, 32),
                 (16, 3, 112, 112, 64), (8, 8, 256, 256, 8)):
        few = capi.Shape(N=dims[0], H=dims[2], W=dims[3], pad=1, T=dims[4], C=dims[1], Y=3, X=3, Rank=16)
        assert capi.plan_query(few, "backward_filter")["variant"] == names[3], dims
        assert L.cp4_conv2d_backward_filter_workspace_bytes(ctypes.byref(few)) >= 2 * 4 * 9 * dims[1] * dims[4]
    c1 = capi.Shape(N=1, H=32, W=32, pad=1, T=16, C=16, Y=3, X=3, Rank=8)
    assert capi.plan_query(c1, "backward_filter")["variant"] != names[3]
    v = ctypes.c_int()
    assert L.cp4_plan_query(ctypes.byref(s), 3, ctypes.byref(v), None, None) == capi.ERR_SHAPE


def test_status_strings(L):
    seen = {L.cp4_status_string(i) for i in range(6)}
    assert len(seen) == 6 and b"ok" in seen


def test_workload_byte_counts():
    """Algorithmic bytes of the five workloads (reference formula,
    Cuda_kernels/cp4Conv2d.cu:176-178)."""
    from paralleltnnlayers_amd.configs import WORKLOADS, algorithmic_bytes, minimal_flops
    want = {"C1": 132288, "C2": 8397184, "C3": 205587200, "C4": 25707136, "C5": 25955328}
    for k, v in want.items():
        assert algorithmic_bytes(WORKLOADS[k]) == v
    assert minimal_flops(WORKLOADS["C3"]) == 3326869504
    assert minimal_flops(WORKLOADS["C5"]) == 1673068544


def test_geometry_helpers_need_no_device(L):
    """cp4_geometry_same / _valid / _symmetric and the checks of the _ex entry points."""
    from paralleltnnlayers_amd import capi
    s = capi.Shape(N=1, H=8, W=9, pad=0, T=2, C=2, Y=3, X=3, Rank=2)
    g = capi.geometry(s, 2, "same")          # even size: no zeros before the image
    assert (g.pad_top, g.pad_left, g.out_h, g.out_w) == (0, 1, 4, 5)
    g = capi.geometry(s, 2, "valid")
    assert (g.pad_top, g.pad_left, g.out_h, g.out_w) == (0, 0, 3, 4)
    g = capi.geometry(s, (2, 1), 1)
    assert (g.stride_h, g.stride_w, g.pad_top, g.out_h, g.out_w) == (2, 1, 1, 4, 9)
    one = ctypes.c_void_p(256)               # never dereferenced: checks fail first
    bad = capi.Geometry(2, 2, 3, 0, 4, 4)    # pad_top > Y - 1
    assert L.cp4_conv2d_forward_ex(ctypes.byref(s), ctypes.byref(bad), one, one, one, one, one,
                                   None, 0, one, None) == capi.ERR_SHAPE
    far = capi.Geometry(2, 2, 0, 0, 40, 4)   # the output plane reaches past the image
    assert L.cp4_conv2d_forward_ex(ctypes.byref(s), ctypes.byref(far), one, one, one, one, one,
                                   None, 0, one, None) == capi.ERR_SHAPE
    assert L.cp4_conv2d_forward_ex(ctypes.byref(s), None, one, one, one, one, one, None, 0, one,
                                   None) == capi.ERR_NULL_POINTER
    assert capi.backward_ex_workspace_bytes(s, capi.geometry(s, 2, "same")) > 0


def test_backward_filter_workspace_sizes_over_random_shapes():
    """The workspace query plans every backward-filter variant on the host: it must
    answer (a positive size, no crash) for any valid shape, also those none of the
    matrix-core variants takes (tiny or odd planes, channel counts off the tiles,
    more than 64 ranks, a padding that is not "same")."""
    from paralleltnnlayers_amd import capi
    L = capi.lib()
    rng = random.Random(7)
    for _ in range(4000):
        fs = rng.choice((1, 2, 3, 5, 7, 9))
        s = capi.Shape(N=rng.choice((1, 2, 3, 8, 64)), H=rng.randint(1, 70), W=rng.randint(1, 70),
                       pad=rng.choice((0, 1, 2, 3, fs // 2)), T=rng.choice((1, 3, 16, 48, 96, 320)),
                       C=rng.choice((1, 5, 16, 32, 64, 256, 528)), Y=fs, X=fs,
                       Rank=rng.choice((1, 2, 7, 16, 32, 33, 64, 65, 130)))
        need = L.cp4_conv2d_backward_filter_workspace_bytes(ctypes.byref(s))
        assert need > 0, s
