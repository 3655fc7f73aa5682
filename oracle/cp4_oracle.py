"""ctypes binding of the CPU oracle (oracle/cp4_oracle.c).

Test infrastructure only: imported by tests/, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of bench.py as the checker / reported CPU
baseline.  The shipped package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcp4oracle.so")


class Shape(ctypes.Structure):
    """Same nine unsigned fields, same order, as the reference's tensor_shape
    (Cuda_kernels/Tensor.cuh:10-19)."""
    _fields_ = [(k, ctypes.c_uint) for k in
                ("N", "H", "W", "pad", "T", "C", "Y", "X", "Rank")]


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
        subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.cp4o_count_exceeding.restype = ctypes.c_long
    return _lib


def _fp(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def shape_of(x_shape, FK, FC, FH, FW, pad):
    """tensor_shape from operand shapes, as CP::Conv2dForward derives it
    (Cuda_kernels/cp4Conv2d.cu:21-30)."""
    N, C, H, W = x_shape
    return Shape(N=N, H=H, W=W, pad=pad, T=FK.shape[0], C=C, Y=FH.shape[0],
                 X=FW.shape[0], Rank=FK.shape[1])


def num_threads():
    return int(lib().cp4o_num_threads())


def recompose(FK, FC, FH, FW):
    FK, FC, FH, FW = map(_f32, (FK, FC, FH, FW))
    s = Shape(T=FK.shape[0], C=FC.shape[0], Y=FH.shape[0], X=FW.shape[0],
              Rank=FK.shape[1])
    K = np.empty((s.T, s.C, s.Y, s.X), np.float32)
    lib().cp4o_recompose(ctypes.byref(s), _fp(FK), _fp(FC), _fp(FH), _fp(FW), _fp(K))
    return K


def forward(x, FK, FC, FH, FW, pad, direct=False):
    x, FK, FC, FH, FW = map(_f32, (x, FK, FC, FH, FW))
    s = shape_of(x.shape, FK, FC, FH, FW, pad)
    assert FC.shape == (s.C, s.Rank)
    y = np.empty((s.N, s.T, s.H, s.W), np.float32)
    fn = lib().cp4o_forward_direct if direct else lib().cp4o_forward_unfused
    rc = fn(ctypes.byref(s), _fp(x), _fp(FK), _fp(FC), _fp(FH), _fp(FW), _fp(y))
    assert direct or rc == 0
    return y


def cp3_forward(x, K0, K1, K2, pad):
    """3-factor CP forward (pointwise K0 [C,R], depthwise K1 [Y,X,R], pointwise K2 [R,T])."""
    x, K0, K1, K2 = map(_f32, (x, K0, K1, K2))
    N, C, H, W = x.shape
    s = Shape(N=N, H=H, W=W, pad=pad, T=K2.shape[1], C=C, Y=K1.shape[0], X=K1.shape[1],
              Rank=K0.shape[1])
    assert K0.shape == (C, s.Rank) and K1.shape[2] == s.Rank and K2.shape[0] == s.Rank
    y = np.empty((N, s.T, H, W), np.float32)
    lib().cp3o_forward_direct(ctypes.byref(s), _fp(x), _fp(K0), _fp(K1), _fp(K2), _fp(y))
    return y


def rcp_forward(x, K0, K1, KC, pad):
    """Reshaped-CP forward: K0 [S0,T0,R], K1 [S1,T1,R], KC [Y,X,R]; x has S0*S1 channels."""
    x, K0, K1, KC = map(_f32, (x, K0, K1, KC))
    N, C, H, W = x.shape
    S0, T0, R = K0.shape
    S1, T1, _ = K1.shape
    assert C == S0 * S1 and K1.shape[2] == R and KC.shape[2] == R
    s = Shape(N=N, H=H, W=W, pad=pad, T=T0 * T1, C=C, Y=KC.shape[0], X=KC.shape[1], Rank=R)
    y = np.empty((N, s.T, H, W), np.float32)
    lib().rcpo_forward_direct(ctypes.byref(s), ctypes.c_uint(S0), ctypes.c_uint(S1),
                              ctypes.c_uint(T0), ctypes.c_uint(T1), _fp(x), _fp(K0), _fp(K1),
                              _fp(KC), _fp(y))
    return y


def backward_data(dy, FK, FC, FH, FW, pad, direct=False):
    dy, FK, FC, FH, FW = map(_f32, (dy, FK, FC, FH, FW))
    N, T, H, W = dy.shape
    assert FK.shape[0] == T
    s = Shape(N=N, H=H, W=W, pad=pad, T=T, C=FC.shape[0], Y=FH.shape[0],
              X=FW.shape[0], Rank=FK.shape[1])
    dx = np.empty((N, s.C, H, W), np.float32)
    fn = (lib().cp4o_backward_data_direct if direct
          else lib().cp4o_backward_data_unfused)
    rc = fn(ctypes.byref(s), _fp(dy), _fp(FK), _fp(FC), _fp(FH), _fp(FW), _fp(dx))
    assert direct or rc == 0
    return dx


def backward_filter(x, dy, FK, FC, FH, FW, pad, direct=False):
    """Returns (dFK, dFC, dFH, dFW)."""
    x, dy, FK, FC, FH, FW = map(_f32, (x, dy, FK, FC, FH, FW))
    s = shape_of(x.shape, FK, FC, FH, FW, pad)
    assert dy.shape == (s.N, s.T, s.H, s.W)
    outs = [np.zeros_like(f) for f in (FK, FC, FH, FW)]
    if direct:
        for which, o in enumerate(outs):
            lib().cp4o_backward_filter_factor_direct(
                ctypes.byref(s), ctypes.c_int(which), _fp(o), _fp(x), _fp(dy),
                _fp(FK), _fp(FC), _fp(FH), _fp(FW))
    else:
        rc = lib().cp4o_backward_filter_unfused(
            ctypes.byref(s), _fp(x), _fp(dy), _fp(FK), _fp(FC), _fp(FH), _fp(FW),
            *[_fp(o) for o in outs])
        assert rc == 0
    return tuple(outs)


class Geometry(ctypes.Structure):
    """stride, zero rows / columns before the image, output plane (cp4o_geometry)."""
    _fields_ = [(k, ctypes.c_uint) for k in
                ("stride_h", "stride_w", "pad_top", "pad_left", "out_h", "out_w")]


def geometry_same(H, W, Y, X, stride):
    """The framework's padding="SAME" that the reference's layers ask for
    (test/layers.py:264-279): out = ceil(in / stride); as many zeros as the last
    window needs, the smaller half of them before the image."""
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    ho, wo = -(-H // sh), -(-W // sw)
    th, tw = max((ho - 1) * sh + Y - H, 0), max((wo - 1) * sw + X - W, 0)
    return Geometry(sh, sw, th // 2, tw // 2, ho, wo)


def geometry_valid(H, W, Y, X, stride):
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    return Geometry(sh, sw, 0, 0, (H - Y) // sh + 1, (W - X) // sw + 1)


def geometry_symmetric(H, W, Y, X, stride, pad):
    """pad zeros on every side: out = (in + 2 pad - filter) / stride + 1."""
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    return Geometry(sh, sw, pad, pad, (H + 2 * pad - Y) // sh + 1, (W + 2 * pad - X) // sw + 1)


def forward_geom(x, FK, FC, FH, FW, g, direct=False):
    x, FK, FC, FH, FW = map(_f32, (x, FK, FC, FH, FW))
    s = shape_of(x.shape, FK, FC, FH, FW, 0)
    y = np.empty((s.N, s.T, g.out_h, g.out_w), np.float32)
    fn = lib().cp4o_forward_geom_direct if direct else lib().cp4o_forward_geom_unfused
    rc = fn(ctypes.byref(s), ctypes.byref(g), _fp(x), _fp(FK), _fp(FC), _fp(FH), _fp(FW), _fp(y))
    assert direct or rc == 0
    return y


def backward_data_geom(dy, x_hw, FK, FC, FH, FW, g):
    """dx [N,C,H,W] of the strided map for dy [N,T,out_h,out_w]; x_hw = (H, W)."""
    dy, FK, FC, FH, FW = map(_f32, (dy, FK, FC, FH, FW))
    N, T = dy.shape[:2]
    assert dy.shape[2:] == (g.out_h, g.out_w)
    s = Shape(N=N, H=x_hw[0], W=x_hw[1], pad=0, T=T, C=FC.shape[0], Y=FH.shape[0],
              X=FW.shape[0], Rank=FK.shape[1])
    dx = np.empty((N, s.C, s.H, s.W), np.float32)
    lib().cp4o_backward_data_geom_direct(ctypes.byref(s), ctypes.byref(g), _fp(dy), _fp(FK),
                                         _fp(FC), _fp(FH), _fp(FW), _fp(dx))
    return dx


def backward_filter_geom(x, dy, FK, FC, FH, FW, g):
    """(dFK, dFC, dFH, dFW) of the strided map."""
    x, dy, FK, FC, FH, FW = map(_f32, (x, dy, FK, FC, FH, FW))
    s = shape_of(x.shape, FK, FC, FH, FW, 0)
    assert dy.shape == (s.N, s.T, g.out_h, g.out_w)
    outs = [np.zeros_like(f) for f in (FK, FC, FH, FW)]
    for which, o in enumerate(outs):
        lib().cp4o_backward_filter_geom_direct(
            ctypes.byref(s), ctypes.byref(g), ctypes.c_int(which), _fp(o), _fp(x), _fp(dy),
            _fp(FK), _fp(FC), _fp(FH), _fp(FW))
    return tuple(outs)


def backward_filter_full(x, dy, Y, X, pad):
    """Dense filter gradient dK[T,C,Y,X] (cp4Conv2dBackwardFilter.cu:23-59)."""
    x, dy = _f32(x), _f32(dy)
    N, C, H, W = x.shape
    s = Shape(N=N, H=H, W=W, pad=pad, T=dy.shape[1], C=C, Y=Y, X=X, Rank=0)
    dK = np.zeros((s.T, C, Y, X), np.float32)
    lib().cp4o_backward_filter_full_direct(ctypes.byref(s), _fp(dK), _fp(x), _fp(dy))
    return dK


def count_exceeding(a, b, tol):
    a, b = _f32(a).ravel(), _f32(b).ravel()
    assert a.size == b.size
    return int(lib().cp4o_count_exceeding(_fp(a), _fp(b), ctypes.c_size_t(a.size),
                                          ctypes.c_float(tol)))
