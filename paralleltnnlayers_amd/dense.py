"""ctypes binding of ``csrc/libcp4dense.so``: the vendor library's (MIOpen's)
dense fp32 NCHW convolution behind the C ABI of ``include/cp4/dense.h`` — the
comparator the reference takes from cuDNN (Cuda_kernels/NVConv2d.cu).  Used by
the tests to check the CP4 kernels against a dense convolution with the
recomposed filter on the device, and for the dense timing column."""
import ctypes
import os

import torch

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "csrc", "libcp4dense.so")
_lib = None


def lib():
    """The loaded comparator library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB):
        raise ImportError(f"{_LIB} is missing: build it with `make -C paralleltnnlayers_amd/csrc`.")
    capi.lib()                                   # libcp4dense.so links against libcp4conv.so
    L = ctypes.CDLL(_LIB)
    L.cp4_dense_last_error_message.restype = ctypes.c_char_p
    S, F = ctypes.POINTER(capi.Shape), ctypes.c_void_p
    for name in ("cp4_dense_conv2d_forward", "cp4_dense_conv2d_backward_data",
                 "cp4_dense_conv2d_backward_filter"):
        fn = getattr(L, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [S, F, F, F, ctypes.c_void_p]
    L.cp4_dense_time_forward.restype = ctypes.c_int
    L.cp4_dense_time_forward.argtypes = [S, F, F, F, ctypes.c_uint, ctypes.c_uint,
                                         ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    L.cp4_dense_release.restype = None
    _lib = L
    return L


def _check(status):
    if status != capi.OK:
        raise capi.Cp4Error(status, f"{capi.lib().cp4_status_string(status).decode()}: "
                                    f"{lib().cp4_dense_last_error_message().decode()}")


def _shape(act_shape, C, Kshape, pad):
    N, _, H, W = act_shape
    T, _, Y, X = Kshape
    return capi.Shape(N=N, H=H, W=W, pad=pad, T=T, C=C, Y=Y, X=X, Rank=0)


def conv2d_forward(x, K, pad, stream=None):
    """x[N,C,H,W] (*) K[T,C,Y,X] -> y[N,T,H,W] (NV::Conv2dForward)."""
    s = _shape(x.shape, x.shape[1], K.shape, pad)
    y = torch.empty((s.N, s.T, s.H, s.W), device=x.device, dtype=torch.float32)
    _check(lib().cp4_dense_conv2d_forward(ctypes.byref(s), capi._ptr(x), capi._ptr(K),
                                          capi._ptr(y), capi._stream(stream)))
    return y


def conv2d_backward_data(dy, K, pad, stream=None):
    """dy[N,T,H,W], K[T,C,Y,X] -> dx[N,C,H,W] (NV::Conv2dBackwardData)."""
    s = _shape(dy.shape, K.shape[1], K.shape, pad)
    dx = torch.empty((s.N, s.C, s.H, s.W), device=dy.device, dtype=torch.float32)
    _check(lib().cp4_dense_conv2d_backward_data(ctypes.byref(s), capi._ptr(dy), capi._ptr(K),
                                                capi._ptr(dx), capi._stream(stream)))
    return dx


def conv2d_backward_filter(x, dy, Y, X, pad, stream=None):
    """x[N,C,H,W], dy[N,T,H,W] -> dK[T,C,Y,X] (NV::Conv2dBackwardFilter)."""
    s = _shape(x.shape, x.shape[1], (dy.shape[1], x.shape[1], Y, X), pad)
    dK = torch.empty((s.T, s.C, Y, X), device=x.device, dtype=torch.float32)
    _check(lib().cp4_dense_conv2d_backward_filter(ctypes.byref(s), capi._ptr(x), capi._ptr(dy),
                                                  capi._ptr(dK), capi._stream(stream)))
    return dK


def time_forward(x, K, y, pad, warmup=1, profcount=47, stream=None):
    s = _shape(x.shape, x.shape[1], K.shape, pad)
    us = ctypes.c_float()
    _check(lib().cp4_dense_time_forward(ctypes.byref(s), capi._ptr(x), capi._ptr(K), capi._ptr(y),
                                        warmup, profcount, ctypes.byref(us),
                                        capi._stream(stream)))
    return us.value
