"""ctypes binding of include/cp4/capi.h.

Device memory and streams come from PyTorch (ROCm): every tensor argument must
be a contiguous float32 CUDA(-HIP) tensor; its ``data_ptr()`` is what crosses
the C ABI.  Launches go on torch's current stream unless ``stream`` is given.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "csrc", "libcp4conv.so")


class Cp4Error(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"cp4 status {status}: {message}")
        self.status = status


class Shape(ctypes.Structure):
    """cp4_shape: the nine unsigned fields of the reference's tensor_shape
    (Cuda_kernels/Tensor.cuh:10-19), same order."""
    _fields_ = [(k, ctypes.c_uint) for k in
                ("N", "H", "W", "pad", "T", "C", "Y", "X", "Rank")]

    def __repr__(self):
        return "Shape(" + ", ".join(f"{k}={getattr(self, k)}" for k, _ in self._fields_) + ")"


class Geometry(ctypes.Structure):
    """cp4_geometry: stride, zero rows / columns before the image, output plane."""
    _fields_ = [(k, ctypes.c_uint) for k in
                ("stride_h", "stride_w", "pad_top", "pad_left", "out_h", "out_w")]

    def __repr__(self):
        return "Geometry(" + ", ".join(f"{k}={getattr(self, k)}" for k, _ in self._fields_) + ")"


class RcpDims(ctypes.Structure):
    """rcp_dims: the channel grids of the reshaped-CP op (C = S0*S1, T = T0*T1)."""
    _fields_ = [(k, ctypes.c_uint) for k in ("S0", "S1", "T0", "T1")]


# status codes of cp4_status
(OK, ERR_NULL_POINTER, ERR_SHAPE, ERR_HIP, ERR_WORKSPACE, ERR_UNSUPPORTED,
 ERR_DEVICE) = range(7)

_lib = None
_F = ctypes.c_void_p          # const float* / float* (device)
_S = ctypes.POINTER(Shape)


def library_path():
    return _LIB


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB):
        raise ImportError(
            f"{_LIB} is missing: build it with `python -c 'import __graft_entry__ as g; "
            "g.build()'` (or `make -C paralleltnnlayers_amd/csrc`). There is no fallback path.")
    L = ctypes.CDLL(_LIB)
    L.cp4_status_string.restype = ctypes.c_char_p
    L.cp4_status_string.argtypes = [ctypes.c_int]
    L.cp4_last_error_message.restype = ctypes.c_char_p
    L.cp4_forward_variant_name.restype = ctypes.c_char_p
    L.cp4_forward_default_variant.restype = ctypes.c_int
    L.cp4_forward_default_variant.argtypes = [_S, ctypes.c_int]
    L.cp4_forward_variant_name.argtypes = [ctypes.c_int]
    L.cp4_conv2d_backward_filter_workspace_bytes.restype = ctypes.c_size_t
    L.cp4_conv2d_backward_filter_workspace_bytes.argtypes = [_S]
    fwd = [_S, _F, _F, _F, _F, _F, _F]
    L.cp4_conv2d_forward.argtypes = fwd + [ctypes.c_void_p]
    L.cp4_conv2d_forward_variant.argtypes = fwd + [ctypes.c_int, ctypes.c_void_p]
    L.cp4_conv2d_backward_data.argtypes = fwd + [ctypes.c_void_p]
    L.cp4_conv2d_forward_bias_act.argtypes = [_S, _F, _F, _F, _F, _F, _F, ctypes.c_int, _F,
                                              ctypes.c_void_p]
    _G = ctypes.POINTER(Geometry)
    L.cp4_geometry_same.argtypes = [_S, ctypes.c_uint, ctypes.c_uint, _G]
    L.cp4_geometry_valid.argtypes = [_S, ctypes.c_uint, ctypes.c_uint, _G]
    L.cp4_geometry_symmetric.argtypes = [_S] + [ctypes.c_uint] * 4 + [_G]
    L.cp4_conv2d_forward_ex.argtypes = [_S, _G] + [_F] * 6 + [ctypes.c_int, _F, ctypes.c_void_p]
    L.cp4_conv2d_backward_ex_workspace_bytes.restype = ctypes.c_size_t
    L.cp4_conv2d_backward_ex_workspace_bytes.argtypes = [_S, _G]
    L.cp4_conv2d_backward_data_ex.argtypes = [_S, _G] + [_F] * 6 + [ctypes.c_void_p, ctypes.c_size_t,
                                                                    ctypes.c_void_p]
    L.cp4_conv2d_backward_filter_ex.argtypes = [_S, _G] + [_F] * 10 + [ctypes.c_void_p,
                                                                       ctypes.c_size_t, ctypes.c_void_p]
    _D = ctypes.POINTER(RcpDims)
    L.rcp_conv2d_workspace_bytes.restype = ctypes.c_size_t
    L.rcp_conv2d_workspace_bytes.argtypes = [_S, _D]
    L.rcp_conv2d_forward.argtypes = [_S, _D] + [_F] * 5 + [ctypes.c_void_p, ctypes.c_size_t,
                                                           ctypes.c_void_p]
    L.rcp_conv2d_backward_data.argtypes = L.rcp_conv2d_forward.argtypes
    L.rcp_conv2d_backward_filter.argtypes = [_S, _D] + [_F] * 8 + [ctypes.c_void_p, ctypes.c_size_t,
                                                                   ctypes.c_void_p]
    L.cp4_conv2d_forward_f16.argtypes = [_S, ctypes.c_void_p, _F, _F, _F, _F, _F, ctypes.c_int,
                                         ctypes.c_void_p, ctypes.c_void_p]
    L.cp4_conv2d_backward_data_f16.argtypes = [_S, ctypes.c_void_p, _F, _F, _F, _F,
                                               ctypes.c_void_p, ctypes.c_void_p]
    L.cp4_bf16_supported.argtypes = [_S, ctypes.c_int]
    L.cp4_conv2d_forward_bf16.argtypes = [_S, ctypes.c_void_p, _F, _F, _F, _F, _F, ctypes.c_int,
                                          ctypes.c_void_p, ctypes.c_void_p]
    L.cp4_conv2d_backward_data_bf16.argtypes = [_S, ctypes.c_void_p, _F, _F, _F, _F,
                                                ctypes.c_void_p, ctypes.c_void_p]
    L.cp4_bf16_backward_filter_supported.argtypes = [_S]
    L.cp4_conv2d_backward_filter_bf16.argtypes = (
        [_S, ctypes.c_void_p, ctypes.c_void_p] + [_F] * 8 +
        [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p])
    L.cp4_conv2d_backward_filter_f16.argtypes = L.cp4_conv2d_backward_filter_bf16.argtypes
    bwf = [_S] + [_F] * 10 + [ctypes.c_void_p, ctypes.c_size_t]
    L.cp4_conv2d_backward_filter.argtypes = bwf + [ctypes.c_void_p]
    L.cp4_conv2d_backward_filter_variant.argtypes = bwf + [ctypes.c_int, ctypes.c_void_p]
    L.cp4_conv2d_backward_filter_noalloc.argtypes = [_S] + [_F] * 10 + [ctypes.c_void_p]
    L.cp4_noalloc_scratch_bytes.restype = ctypes.c_size_t
    L.cp4_conv2d_backward_filter_full.argtypes = [_S, _F, _F, _F, ctypes.c_int, ctypes.c_void_p]
    timing = [ctypes.c_uint, ctypes.c_uint, ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    L.cp4_time_forward.argtypes = fwd + timing
    L.cp4_time_backward_data.argtypes = fwd + timing
    L.cp4_time_forward_sets.argtypes = [_S, ctypes.POINTER(ctypes.c_void_p),
                                        ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint,
                                        _F, _F, _F, _F] + timing
    L.cp4_time_backward_filter.argtypes = bwf + timing
    L.cp4_forward_variant_supported.argtypes = [_S, ctypes.c_int]
    L.cp4_tune_forward.argtypes = fwd + [ctypes.c_uint, ctypes.c_uint,
                                         ctypes.POINTER(ctypes.c_int),
                                         ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    L.cp4_tune_backward_data.argtypes = L.cp4_tune_forward.argtypes
    L.cp4_tune_backward_filter.argtypes = bwf + [ctypes.c_uint, ctypes.c_uint,
                                                 ctypes.POINTER(ctypes.c_int),
                                                 ctypes.POINTER(ctypes.c_float), ctypes.c_void_p]
    L.cp4_tuned_choice.argtypes = [_S, ctypes.c_int] + [ctypes.POINTER(ctypes.c_int)] * 4
    L.cp4_plan_query.argtypes = [_S, ctypes.c_int] + [ctypes.POINTER(ctypes.c_int)] * 3
    L.cp4_set_tuned_choice.argtypes = [_S] + [ctypes.c_int] * 5
    L.cp4_tuned_count.restype = ctypes.c_int
    L.cp4_tuned_entry.argtypes = [ctypes.c_int, _S] + [ctypes.POINTER(ctypes.c_int)] * 5
    L.cp4_tune_clear.restype = None
    L.cp4_backward_filter_variant_name.restype = ctypes.c_char_p
    L.cp4_backward_filter_variant_name.argtypes = [ctypes.c_int]
    L.cp4_tuned_filter_count.restype = ctypes.c_int
    L.cp4_tuned_filter_entry.argtypes = [ctypes.c_int, _S, ctypes.POINTER(ctypes.c_int)]
    L.cp4_set_tuned_filter_choice.argtypes = [_S, ctypes.c_int]
    L.cp4_device_status.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
    L.cp4_set_spin_limit.argtypes = [ctypes.c_int]
    L.cp4_set_spin_limit.restype = None
    L.cp4_set_backward_filter_tile_kernel.argtypes = [ctypes.c_int]
    L.cp4_set_backward_filter_tile_kernel.restype = None
    L.cp4_recompose.argtypes = [_S, _F, _F, _F, _F, _F, ctypes.c_void_p]
    L.cp3_expand_factors.argtypes = [_S] + [_F] * 7 + [ctypes.c_void_p]
    L.cp3_fold_gradients.argtypes = [_S] + [_F] * 6 + [ctypes.c_void_p]
    L.cp3_conv2d_forward_workspace_bytes.restype = ctypes.c_size_t
    L.cp3_conv2d_forward_workspace_bytes.argtypes = [_S]
    L.cp3_conv2d_forward.argtypes = [_S] + [_F] * 5 + [ctypes.c_void_p, ctypes.c_size_t,
                                                        ctypes.c_void_p]
    L.cp3_conv2d_backward_data.argtypes = L.cp3_conv2d_forward.argtypes
    L.cp3_conv2d_backward_filter_workspace_bytes.restype = ctypes.c_size_t
    L.cp3_conv2d_backward_filter_workspace_bytes.argtypes = [_S]
    L.cp3_conv2d_backward_filter.argtypes = [_S] + [_F] * 8 + [ctypes.c_void_p, ctypes.c_size_t,
                                                              ctypes.c_void_p]
    L.cp4_count_exceeding.argtypes = [_F, _F, ctypes.c_size_t, ctypes.c_float,
                                      ctypes.POINTER(ctypes.c_longlong), ctypes.c_void_p]
    L.cp4_random_uniform.argtypes = [_F, ctypes.c_size_t, ctypes.c_ulonglong, ctypes.c_void_p]
    L.cp4_copy_f32.argtypes = [_F, _F, ctypes.c_size_t, ctypes.c_void_p]
    L.cp4_time_copy_f32.argtypes = [_F, _F, ctypes.c_size_t] + timing
    L.cp4_device_malloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
    L.cp4_device_free.argtypes = [ctypes.c_void_p]
    L.cp4_host_malloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
    L.cp4_host_free.argtypes = [ctypes.c_void_p]
    for name in ("cp4_memcpy_h2d", "cp4_memcpy_d2h", "cp4_memcpy_d2d"):
        getattr(L, name).argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                     ctypes.c_void_p]
    L.cp4_memset_zero.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    L.cp4_stream_synchronize.argtypes = [ctypes.c_void_p]
    L.cp4_pointer_is_device.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
    L.cp4_set_device.argtypes = [ctypes.c_int]
    _lib = L
    return L


def check(status):
    if status != OK:
        L = lib()
        raise Cp4Error(status, f"{L.cp4_status_string(status).decode()}: "
                               f"{L.cp4_last_error_message().decode()}")


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous(), \
        "expected a contiguous float32 device tensor"
    return ctypes.c_void_p(t.data_ptr())


def _stream(stream):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def shape_for(x_or_dy_shape, FK, FC, FH, FW, pad):
    """tensor_shape as CP::Conv2dForward / Conv2dBackwardData derive it
    (Cuda_kernels/cp4Conv2d.cu:21-30, 55-64): N,H,W from the activation, T and
    Rank from FK, C from FC, Y from FH, X from FW."""
    N, _, H, W = x_or_dy_shape
    return Shape(N=N, H=H, W=W, pad=pad, T=FK.shape[0], C=FC.shape[0],
                 Y=FH.shape[0], X=FW.shape[0], Rank=FK.shape[1])


def conv2d_forward(x, FK, FC, FH, FW, pad=1, out=None, variant=-1, stream=None):
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert x.shape[1] == s.C and FC.shape[1] == s.Rank
    y = out if out is not None else torch.empty((s.N, s.T, s.H, s.W), device=x.device,
                                                dtype=torch.float32)
    check(lib().cp4_conv2d_forward_variant(ctypes.byref(s), _ptr(x), _ptr(FK), _ptr(FC),
                                           _ptr(FH), _ptr(FW), _ptr(y), variant,
                                           _stream(stream)))
    return y


ACTIVATIONS = {None: 0, "none": 0, "relu": 1}


def conv2d_forward_bias_act(x, FK, FC, FH, FW, bias=None, activation=None, pad=1, out=None,
                            stream=None):
    """y = act(conv(x) + bias[t]) with the epilogue fused into the stores."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert x.shape[1] == s.C and FC.shape[1] == s.Rank
    assert bias is None or tuple(bias.shape) == (s.T,)
    y = out if out is not None else torch.empty((s.N, s.T, s.H, s.W), device=x.device,
                                                dtype=torch.float32)
    check(lib().cp4_conv2d_forward_bias_act(
        ctypes.byref(s), _ptr(x), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        _ptr(bias) if bias is not None else None, ACTIVATIONS[activation], _ptr(y),
        _stream(stream)))
    return y


def geometry(s, stride=1, padding="same"):
    """cp4_geometry of a layer on shape `s`: padding "same" (the framework's rule the
    reference's layers use, test/layers.py:264-279), "valid", an int or an (h, w)
    pair of zeros on every side."""
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    g = Geometry()
    if padding == "same":
        check(lib().cp4_geometry_same(ctypes.byref(s), sh, sw, ctypes.byref(g)))
    elif padding == "valid":
        check(lib().cp4_geometry_valid(ctypes.byref(s), sh, sw, ctypes.byref(g)))
    else:
        ph, pw = (padding, padding) if isinstance(padding, int) else padding
        check(lib().cp4_geometry_symmetric(ctypes.byref(s), sh, sw, ph, pw, ctypes.byref(g)))
    return g


def conv2d_forward_ex(x, FK, FC, FH, FW, g, bias=None, activation=None, out=None, stream=None):
    """Forward with a stride / explicit padding / an output plane of its own."""
    s = shape_for(x.shape, FK, FC, FH, FW, 0)
    assert x.shape[1] == s.C and FC.shape[1] == s.Rank
    y = out if out is not None else torch.empty((s.N, s.T, g.out_h, g.out_w), device=x.device,
                                                dtype=torch.float32)
    check(lib().cp4_conv2d_forward_ex(
        ctypes.byref(s), ctypes.byref(g), _ptr(x), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        _ptr(bias) if bias is not None else None, ACTIVATIONS[activation], _ptr(y),
        _stream(stream)))
    return y


def backward_ex_workspace_bytes(s, g):
    return int(lib().cp4_conv2d_backward_ex_workspace_bytes(ctypes.byref(s), ctypes.byref(g)))


def _ex_workspace(s, g, device, workspace):
    need = backward_ex_workspace_bytes(s, g)
    if workspace is None:
        workspace = torch.empty(need + 256, device=device, dtype=torch.uint8)
        off = (-workspace.data_ptr()) % 256
        workspace = workspace[off:off + need]
    return workspace, workspace.numel() * workspace.element_size()


def conv2d_backward_data_ex(dy, x_hw, FK, FC, FH, FW, g, out=None, workspace=None, stream=None):
    """dx [N,C,H,W] of the layer with geometry g for dy [N,T,out_h,out_w]; x_hw = (H, W)."""
    N, T = dy.shape[:2]
    assert tuple(dy.shape[2:]) == (g.out_h, g.out_w) and FK.shape[0] == T
    s = Shape(N=N, H=x_hw[0], W=x_hw[1], pad=0, T=T, C=FC.shape[0], Y=FH.shape[0], X=FW.shape[0],
              Rank=FK.shape[1])
    dx = out if out is not None else torch.empty((N, s.C, s.H, s.W), device=dy.device,
                                                 dtype=torch.float32)
    ws, nbytes = _ex_workspace(s, g, dy.device, workspace)
    check(lib().cp4_conv2d_backward_data_ex(
        ctypes.byref(s), ctypes.byref(g), _ptr(dy), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW), _ptr(dx),
        ctypes.c_void_p(ws.data_ptr()), nbytes, _stream(stream)))
    return dx


def conv2d_backward_filter_ex(x, dy, FK, FC, FH, FW, g, workspace=None, stream=None):
    """(dFK, dFC, dFH, dFW) of the layer with geometry g."""
    s = shape_for(x.shape, FK, FC, FH, FW, 0)
    assert tuple(dy.shape) == (s.N, s.T, g.out_h, g.out_w) and x.shape[1] == s.C
    outs = [torch.empty_like(f) for f in (FK, FC, FH, FW)]
    ws, nbytes = _ex_workspace(s, g, x.device, workspace)
    check(lib().cp4_conv2d_backward_filter_ex(
        ctypes.byref(s), ctypes.byref(g), _ptr(x), _ptr(dy), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr()), nbytes, _stream(stream)))
    return tuple(outs)


def _ptr16(t, dtype=torch.bfloat16):
    assert t.is_cuda and t.is_contiguous() and t.dtype == dtype
    return ctypes.c_void_p(t.data_ptr())


def conv2d_forward_f16(x, FK, FC, FH, FW, bias=None, activation=None, pad=1, out=None,
                       stream=None):
    """float16 x -> float16 y = act(conv(x) + bias); fp32 factors, bias and arithmetic."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert x.shape[1] == s.C and FC.shape[1] == s.Rank
    y = out if out is not None else torch.empty((s.N, s.T, s.H, s.W), device=x.device,
                                                dtype=torch.float16)
    check(lib().cp4_conv2d_forward_f16(
        ctypes.byref(s), _ptr16(x, torch.float16), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        _ptr(bias) if bias is not None else None, ACTIVATIONS[activation],
        _ptr16(y, torch.float16), _stream(stream)))
    return y


def conv2d_backward_data_f16(dy, FK, FC, FH, FW, pad=1, out=None, stream=None):
    """float16 dy -> float16 dx; fp32 factors and arithmetic."""
    s = shape_for(dy.shape, FK, FC, FH, FW, pad)
    assert dy.shape[1] == s.T
    dx = out if out is not None else torch.empty((s.N, s.C, s.H, s.W), device=dy.device,
                                                 dtype=torch.float16)
    check(lib().cp4_conv2d_backward_data_f16(
        ctypes.byref(s), _ptr16(dy, torch.float16), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        _ptr16(dx, torch.float16), _stream(stream)))
    return dx


def _rcp_shape(act_shape, K0, K1, KC, pad):
    N, _, H, W = act_shape
    S0, T0, R = K0.shape
    S1, T1, _ = K1.shape
    assert K1.shape[2] == R and KC.shape[2] == R
    s = Shape(N=N, H=H, W=W, pad=pad, T=T0 * T1, C=S0 * S1, Y=KC.shape[0], X=KC.shape[1], Rank=R)
    return s, RcpDims(S0, S1, T0, T1)


def _rcp_workspace(s, d, device):
    n = int(lib().rcp_conv2d_workspace_bytes(ctypes.byref(s), ctypes.byref(d)))
    return torch.empty(n + 256, device=device, dtype=torch.uint8), n + 256


def rcp_conv2d_forward(x, K0, K1, KC, pad=1, out=None, stream=None):
    """Reshaped-CP op: x [N,S0*S1,H,W], K0 [S0,T0,R], K1 [S1,T1,R], KC [Y,X,R] -> [N,T0*T1,H,W]."""
    s, d = _rcp_shape(x.shape, K0, K1, KC, pad)
    assert x.shape[1] == s.C
    y = out if out is not None else torch.empty((s.N, s.T, s.H, s.W), device=x.device,
                                                dtype=torch.float32)
    ws, n = _rcp_workspace(s, d, x.device)
    check(lib().rcp_conv2d_forward(ctypes.byref(s), ctypes.byref(d), _ptr(x), _ptr(K0), _ptr(K1),
                                   _ptr(KC), _ptr(y), ctypes.c_void_p(ws.data_ptr()), n,
                                   _stream(stream)))
    return y


def rcp_conv2d_backward_data(dy, K0, K1, KC, pad=1, out=None, stream=None):
    s, d = _rcp_shape(dy.shape, K0, K1, KC, pad)
    assert dy.shape[1] == s.T
    dx = out if out is not None else torch.empty((s.N, s.C, s.H, s.W), device=dy.device,
                                                 dtype=torch.float32)
    ws, n = _rcp_workspace(s, d, dy.device)
    check(lib().rcp_conv2d_backward_data(ctypes.byref(s), ctypes.byref(d), _ptr(dy), _ptr(K0),
                                         _ptr(K1), _ptr(KC), _ptr(dx),
                                         ctypes.c_void_p(ws.data_ptr()), n, _stream(stream)))
    return dx


def rcp_conv2d_backward_filter(x, dy, K0, K1, KC, pad=1, stream=None):
    """(dK0, dK1, dKC)."""
    s, d = _rcp_shape(x.shape, K0, K1, KC, pad)
    assert tuple(dy.shape) == (s.N, s.T, s.H, s.W)
    outs = [torch.empty_like(t) for t in (K0, K1, KC)]
    ws, n = _rcp_workspace(s, d, x.device)
    check(lib().rcp_conv2d_backward_filter(
        ctypes.byref(s), ctypes.byref(d), _ptr(x), _ptr(dy), _ptr(K0), _ptr(K1), _ptr(KC),
        *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr()), n, _stream(stream)))
    return tuple(outs)


def bf16_supported(s, backward_data=False):
    return bool(lib().cp4_bf16_supported(ctypes.byref(s), int(backward_data)))


def bf16_backward_filter_supported(s):
    return bool(lib().cp4_bf16_backward_filter_supported(ctypes.byref(s)))


def conv2d_forward_bf16(x, FK, FC, FH, FW, bias=None, activation=None, pad=1, out=None,
                        stream=None):
    """bfloat16 x -> bfloat16 y = act(conv(x) + bias); fp32 factors, bias and arithmetic."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert x.shape[1] == s.C and FC.shape[1] == s.Rank
    assert bias is None or tuple(bias.shape) == (s.T,)
    y = out if out is not None else torch.empty((s.N, s.T, s.H, s.W), device=x.device,
                                                dtype=torch.bfloat16)
    check(lib().cp4_conv2d_forward_bf16(
        ctypes.byref(s), _ptr16(x), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        _ptr(bias) if bias is not None else None, ACTIVATIONS[activation], _ptr16(y),
        _stream(stream)))
    return y


def conv2d_backward_data_bf16(dy, FK, FC, FH, FW, pad=1, out=None, stream=None):
    """bfloat16 dy -> bfloat16 dx; fp32 factors and arithmetic."""
    s = shape_for(dy.shape, FK, FC, FH, FW, pad)
    assert dy.shape[1] == s.T
    dx = out if out is not None else torch.empty((s.N, s.C, s.H, s.W), device=dy.device,
                                                 dtype=torch.bfloat16)
    check(lib().cp4_conv2d_backward_data_bf16(ctypes.byref(s), _ptr16(dy), _ptr(FK), _ptr(FC),
                                              _ptr(FH), _ptr(FW), _ptr16(dx), _stream(stream)))
    return dx


def conv2d_backward_filter_bf16(x, dy, FK, FC, FH, FW, pad=1, workspace=None, stream=None):
    """bfloat16 x, dy -> fp32 (dFK, dFC, dFH, dFW); fp32 factors and arithmetic."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert tuple(dy.shape) == (s.N, s.T, s.H, s.W) and x.shape[1] == s.C
    outs = [torch.empty_like(f) for f in (FK, FC, FH, FW)]
    ws, ws_bytes = _workspace(s, x.device, workspace)
    check(lib().cp4_conv2d_backward_filter_bf16(
        ctypes.byref(s), _ptr16(x), _ptr16(dy), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr()), ws_bytes, _stream(stream)))
    return tuple(outs)


def conv2d_backward_filter_f16(x, dy, FK, FC, FH, FW, pad=1, workspace=None, stream=None):
    """float16 x, dy -> fp32 (dFK, dFC, dFH, dFW); fp32 factors and arithmetic."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert tuple(dy.shape) == (s.N, s.T, s.H, s.W) and x.shape[1] == s.C
    outs = [torch.empty_like(f) for f in (FK, FC, FH, FW)]
    ws, ws_bytes = _workspace(s, x.device, workspace)
    check(lib().cp4_conv2d_backward_filter_f16(
        ctypes.byref(s), _ptr16(x, torch.float16), _ptr16(dy, torch.float16), _ptr(FK), _ptr(FC),
        _ptr(FH), _ptr(FW), *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr()), ws_bytes,
        _stream(stream)))
    return tuple(outs)


def conv2d_backward_data(dy, FK, FC, FH, FW, pad=1, out=None, stream=None):
    s = shape_for(dy.shape, FK, FC, FH, FW, pad)
    assert dy.shape[1] == s.T
    dx = out if out is not None else torch.empty((s.N, s.C, s.H, s.W), device=dy.device,
                                                 dtype=torch.float32)
    check(lib().cp4_conv2d_backward_data(ctypes.byref(s), _ptr(dy), _ptr(FK), _ptr(FC),
                                         _ptr(FH), _ptr(FW), _ptr(dx), _stream(stream)))
    return dx


def backward_filter_workspace_bytes(s):
    return int(lib().cp4_conv2d_backward_filter_workspace_bytes(ctypes.byref(s)))


def _workspace(s, device, workspace):
    """(tensor, its size in bytes): the caller's workspace of any dtype, or a new one."""
    need = backward_filter_workspace_bytes(s)
    if workspace is None:
        workspace = torch.empty(max(need, 4) // 4 + 1, device=device, dtype=torch.float32)
    assert workspace.is_cuda and workspace.is_contiguous(), \
        "the workspace must be a contiguous device tensor"
    return workspace, workspace.numel() * workspace.element_size()


def conv2d_backward_filter(x, dy, FK, FC, FH, FW, pad=1, workspace=None, stream=None,
                           variant=-1):
    """Returns (dFK, dFC, dFH, dFW)."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert tuple(dy.shape) == (s.N, s.T, s.H, s.W) and x.shape[1] == s.C
    outs = [torch.empty_like(f) for f in (FK, FC, FH, FW)]
    ws, ws_bytes = _workspace(s, x.device, workspace)
    check(lib().cp4_conv2d_backward_filter_variant(
        ctypes.byref(s), _ptr(x), _ptr(dy), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr()), ws_bytes, variant,
        _stream(stream)))
    return tuple(outs)


def conv2d_backward_filter_noalloc(x, dy, FK, FC, FH, FW, outs, pad=1, stream=None):
    """The factor gradients into the caller's `outs` = (dFK, dFC, dFH, dFW) through the
    entry point that allocates nothing (the library's static scratch)."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    assert tuple(dy.shape) == (s.N, s.T, s.H, s.W) and x.shape[1] == s.C
    check(lib().cp4_conv2d_backward_filter_noalloc(
        ctypes.byref(s), _ptr(x), _ptr(dy), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        *[_ptr(o) for o in outs], _stream(stream)))
    return tuple(outs)


def conv2d_backward_filter_full(x, dy, Y, X, pad=1, out=None, stream=None):
    N, C, H, W = x.shape
    s = Shape(N=N, H=H, W=W, pad=pad, T=dy.shape[1], C=C, Y=Y, X=X, Rank=0)
    accumulate = out is not None
    dK = out if accumulate else torch.empty((s.T, C, Y, X), device=x.device,
                                            dtype=torch.float32)
    check(lib().cp4_conv2d_backward_filter_full(ctypes.byref(s), _ptr(x), _ptr(dy), _ptr(dK),
                                                int(accumulate), _stream(stream)))
    return dK


def time_forward(x, FK, FC, FH, FW, y, pad, warmup=1, profcount=47, stream=None):
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    us = ctypes.c_float()
    check(lib().cp4_time_forward(ctypes.byref(s), _ptr(x), _ptr(FK), _ptr(FC), _ptr(FH),
                                 _ptr(FW), _ptr(y), warmup, profcount, ctypes.byref(us),
                                 _stream(stream)))
    return us.value


def time_forward_sets(xs, FK, FC, FH, FW, ys, pad, warmup=1, profcount=47, stream=None):
    """The timed loop over several buffer sets taken in turn (launch i uses set
    i % len(xs)): with a footprint beyond the memory-side cache every launch
    streams from and to HBM."""
    assert len(xs) == len(ys) >= 1
    s = shape_for(xs[0].shape, FK, FC, FH, FW, pad)
    n = len(xs)
    xp = (ctypes.c_void_p * n)(*[_ptr(x) for x in xs])
    yp = (ctypes.c_void_p * n)(*[_ptr(y) for y in ys])
    us = ctypes.c_float()
    check(lib().cp4_time_forward_sets(ctypes.byref(s), xp, yp, n, _ptr(FK), _ptr(FC), _ptr(FH),
                                      _ptr(FW), warmup, profcount, ctypes.byref(us),
                                      _stream(stream)))
    return us.value


def time_backward_data(dy, FK, FC, FH, FW, dx, pad, warmup=1, profcount=47, stream=None):
    s = shape_for(dy.shape, FK, FC, FH, FW, pad)
    us = ctypes.c_float()
    check(lib().cp4_time_backward_data(ctypes.byref(s), _ptr(dy), _ptr(FK), _ptr(FC),
                                       _ptr(FH), _ptr(FW), _ptr(dx), warmup, profcount,
                                       ctypes.byref(us), _stream(stream)))
    return us.value


def time_backward_filter(x, dy, FK, FC, FH, FW, pad, warmup=1, profcount=47,
                         workspace=None, stream=None):
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    outs = [torch.empty_like(f) for f in (FK, FC, FH, FW)]
    ws, ws_bytes = _workspace(s, x.device, workspace)
    us = ctypes.c_float()
    check(lib().cp4_time_backward_filter(
        ctypes.byref(s), _ptr(x), _ptr(dy), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr()), ws_bytes, warmup,
        profcount, ctypes.byref(us), _stream(stream)))
    return us.value


def forward_variants(s=None):
    """[(index, name, supported-for-shape)]"""
    L = lib()
    out = []
    for v in range(L.cp4_forward_variant_count()):
        ok = None if s is None else L.cp4_forward_variant_supported(ctypes.byref(s), v) == OK
        out.append((v, L.cp4_forward_variant_name(v).decode(), ok))
    return out


def default_variant(s, backward_data=False):
    """Name of the variant the library runs for shape s unless told otherwise
    (None: no variant takes the shape)."""
    L = lib()
    v = L.cp4_forward_default_variant(ctypes.byref(s), int(backward_data))
    return L.cp4_forward_variant_name(v).decode() if v >= 0 else None


def tune_forward(x, FK, FC, FH, FW, y, pad, warmup=1, profcount=10, stream=None):
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    best, us = ctypes.c_int(-1), ctypes.c_float()
    check(lib().cp4_tune_forward(ctypes.byref(s), _ptr(x), _ptr(FK), _ptr(FC), _ptr(FH),
                                 _ptr(FW), _ptr(y), warmup, profcount, ctypes.byref(best),
                                 ctypes.byref(us), _stream(stream)))
    return best.value, us.value


def tune_backward_data(dy, FK, FC, FH, FW, dx, pad, warmup=1, profcount=10, stream=None):
    s = shape_for(dy.shape, FK, FC, FH, FW, pad)
    best, us = ctypes.c_int(-1), ctypes.c_float()
    check(lib().cp4_tune_backward_data(ctypes.byref(s), _ptr(dy), _ptr(FK), _ptr(FC), _ptr(FH),
                                       _ptr(FW), _ptr(dx), warmup, profcount,
                                       ctypes.byref(best), ctypes.byref(us), _stream(stream)))
    return best.value, us.value


def tune_backward_filter(x, dy, FK, FC, FH, FW, pad, warmup=1, profcount=10, workspace=None,
                         stream=None):
    """(best variant: 0 general / 1 matrix cores in four launches / 2 with the tap step
    inside the gradient GEMMs, its mean us)."""
    s = shape_for(x.shape, FK, FC, FH, FW, pad)
    outs = [torch.empty_like(f) for f in (FK, FC, FH, FW)]
    ws, ws_bytes = _workspace(s, x.device, workspace)
    best, us = ctypes.c_int(-1), ctypes.c_float()
    check(lib().cp4_tune_backward_filter(
        ctypes.byref(s), _ptr(x), _ptr(dy), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
        *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr()), ws_bytes, warmup, profcount,
        ctypes.byref(best), ctypes.byref(us), _stream(stream)))
    return best.value, us.value


def tuned_choice(s, backward_data=False):
    """{'variant', 'tile_rows', 'tile_cols', 'role_split'} a shape would run with now."""
    v = [ctypes.c_int() for _ in range(4)]
    check(lib().cp4_tuned_choice(ctypes.byref(s), int(backward_data), *[ctypes.byref(i) for i in v]))
    return dict(zip(("variant", "tile_rows", "tile_cols", "role_split"), (i.value for i in v)))


def plan_query(s, pass_="forward"):
    """{'variant' (its name), 'strip_rows', 'workgroups'} a launch of this pass would run with
    now; rows and workgroups are 0 unless the whole-row strip kernel takes the shape."""
    idx = ("forward", "backward_data", "backward_filter").index(pass_)
    v = [ctypes.c_int() for _ in range(3)]
    check(lib().cp4_plan_query(ctypes.byref(s), idx, *[ctypes.byref(i) for i in v]))
    if idx == 2:
        names = dict(enumerate(backward_filter_variants()))
    else:
        names = {i: n for i, n, _ in forward_variants()}
    return {"variant": names.get(v[0].value, str(v[0].value)), "strip_rows": v[1].value,
            "workgroups": v[2].value}


def set_tuned_choice(s, variant, tile_rows=0, tile_cols=0, schedule=1, backward_data=False):
    """Enters a choice into the tuner's table (tuned_choice's terms: schedule 1 = the
    kernel's rule, 0 = no role split, 2 = whole pixel groups per consumer wave)."""
    check(lib().cp4_set_tuned_choice(ctypes.byref(s), int(backward_data), int(variant),
                                     int(tile_rows), int(tile_cols), int(schedule)))


def tuned_table():
    """The forward / backward-data tuner table as a list of dicts (shape fields, pass,
    variant name, tile, schedule)."""
    L = lib()
    names = {v: n for v, n, _ in forward_variants()}
    out = []
    for i in range(L.cp4_tuned_count()):
        s = Shape()
        v = [ctypes.c_int() for _ in range(5)]
        check(L.cp4_tuned_entry(i, ctypes.byref(s), *[ctypes.byref(k) for k in v]))
        out.append({"N": s.N, "H": s.H, "W": s.W, "pad": s.pad, "T": s.T, "C": s.C, "Y": s.Y,
                    "X": s.X, "Rank": s.Rank, "backward_data": bool(v[0].value),
                    "variant": names[v[1].value], "tile_rows": v[2].value,
                    "tile_cols": v[3].value, "schedule": v[4].value})
    return out


def backward_filter_variants():
    """Names of the backward-filter variants, by number."""
    L = lib()
    out = []
    while L.cp4_backward_filter_variant_name(len(out)) is not None:
        out.append(L.cp4_backward_filter_variant_name(len(out)).decode())
    return out


def tuned_filter_table():
    """The backward-filter tuner table as a list of dicts (shape fields, variant name)."""
    L = lib()
    names = backward_filter_variants()
    out = []
    for i in range(L.cp4_tuned_filter_count()):
        s, v = Shape(), ctypes.c_int()
        check(L.cp4_tuned_filter_entry(i, ctypes.byref(s), ctypes.byref(v)))
        out.append({"N": s.N, "H": s.H, "W": s.W, "pad": s.pad, "T": s.T, "C": s.C, "Y": s.Y,
                    "X": s.X, "Rank": s.Rank, "pass": "backward_filter",
                    "variant": names[v.value]})
    return out


def set_tuned_filter_choice(s, variant):
    check(lib().cp4_set_tuned_filter_choice(ctypes.byref(s), int(variant)))


def save_tuned(path):
    """Writes the tuner tables of all three passes as JSON (variants by name, so that
    the file survives a rebuild of the library)."""
    import json
    with open(path, "w") as f:
        json.dump(tuned_table() + tuned_filter_table(), f, indent=1)


def load_tuned(path):
    """Re-enters a table written by save_tuned; entries this build does not take are
    skipped.  Returns the number entered."""
    import json
    numbers = {n: v for v, n, _ in forward_variants()}
    filter_numbers = {n: v for v, n in enumerate(backward_filter_variants())}
    done = 0
    with open(path) as f:
        entries = json.load(f)
    for e in entries:
        s = Shape(e["N"], e["H"], e["W"], e["pad"], e["T"], e["C"], e["Y"], e["X"], e["Rank"])
        if e.get("pass") == "backward_filter":
            if e["variant"] in filter_numbers:
                set_tuned_filter_choice(s, filter_numbers[e["variant"]])
                done += 1
            continue
        if e["variant"] not in numbers:
            continue
        try:
            set_tuned_choice(s, numbers[e["variant"]], e["tile_rows"], e["tile_cols"],
                             e["schedule"], backward_data=e["backward_data"])
            done += 1
        except Cp4Error:
            pass
    return done


def tune_clear():
    lib().cp4_tune_clear()


def device_status(stream=None):
    """Synchronises the stream; raises Cp4Error(ERR_DEVICE) if a kernel gave up a
    wait between its waves since the last call (the record is cleared)."""
    check(lib().cp4_device_status(_stream(stream), None))


def device_status_detail(stream=None):
    """(status, [flag, workgroup, wave, wait site]) without raising."""
    d = (ctypes.c_int * 4)()
    st = lib().cp4_device_status(_stream(stream), d)
    return st, list(d)


def set_spin_limit(polls):
    """Polls after which an in-kernel wait gives up (0: the default); fault injection."""
    lib().cp4_set_spin_limit(int(polls))


def set_backward_filter_tile_kernel(which):
    """Backward-filter variant 3: 0 the plain multiply-add tile kernel, 1 the matrix-core one
    (wherever both can run the shape), anything else the library's choice."""
    lib().cp4_set_backward_filter_tile_kernel(int(which))


def recompose(FK, FC, FH, FW, stream=None):
    s = Shape(T=FK.shape[0], C=FC.shape[0], Y=FH.shape[0], X=FW.shape[0], Rank=FK.shape[1])
    K = torch.empty((s.T, s.C, s.Y, s.X), device=FK.device, dtype=torch.float32)
    check(lib().cp4_recompose(ctypes.byref(s), _ptr(FK), _ptr(FC), _ptr(FH), _ptr(FW),
                              _ptr(K), _stream(stream)))
    return K


def cp3_shape_for(x_shape, K0, K1, K2, pad):
    """tensor_shape of the 3-factor CP op: K0 [C,R], K1 [Y,X,R], K2 [R,T]
    (Kernels/cp_fused_nchw.cc:20-24); Rank is the CP rank."""
    N, _, H, W = x_shape
    assert K1.shape[2] == K0.shape[1] == K2.shape[0]
    return Shape(N=N, H=H, W=W, pad=pad, T=K2.shape[1], C=K0.shape[0], Y=K1.shape[0],
                 X=K1.shape[1], Rank=K0.shape[1])


def cp3_expand_factors(K0, K1, K2, stream=None):
    """The CP4 factors (FK, FC, FH, FW) of rank Y*R that compute the same convolution."""
    s = cp3_shape_for((0, 0, 1, 1), K0, K1, K2, 0)
    Q = s.Y * s.Rank
    out = [torch.empty((d, Q), device=K0.device, dtype=torch.float32)
           for d in (s.T, s.C, s.Y, s.X)]
    check(lib().cp3_expand_factors(ctypes.byref(s), _ptr(K0), _ptr(K1), _ptr(K2),
                                   *[_ptr(o) for o in out], _stream(stream)))
    return tuple(out)


def cp3_fold_gradients(dFK, dFC, dFW, Y, stream=None):
    """(dK0, dK1, dK2) from the gradients of the expanded CP4 factors."""
    Q = dFK.shape[1]
    assert Q % Y == 0
    s = Shape(T=dFK.shape[0], C=dFC.shape[0], Y=Y, X=dFW.shape[0], Rank=Q // Y)
    dK0 = torch.empty((s.C, s.Rank), device=dFK.device, dtype=torch.float32)
    dK1 = torch.empty((s.Y, s.X, s.Rank), device=dFK.device, dtype=torch.float32)
    dK2 = torch.empty((s.Rank, s.T), device=dFK.device, dtype=torch.float32)
    check(lib().cp3_fold_gradients(ctypes.byref(s), _ptr(dFK), _ptr(dFC), _ptr(dFW), _ptr(dK0),
                                   _ptr(dK1), _ptr(dK2), _stream(stream)))
    return dK0, dK1, dK2


def _cp3_pass(fn, s, src, K0, K1, K2, dst, workspace, stream):
    nbytes = lib().cp3_conv2d_forward_workspace_bytes(ctypes.byref(s))
    ws = workspace if workspace is not None else torch.empty(nbytes, device=src.device,
                                                             dtype=torch.uint8)
    assert ws.numel() * ws.element_size() >= nbytes
    check(fn(ctypes.byref(s), _ptr(src), _ptr(K0), _ptr(K1), _ptr(K2), _ptr(dst),
             ctypes.c_void_p(ws.data_ptr()), nbytes, _stream(stream)))
    return dst


def cp3_conv2d_forward(x, K0, K1, K2, pad=1, out=None, workspace=None, stream=None):
    s = cp3_shape_for(x.shape, K0, K1, K2, pad)
    assert x.shape[1] == s.C
    y = out if out is not None else torch.empty((s.N, s.T, s.H, s.W), device=x.device,
                                                dtype=torch.float32)
    return _cp3_pass(lib().cp3_conv2d_forward, s, x, K0, K1, K2, y, workspace, stream)


def cp3_conv2d_backward_data(dy, K0, K1, K2, pad=1, out=None, workspace=None, stream=None):
    s = cp3_shape_for(dy.shape, K0, K1, K2, pad)
    assert dy.shape[1] == s.T
    dx = out if out is not None else torch.empty((s.N, s.C, s.H, s.W), device=dy.device,
                                                 dtype=torch.float32)
    return _cp3_pass(lib().cp3_conv2d_backward_data, s, dy, K0, K1, K2, dx, workspace, stream)


def cp3_conv2d_backward_filter(x, dy, K0, K1, K2, pad=1, stream=None):
    """(dK0 [C,R], dK1 [Y,X,R], dK2 [R,T]) of the 3-factor CP op."""
    s = cp3_shape_for(x.shape, K0, K1, K2, pad)
    assert tuple(dy.shape) == (s.N, s.T, s.H, s.W)
    outs = [torch.empty_like(t) for t in (K0, K1, K2)]
    n = int(lib().cp3_conv2d_backward_filter_workspace_bytes(ctypes.byref(s)))
    ws = torch.empty(n + 512, device=x.device, dtype=torch.uint8)
    off = (-ws.data_ptr()) % 256
    check(lib().cp3_conv2d_backward_filter(
        ctypes.byref(s), _ptr(x), _ptr(dy), _ptr(K0), _ptr(K1), _ptr(K2),
        *[_ptr(o) for o in outs], ctypes.c_void_p(ws.data_ptr() + off), n, _stream(stream)))
    return tuple(outs)


def count_exceeding(a, b, tol, stream=None):
    assert a.numel() == b.numel()
    n = ctypes.c_longlong()
    check(lib().cp4_count_exceeding(_ptr(a), _ptr(b), a.numel(), tol, ctypes.byref(n),
                                    _stream(stream)))
    return n.value


def random_uniform(shape, seed, device="cuda", stream=None):
    t = torch.empty(shape, device=device, dtype=torch.float32)
    check(lib().cp4_random_uniform(_ptr(t), t.numel(), seed, _stream(stream)))
    return t


def time_copy(dst, src, warmup=1, profcount=47, stream=None):
    us = ctypes.c_float()
    check(lib().cp4_time_copy_f32(_ptr(dst), _ptr(src), src.numel(), warmup, profcount,
                                  ctypes.byref(us), _stream(stream)))
    return us.value
