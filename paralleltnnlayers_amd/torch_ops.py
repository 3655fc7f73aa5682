"""PyTorch autograd binding of the fused CP4 Conv2d C ABI.

Stands where the reference registers its TensorFlow custom op
(Kernels/cp4_conv_nchw.cc:6-108, ``Cp4Conv2dNchw``: input + four factor
tensors -> output, NCHW): a ``torch.autograd.Function`` whose forward, input
gradient and factor gradients are the three passes of ``libcp4conv.so``.
PyTorch only owns the tensors and the stream; all arithmetic is in the HIP
library, and there is no eager fallback.

Factor layout is the C ABI's: FK [T,R], FC [C,R], FH [Y,R], FW [X,R].
For "same" padding at stride 1 (2*pad = Y-1 = X-1) the reference's three passes
run as they are; that is the only case in which its backward-data formula
(flipped taps at offset +y-pad, Cuda_kernels/cp4Conv2dBackwardData.cu:79-87) is
the adjoint of its forward.  Strides and every other padding go through the
library's geometry entry points (cp4_conv2d_forward_ex and its exact gradients).

Launches are asynchronous.  A producer / consumer kernel whose wait between waves
runs out ends early and leaves its output incomplete; the library records that per
device and reports it from ``cp4_device_status``, which synchronises the stream.
``check_device()`` is that call: use it wherever the training loop synchronises
anyway (reading the loss, a checkpoint).  ``set_device_checks(True)`` - or the
environment variable ``CP4_CHECK_DEVICE=1`` - makes every backward pass of the
Functions below end with it, at the price of one synchronisation per layer and step.
"""
import os

import torch

from . import capi

_check_every_backward = os.environ.get("CP4_CHECK_DEVICE", "0") not in ("", "0")


def set_device_checks(on):
    """Check the device's fault record at the end of every backward pass (synchronises)."""
    global _check_every_backward
    _check_every_backward = bool(on)


def check_device(stream=None):
    """Synchronises ``stream`` and raises ``capi.Cp4Error`` (ERR_DEVICE) if a kernel of
    the library gave up a wait since the last check: outputs computed since then are
    incomplete.  The record is cleared."""
    capi.device_status(stream)


def _after_backward():
    if _check_every_backward:
        capi.device_status()


class CP4Conv2dFunction(torch.autograd.Function):
    """y = act(cp4conv2d(x, FK, FC, FH, FW, pad) + bias).

    A bfloat16 ``x`` selects the library's bfloat16-activation entry points
    (y and the input gradient are bfloat16 then; factors, bias and their
    gradients stay float32); shapes those do not take are widened to float32.
    """

    @staticmethod
    def forward(ctx, x, FK, FC, FH, FW, pad, bias=None, activation=None):
        if 2 * pad + 1 != FH.shape[0] or 2 * pad + 1 != FW.shape[0]:
            raise ValueError("autograd binding needs 2*pad = Y-1 = X-1 (the reference's "
                             "backward-data pass is the adjoint only then)")
        FK, FC, FH, FW = (t.contiguous().float() for t in (FK, FC, FH, FW))
        if bias is not None:
            bias = bias.contiguous().float()
        s = capi.shape_for(x.shape, FK, FC, FH, FW, pad)
        ctx.half = x.dtype == torch.float16
        if ctx.half:
            # half-precision activations: all three passes on the library's float16 entry
            # points where they take the shape, else on widened copies
            x = x.contiguous()
            ctx.pad, ctx.bf16, ctx.shape = pad, False, s
            ctx.relu = capi.ACTIVATIONS[activation] == 1
            if capi.bf16_supported(s):
                y = capi.conv2d_forward_f16(x, FK, FC, FH, FW, bias, activation, pad=pad)
            else:
                y = capi.conv2d_forward_bias_act(x.float(), FK, FC, FH, FW, bias, activation,
                                                 pad=pad).half()
            ctx.save_for_backward(x, FK, FC, FH, FW, y if ctx.relu else None)
            return y
        ctx.bf16 = x.dtype == torch.bfloat16
        ctx.fwd16 = ctx.bf16 and capi.bf16_supported(s)
        x = x.contiguous() if ctx.bf16 else x.contiguous().float()
        ctx.pad = pad
        if ctx.fwd16:
            y = capi.conv2d_forward_bf16(x, FK, FC, FH, FW, bias, activation, pad=pad)
        else:
            y = capi.conv2d_forward_bias_act(x.float(), FK, FC, FH, FW, bias, activation, pad=pad)
            if ctx.bf16:
                y = y.to(torch.bfloat16)
        ctx.relu = capi.ACTIVATIONS[activation] == 1
        ctx.shape = s
        ctx.save_for_backward(x, FK, FC, FH, FW, y if ctx.relu else None)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, FK, FC, FH, FW, y = ctx.saved_tensors
        s = ctx.shape
        dy = dy.contiguous()
        if ctx.relu:
            dy = dy * (y > 0)
        dbias = dy.float().sum(dim=(0, 2, 3)) if ctx.needs_input_grad[6] else None
        dy16 = ctx.bf16 and dy.dtype == torch.bfloat16
        dx = None
        if ctx.half:
            if ctx.needs_input_grad[0]:
                if dy.dtype == torch.float16 and capi.bf16_supported(s, backward_data=True):
                    dx = capi.conv2d_backward_data_f16(dy, FK, FC, FH, FW, pad=ctx.pad)
                else:
                    dx = capi.conv2d_backward_data(dy.float(), FK, FC, FH, FW, pad=ctx.pad).half()
            grads = (None, None, None, None)
            if any(ctx.needs_input_grad[1:5]):
                if dy.dtype == torch.float16 and capi.bf16_backward_filter_supported(s):
                    grads = capi.conv2d_backward_filter_f16(x, dy, FK, FC, FH, FW, pad=ctx.pad)
                else:
                    grads = capi.conv2d_backward_filter(x.float(), dy.float(), FK, FC, FH, FW,
                                                        pad=ctx.pad)
                grads = tuple(g if need else None
                              for g, need in zip(grads, ctx.needs_input_grad[1:5]))
            _after_backward()
            return (dx,) + grads + (None, dbias, None)
        if ctx.needs_input_grad[0]:
            if dy16 and capi.bf16_supported(s, backward_data=True):
                dx = capi.conv2d_backward_data_bf16(dy, FK, FC, FH, FW, pad=ctx.pad)
            else:
                dx = capi.conv2d_backward_data(dy.float(), FK, FC, FH, FW, pad=ctx.pad)
                if ctx.bf16:
                    dx = dx.to(torch.bfloat16)
        grads = (None, None, None, None)
        if any(ctx.needs_input_grad[1:5]):
            if dy16 and capi.bf16_backward_filter_supported(s):
                grads = capi.conv2d_backward_filter_bf16(x, dy, FK, FC, FH, FW, pad=ctx.pad)
            else:
                grads = capi.conv2d_backward_filter(x.float(), dy.float(), FK, FC, FH, FW,
                                                    pad=ctx.pad)
            grads = tuple(g if need else None
                          for g, need in zip(grads, ctx.needs_input_grad[1:5]))
        _after_backward()
        return (dx,) + grads + (None, dbias, None)


class CP4Conv2dGeometryFunction(torch.autograd.Function):
    """The layer with a stride, explicit padding or an output plane of its own
    (cp4_conv2d_forward_ex and its two gradients; float32)."""

    @staticmethod
    def forward(ctx, x, FK, FC, FH, FW, geom, bias=None, activation=None):
        x, FK, FC, FH, FW = (t.contiguous().float() for t in (x, FK, FC, FH, FW))
        if bias is not None:
            bias = bias.contiguous().float()
        y = capi.conv2d_forward_ex(x, FK, FC, FH, FW, geom, bias, activation)
        ctx.geom = geom
        ctx.relu = capi.ACTIVATIONS[activation] == 1
        ctx.save_for_backward(x, FK, FC, FH, FW, y if ctx.relu else None)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, FK, FC, FH, FW, y = ctx.saved_tensors
        dy = dy.contiguous().float()
        if ctx.relu:
            dy = dy * (y > 0)
        dbias = dy.sum(dim=(0, 2, 3)) if ctx.needs_input_grad[6] else None
        dx = None
        if ctx.needs_input_grad[0]:
            dx = capi.conv2d_backward_data_ex(dy, x.shape[2:], FK, FC, FH, FW, ctx.geom)
        grads = (None, None, None, None)
        if any(ctx.needs_input_grad[1:5]):
            grads = capi.conv2d_backward_filter_ex(x, dy, FK, FC, FH, FW, ctx.geom)
            grads = tuple(g if need else None
                          for g, need in zip(grads, ctx.needs_input_grad[1:5]))
        _after_backward()
        return (dx,) + grads + (None, dbias, None)


def cp4_conv2d(x, FK, FC, FH, FW, pad, bias=None, activation=None, stride=1, padding=None):
    """Functional form: differentiable fused CP4 convolution (NCHW), with the
    optional bias [T] and activation ("relu") fused into the forward stores.

    ``pad`` zeros on every side, stride 1 and 2*pad = Y - 1 is the reference's own
    layer and runs its three passes (bfloat16 activations included).  A ``stride``,
    ``padding`` = "same" (the framework's rule of the reference's Python layers,
    test/layers.py:264-279: out = ceil(in / stride), on even sizes one more zero
    after the image than before it), "valid", an int or an (h, w) pair run the
    strided kernels: only the kept outputs are computed.
    """
    if padding is None:
        padding = pad
    y_taps, x_taps = FH.shape[0], FW.shape[0]
    plain = stride == 1 and (
        (isinstance(padding, int) and 2 * padding + 1 == y_taps == x_taps) or
        (padding == "same" and y_taps == x_taps and y_taps % 2 == 1))
    if plain:
        return CP4Conv2dFunction.apply(x, FK, FC, FH, FW, y_taps // 2, bias, activation)
    s = capi.shape_for(x.shape, FK, FC, FH, FW, 0)
    geom = capi.geometry(s, stride, padding)
    return CP4Conv2dGeometryFunction.apply(x, FK, FC, FH, FW, geom, bias, activation)


class CP4Conv2d(torch.nn.Module):
    """A rank-R CP4-decomposed convolution layer, "same" padding.

    Equivalent dense filter: K[t,c,y,x] = sum_r FK[t,r] FC[c,r] FH[y,r] FW[x,r]
    (Cuda_kernels/Utils.cu:55-62).  Factors start as normal(0, s) with s chosen
    so that the recomposed filter has the variance of a Kaiming-normal dense
    filter of the same shape.
    """

    def __init__(self, in_channels, out_channels, kernel_size, rank, device="cuda", bias=False,
                 activation=None, stride=1, padding=None):
        super().__init__()
        if kernel_size % 2 != 1 and padding is None:
            raise ValueError("kernel_size must be odd for the default padding")
        self.pad = kernel_size // 2
        self.padding = padding
        fan_in = in_channels * kernel_size * kernel_size
        # Var[K] = R * s^8 for four independent N(0, s^2) factors; target 2 / fan_in
        s = (2.0 / (fan_in * rank)) ** 0.125
        mk = lambda d: torch.nn.Parameter(torch.randn(d, rank, device=device) * s)
        self.FK, self.FC = mk(out_channels), mk(in_channels)
        self.FH, self.FW = mk(kernel_size), mk(kernel_size)
        self.bias = torch.nn.Parameter(torch.zeros(out_channels, device=device)) if bias else None
        self.activation = activation
        self.stride = stride

    def forward(self, x):
        return cp4_conv2d(x, self.FK, self.FC, self.FH, self.FW, self.pad, self.bias,
                          self.activation, self.stride, self.padding)

    @staticmethod
    def check_device(stream=None):
        """See ``check_device``: call where the loop synchronises anyway."""
        check_device(stream)

    def dense_filter(self):
        """The recomposed [T,C,Y,X] filter (on the device, through cp4_recompose)."""
        return capi.recompose(self.FK.detach(), self.FC.detach(), self.FH.detach(),
                              self.FW.detach())


class CP3Conv2dFunction(torch.autograd.Function):
    """The 3-factor CP convolution of the reference's ``Conv2dCpFusedNchw`` op
    (Kernels/cp_fused_nchw.cc:6-30; its Python definition is pointwise K0,
    depthwise K1, pointwise K2, test/layers.py:265-282):

        y[n,t] = sum_r K2[r,t] * (K1[:,:,r] (*) sum_c K0[c,r] x[n,c])

    K0 [C,R], K1 [Y,X,R], K2 [R,T].  All three passes are the library's cp3 entry
    points.
    """

    @staticmethod
    def forward(ctx, x, K0, K1, K2, pad):
        if 2 * pad + 1 != K1.shape[0] or 2 * pad + 1 != K1.shape[1]:
            raise ValueError("autograd binding needs 2*pad = Y-1 = X-1")
        K0, K1, K2 = (t.contiguous().float() for t in (K0, K1, K2))
        x = x.contiguous().float()
        ctx.pad = pad
        ctx.save_for_backward(x, K0, K1, K2)
        return capi.cp3_conv2d_forward(x, K0, K1, K2, pad=pad)

    @staticmethod
    def backward(ctx, dy):
        x, K0, K1, K2 = ctx.saved_tensors
        dy = dy.contiguous().float()
        dx = None
        if ctx.needs_input_grad[0]:
            dx = capi.cp3_conv2d_backward_data(dy, K0, K1, K2, pad=ctx.pad)
        grads = (None, None, None)
        if any(ctx.needs_input_grad[1:4]):
            grads = capi.cp3_conv2d_backward_filter(x, dy, K0, K1, K2, pad=ctx.pad)
            grads = tuple(g if need else None for g, need in zip(grads, ctx.needs_input_grad[1:4]))
        _after_backward()
        return (dx,) + grads + (None,)


def cp3_conv2d(x, K0, K1, K2, pad):
    """Functional form of the differentiable 3-factor CP convolution (NCHW)."""
    return CP3Conv2dFunction.apply(x, K0, K1, K2, pad)


class CP3Conv2d(torch.nn.Module):
    """A rank-R 3-factor CP convolution layer, "same" padding: pointwise K0 [C,R],
    depthwise K1 [k,k,R], pointwise K2 [R,T] (the kernels of the reference's Python
    layer, test/layers.py:285-294, in the fused op's layouts).  Factors start as
    normal(0, s) with s chosen so that the equivalent dense filter
    sum_r K0[c,r] K1[i,j,r] K2[r,t] has the variance of a Kaiming-normal one."""

    def __init__(self, in_channels, out_channels, kernel_size, rank, device="cuda"):
        super().__init__()
        if kernel_size % 2 != 1:
            raise ValueError("kernel_size must be odd (same padding)")
        self.pad = kernel_size // 2
        fan_in = in_channels * kernel_size * kernel_size
        # Var = R * s^6 for three independent N(0, s^2) factors; target 2 / fan_in
        s = (2.0 / (fan_in * rank)) ** (1.0 / 6.0)
        mk = lambda *d: torch.nn.Parameter(torch.randn(*d, device=device) * s)
        self.K0 = mk(in_channels, rank)
        self.K1 = mk(kernel_size, kernel_size, rank)
        self.K2 = mk(rank, out_channels)

    def forward(self, x):
        return cp3_conv2d(x, self.K0, self.K1, self.K2, self.pad)


class RCPConv2dFunction(torch.autograd.Function):
    """The reshaped-CP convolution of the reference's ``Conv2dRcpFusedNchw`` op
    (Kernels/rcp_fused_nchw.cc:6-12; test/test_conv2d_rcp.py:38-41):

        y[n,(x,y)] = sum_r sum_{a,b} K0[a,x,r] K1[b,y,r] * (KC[:,:,r] (*) x[n,(a,b)])

    K0 [S0,T0,R], K1 [S1,T1,R], KC [Y,X,R]; x has S0*S1 channels, y T0*T1.  All three
    passes are the library's rcp entry points."""

    @staticmethod
    def forward(ctx, x, K0, K1, KC, pad):
        if 2 * pad + 1 != KC.shape[0] or 2 * pad + 1 != KC.shape[1]:
            raise ValueError("autograd binding needs 2*pad = Y-1 = X-1")
        K0, K1, KC = (t.contiguous().float() for t in (K0, K1, KC))
        x = x.contiguous().float()
        ctx.pad = pad
        ctx.save_for_backward(x, K0, K1, KC)
        return capi.rcp_conv2d_forward(x, K0, K1, KC, pad=pad)

    @staticmethod
    def backward(ctx, dy):
        x, K0, K1, KC = ctx.saved_tensors
        dy = dy.contiguous().float()
        dx = None
        if ctx.needs_input_grad[0]:
            dx = capi.rcp_conv2d_backward_data(dy, K0, K1, KC, pad=ctx.pad)
        grads = (None, None, None)
        if any(ctx.needs_input_grad[1:4]):
            grads = capi.rcp_conv2d_backward_filter(x, dy, K0, K1, KC, pad=ctx.pad)
            grads = tuple(g if need else None for g, need in zip(grads, ctx.needs_input_grad[1:4]))
        _after_backward()
        return (dx,) + grads + (None,)


def rcp_conv2d(x, K0, K1, KC, pad):
    """Functional form of the differentiable reshaped-CP convolution (NCHW)."""
    return RCPConv2dFunction.apply(x, K0, K1, KC, pad)
