"""Grouped (depthwise) causal conv1d + activation: ``GroupedConv1dNKI`` / ``nki_conv1d`` /
``ConvNKI`` with the reference's signatures (``mamba2/conv1d_grouped.py:265-334``), computed by
the gfx950 HIP kernels.

Layout: the reference module takes (B, C, L) (``:300-306``); the mixer's fused path uses the
sequence-major (B, L, C) layout (``:66-125``).  Both are supported here: ``channels_last=False``
(default, reference layout) or ``True``.  weight is (C, 1, k), bias (C) or None.
"""
from typing import Union

import torch
import torch.nn as nn

from . import _lib
from ._lib import Conv1dParams, ptr


def _blc_strides(t, channels_last):
    # returns (stride_b, stride_l, stride_c)
    return (t.stride(0), t.stride(1), t.stride(2)) if channels_last else (t.stride(0), t.stride(2), t.stride(1))


def _dims(t, channels_last):
    b, d1, d2 = t.shape
    return (b, d1, d2) if channels_last else (b, d2, d1)     # (b, l, C)


def _activation_code(activation):
    if activation not in _lib.ACT:
        raise ValueError(f"Invalid activation {activation}")
    return _lib.ACT[activation]


def _check(input, weight, bias):
    if input.dim() != 3 or weight.dim() != 3 or weight.shape[1] != 1:
        raise ValueError("expected input (B, C, L) or (B, L, C) and weight (C, 1, k)")
    if bias is not None and (bias.shape != (weight.shape[0],) or bias.dtype != weight.dtype):
        raise ValueError("bias must have shape (C,) and the dtype of weight")
    _lib.require_gpu(input, weight, bias)


def conv1d_forward(input, weight, bias=None, activation=None, channels_last=False, out=None):
    _check(input, weight, bias)
    lib = _lib.load()
    b, l, Cc = _dims(input, channels_last)
    if weight.shape[0] != Cc:
        raise ValueError(f"weight has {weight.shape[0]} channels, input has {Cc}")
    w = weight.detach().contiguous()
    bi = bias.detach().contiguous() if bias is not None else None
    y = out if out is not None else torch.empty_like(input, memory_format=torch.contiguous_format)
    p = Conv1dParams()
    p.x, p.w, p.bias, p.y = ptr(input), ptr(w), ptr(bi), ptr(y)
    p.batch, p.seqlen, p.channels, p.k = b, l, Cc, weight.shape[2]
    p.x_stride_b, p.x_stride_l, p.x_stride_c = _blc_strides(input, channels_last)
    p.y_stride_b, p.y_stride_l, p.y_stride_c = _blc_strides(y, channels_last)
    p.dtype, p.param_dtype, p.activation = _lib.dtype_code(input.dtype), _lib.dtype_code(w.dtype), _activation_code(activation)
    with torch.cuda.device(input.device):
        _lib.check(lib.m2_conv1d_fwd(p, _lib.stream_ptr(input.device)), "m2_conv1d_fwd")
    return y


def conv1d_backward(input, weight, bias, d_output, activation=None, channels_last=False, out_dx=None):
    _check(input, weight, bias)
    lib = _lib.load()
    b, l, Cc = _dims(input, channels_last)
    k = weight.shape[2]
    w = weight.detach().contiguous()
    bi = bias.detach().contiguous() if bias is not None else None
    if d_output.dtype != input.dtype:
        d_output = d_output.to(input.dtype)
    dx = out_dx if out_dx is not None else torch.empty_like(input, memory_format=torch.contiguous_format)
    dw = torch.empty_like(w)
    db = torch.empty_like(bi) if bi is not None else None
    nbytes = lib.m2_conv1d_bwd_workspace_bytes(b, l, Cc, k)
    ws = _lib.Workspace.get(nbytes, input.device)
    p = Conv1dParams()
    p.x, p.w, p.bias, p.dy, p.dx, p.dw, p.db = ptr(input), ptr(w), ptr(bi), ptr(d_output), ptr(dx), ptr(dw), ptr(db)
    p.workspace, p.workspace_bytes = ptr(ws), ws.numel()
    p.batch, p.seqlen, p.channels, p.k = b, l, Cc, k
    p.x_stride_b, p.x_stride_l, p.x_stride_c = _blc_strides(input, channels_last)
    p.y_stride_b, p.y_stride_l, p.y_stride_c = _blc_strides(d_output, channels_last)
    p.dx_stride_b, p.dx_stride_l, p.dx_stride_c = _blc_strides(dx, channels_last)
    p.dtype, p.param_dtype, p.activation = _lib.dtype_code(input.dtype), _lib.dtype_code(w.dtype), _activation_code(activation)
    with torch.cuda.device(input.device):
        _lib.check(lib.m2_conv1d_bwd(p, _lib.stream_ptr(input.device)), "m2_conv1d_bwd")
    return dx, dw.view_as(weight), db


class GroupedConv1dNKI(torch.autograd.Function):
    """forward(ctx, input, weight, bias, activation=None) -> output;
    backward -> (dinput, dweight, dbias, None)   (``conv1d_grouped.py:267,279,288``)."""

    @staticmethod
    def forward(ctx, input, weight, bias, activation=None, channels_last=False):
        output = conv1d_forward(input, weight, bias, activation, channels_last)
        ctx.save_for_backward(input, weight, bias)
        ctx.activation = activation
        ctx.channels_last = channels_last
        return output

    @staticmethod
    def backward(ctx, d_output):
        input, weight, bias = ctx.saved_tensors
        dinput, dweight, dbias = conv1d_backward(input, weight, bias, d_output, ctx.activation, ctx.channels_last)
        return dinput, dweight, dbias, None, None


def nki_conv1d(input, weight, bias=None, activation=None, channels_last=False):
    return GroupedConv1dNKI.apply(input, weight, bias, activation, channels_last)


class ConvNKI(nn.Conv1d):
    """Depthwise causal conv layer equivalent to ``nn.Conv1d(C, C, k, groups=C, padding=k-1)(x)[..., :L]``
    followed by ``activation``.  input (B, C, L), weight (C, 1, k), bias (C)  (``conv1d_grouped.py:295-334``).
    The tensor-parallel slicing of the reference (``:323-331``) is the identity on one GPU."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size: int, stride: int = 1,
                 padding: Union[str, int] = 0, dilation: int = 1, groups: int = 1, bias: bool = True,
                 padding_mode: str = 'zeros', device=None, dtype=None, activation=None) -> None:
        assert groups == in_channels, "grouped conv kernel only supports groups == in_channels"
        assert padding == kernel_size - 1
        assert padding_mode == 'zeros'
        assert dilation == 1
        assert stride == 1
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias, padding_mode,
                         device, dtype)
        self.activation = activation

    def forward(self, input):
        return GroupedConv1dNKI.apply(input, self.weight, self.bias, self.activation, False)
