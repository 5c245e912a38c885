"""Mixer core ``zxBCdt -> norm_out`` with the reference's signatures (``mamba2/fused_kernel.py:423-487``):

    mamba2_fused_kernel(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias, norm_weight,
                        n_groups, ssm_state_size, intermediate_size, head_dim) -> norm_out[b,l,d_inner]

Pipeline (``fused_kernel.py:252-282``): split [z | xBC | dt] -> depthwise conv + SiLU ->
softplus(dt + dt_bias) -> SSD scan -> gated RMSNorm per group (eps 1e-5).  Here that is three kernel
stages: conv, scan (softplus applied where the scan builds its decay tables, its gradient and d_dt_bias
formed where the scan writes ddt), norm.

Every stage is a HIP kernel.  The split is never materialised: the kernels take strided views of ``zxBCdt`` (the conv reads
the xBC columns in place; the scan reads x, B, C as views of the conv output), and in the backward
the scan writes dx, dB, dC straight into one packed buffer and the conv writes its dx straight into
the xBC columns of ``d_zxBCdt``.  ``Mamba2FusedKernel`` saves only its inputs and recomputes conv,
softplus and scan in the backward (as the reference does, ``:352-367``); ``...WithCaching`` keeps the
intermediates (``:449-471``).

``mamba2_fused_prefill`` is the inference form of the same pipeline that also hands the sequence over to the
decode step: it leaves the SSM state after the last token and the last W conv inputs in the caller's cache
tensors, and continues from them when the cache already holds a prefix.  The reference has no such path
(``mamba2_mixer.py:220``: "cache not supported yet"); the layouts are those its ``step`` reads (``:270-276``).
"""
import torch

from . import glue
from .conv1d_grouped import conv1d_backward, conv1d_forward
from .mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward

NORM_EPS = 1e-5     # fixed in the reference's fused kernel (fused_kernel.py:254)


def _views(zxBCdt, n_groups, d_state, d_inner, d_head):
    b, l, width = zxBCdt.shape
    h = d_inner // d_head
    d_conv = d_inner + 2 * n_groups * d_state
    if width != d_inner + d_conv + h:
        raise ValueError(f"zxBCdt width {width} != 2*d_inner + 2*g*n + h = {d_inner + d_conv + h}")
    z = zxBCdt[..., :d_inner]
    xBC = zxBCdt[..., d_inner:d_inner + d_conv]
    dt = zxBCdt[..., d_inner + d_conv:]
    return z, xBC, dt, h, d_conv


def _empty_rows_128(like):
    """An uninitialised (b, l, width) tensor like ``like`` whose row pitch is a whole number of 128-byte cache lines (the
    width itself when it already is one: 18560 columns of the 7B layer; 10576 columns of bf16 are 165.25 lines, and every
    wave-wide access to a column slice of such a buffer straddles two lines in three rows out of four).  The padded form is
    a column slice of a wider allocation: consumers that take a leading dimension (the projection's backward GEMM) read
    it in place."""
    b, l, width = like.shape
    per_line = 128 // like.element_size()
    pitch = -(-width // per_line) * per_line
    if pitch == width:
        return torch.empty((b, l, width), dtype=like.dtype, device=like.device)
    return torch.empty((b, l, pitch), dtype=like.dtype, device=like.device)[..., :width]


def _xbc_views(conv_out, n_groups, d_state, d_inner, d_head):
    h = d_inner // d_head
    gn = n_groups * d_state
    x = conv_out[..., :d_inner].unflatten(-1, (h, d_head))
    Bm = conv_out[..., d_inner:d_inner + gn].unflatten(-1, (n_groups, d_state))
    Cm = conv_out[..., d_inner + gn:].unflatten(-1, (n_groups, d_state))
    return x, Bm, Cm


def _forward_parts(zxBCdt, logA, D, conv_w, conv_b, dt_bias, norm_w, n_groups, d_state, d_inner, d_head, keep_states=False):
    z, xBC, dt, h, d_conv = _views(zxBCdt, n_groups, d_state, d_inner, d_head)
    b, l, _ = zxBCdt.shape
    conv_out = torch.empty((b, l, d_conv), dtype=zxBCdt.dtype, device=zxBCdt.device)
    conv1d_forward(xBC, conv_w, conv_b, "silu", channels_last=True, out=conv_out)
    x, Bm, Cm = _xbc_views(conv_out, n_groups, d_state, d_inner, d_head)
    # the scan's chunk states are kept for the backward when one follows directly (no second recompute there)
    states = alloc_chunk_states(dt, logA, x, Bm, Cm) if (keep_states and x.numel() > 0) else None
    # softplus(dt + dt_bias) is applied inside the scan, on the dt columns of zxBCdt where they lie
    y, _ = ssd_forward(dt, logA, x, Bm, Cm, D, chunk_states=states, dt_bias=dt_bias)
    scan_out = y.view(b, l, d_inner)
    norm_out = glue.rmsnorm_gated_hip(scan_out, z, norm_w, n_groups, NORM_EPS, out_dtype=zxBCdt.dtype)
    return norm_out, conv_out, scan_out, states


def _backward_parts(d_output, zxBCdt, logA, D, conv_w, conv_b, dt_bias, norm_w, conv_out, scan_out, states,
                    n_groups, d_state, d_inner, d_head):
    z, xBC, dt, h, d_conv = _views(zxBCdt, n_groups, d_state, d_inner, d_head)
    b, l, width = zxBCdt.shape
    d_zxBCdt = _empty_rows_128(zxBCdt)
    dz_view = d_zxBCdt[..., :d_inner]
    dxBC_view = d_zxBCdt[..., d_inner:d_inner + d_conv]
    ddt_view = d_zxBCdt[..., d_inner + d_conv:]
    # gated RMSNorm backward: d_scan_out, d_z (written into d_zxBCdt), d_norm_weight
    d_scan_out, d_norm_w, _ = glue.rmsnorm_gated_bwd_hip(scan_out, z, norm_w, d_output, n_groups, NORM_EPS, out_dz=dz_view)
    # SSD backward, gradients of x, B, C written into one packed [dx | dB | dC] buffer
    x, Bm, Cm = _xbc_views(conv_out, n_groups, d_state, d_inner, d_head)
    d_conv_out = torch.empty_like(conv_out)
    dx_v, dB_v, dC_v = _xbc_views(d_conv_out, n_groups, d_state, d_inner, d_head)
    # (the gradient of the raw dt goes straight into the dt columns of d_zxBCdt, d_dt_bias comes back summed)
    _, d_logA, _, _, _, d_D, _, d_dt_bias = ssd_backward(dt, logA, x, Bm, Cm, D, d_scan_out.view(b, l, h, d_head),
                                                         out_dX=dx_v, out_dB=dB_v, out_dC=dC_v, chunk_states=states,
                                                         dt_bias=dt_bias, out_ddt=ddt_view)
    # conv backward (into the xBC columns)
    _, d_conv_w, d_conv_b = conv1d_backward(xBC, conv_w, conv_b, d_conv_out, "silu", channels_last=True, out_dx=dxBC_view)
    return (d_zxBCdt, d_logA.to(logA.dtype), d_D.to(D.dtype) if D is not None else None, d_conv_w, d_conv_b,
            d_dt_bias.to(dt_bias.dtype), d_norm_w.to(norm_w.dtype))


class Mamba2FusedKernel(torch.autograd.Function):
    @staticmethod
    def forward(ctx, zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias,
                norm_weight, n_groups, ssm_state_size, intermediate_size, head_dim):
        norm_out, *_ = _forward_parts(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias, norm_weight,
                                      n_groups, ssm_state_size, intermediate_size, head_dim)
        ctx.dims = (n_groups, ssm_state_size, intermediate_size, head_dim)
        ctx.save_for_backward(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias, norm_weight)
        return norm_out

    @staticmethod
    def backward(ctx, d_output):
        zxBCdt, logA, D, conv_w, conv_b, dt_bias, norm_w = ctx.saved_tensors
        # recompute conv, softplus and scan (only the inputs were saved)
        _, conv_out, scan_out, states = _forward_parts(zxBCdt, logA, D, conv_w, conv_b, dt_bias, norm_w, *ctx.dims, keep_states=True)
        grads = _backward_parts(d_output, zxBCdt, logA, D, conv_w, conv_b, dt_bias, norm_w, conv_out, scan_out, states, *ctx.dims)
        return (*grads, None, None, None, None)


class Mamba2FusedKernelWithCaching(torch.autograd.Function):
    @staticmethod
    def forward(ctx, zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias,
                norm_weight, n_groups, ssm_state_size, intermediate_size, head_dim):
        norm_out, conv_out, scan_out, states = _forward_parts(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias,
                                                              norm_weight, n_groups, ssm_state_size, intermediate_size,
                                                              head_dim, keep_states=True)
        ctx.dims = (n_groups, ssm_state_size, intermediate_size, head_dim)
        ctx.chunk_states = states
        ctx.save_for_backward(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias, norm_weight, conv_out, scan_out)
        return norm_out

    @staticmethod
    def backward(ctx, d_output):
        zxBCdt, logA, D, conv_w, conv_b, dt_bias, norm_w, conv_out, scan_out = ctx.saved_tensors
        grads = _backward_parts(d_output, zxBCdt, logA, D, conv_w, conv_b, dt_bias, norm_w, conv_out, scan_out,
                                ctx.chunk_states, *ctx.dims)
        return (*grads, None, None, None, None)


def mamba2_fused_kernel(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias,
                        norm_weight, n_groups, ssm_state_size, intermediate_size,
                        head_dim):
    return Mamba2FusedKernel.apply(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias,
                                   norm_weight, n_groups, ssm_state_size, intermediate_size,
                                   head_dim)


def mamba2_fused_kernel_with_caching(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias,
                                     norm_weight, n_groups, ssm_state_size, intermediate_size,
                                     head_dim):
    return Mamba2FusedKernelWithCaching.apply(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias,
                                              norm_weight, n_groups, ssm_state_size, intermediate_size,
                                              head_dim)


def mamba2_fused_prefill(zxBCdt, logA, D, conv1d_weight, conv1d_bias, dt_bias, norm_weight, n_groups, ssm_state_size,
                         intermediate_size, head_dim, conv_state, ssm_state, continuing=False):
    """Inference forward ``zxBCdt -> norm_out`` that updates the decode cache in place.

    ``conv_state`` (b, conv_dim, W), W in {k-1, k}: on return the last W rows of xBC (before the conv), oldest first.
    ``ssm_state`` (b, h, p, n) fp32: on return the scan's state after the last token.
    ``continuing``: the two tensors hold the state after an earlier prefix (prefill in pieces, or prefill after decode
    steps); otherwise they are taken as zero and only written."""
    z, xBC, dt, h, d_conv = _views(zxBCdt, n_groups, ssm_state_size, intermediate_size, head_dim)
    b, l, _ = zxBCdt.shape
    k, W = conv1d_weight.shape[-1], conv_state.shape[-1]
    if conv_state.shape != (b, d_conv, W) or not (k - 1 <= W):
        raise ValueError(f"conv_state must be (b, conv_dim, W >= k-1), got {tuple(conv_state.shape)}")
    if ssm_state.shape != (b, h, head_dim, ssm_state_size) or ssm_state.dtype != torch.float32:
        raise ValueError("ssm_state must be (b, h, p, n) float32")
    if l == 0:
        return torch.empty((b, 0, intermediate_size), dtype=zxBCdt.dtype, device=zxBCdt.device)
    with torch.no_grad():
        if continuing:
            # the cached inputs go in front of the new ones; the outputs for them are dropped
            hist = torch.cat([conv_state.transpose(1, 2).to(xBC.dtype), xBC], dim=1)
            conv_out = conv1d_forward(hist, conv1d_weight, conv1d_bias, "silu", channels_last=True)[:, W:]
            tail = hist[:, l:]
        else:
            conv_out = conv1d_forward(xBC, conv1d_weight, conv1d_bias, "silu", channels_last=True)
            tail = xBC[:, l - W:] if l >= W else torch.cat([xBC.new_zeros(b, W - l, d_conv), xBC], dim=1)
        x, Bm, Cm = _xbc_views(conv_out, n_groups, ssm_state_size, intermediate_size, head_dim)
        y, S = ssd_forward(dt, logA, x, Bm, Cm, D, initial_state=ssm_state if continuing else None, want_final_state=True,
                           dt_bias=dt_bias)
        ssm_state.copy_(S)
        conv_state.copy_(tail.transpose(1, 2))
        return glue.rmsnorm_gated_hip(y.view(b, l, intermediate_size), z, norm_weight, n_groups, NORM_EPS, out_dtype=zxBCdt.dtype)
