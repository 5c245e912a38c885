"""Elementwise glue of the mixer core: softplus(dt + dt_bias) and the gated, grouped RMSNorm, forward and
backward (``mamba2/fused_kernel.py:33-73,76-175``; torch twins ``mamba2/mamba2_mixer.py:36-38,88-105``).

The ``*_hip`` functions call the HIP kernels (one pass over each tensor, strided rows taken in place) and are what the
fused mixer core uses.  ``rmsnorm_gated_fn`` wraps the forward and backward kernels in an autograd function, for the norm
modules (``MambaRMSNormGated``, the blocks' ``Mamba2RMSNorm``) and the one-token decode step.  There is no other path:
shapes the kernels do not take (a group wider than 8192 channels, or not a multiple of the 16-byte vector) raise.
"""
import ctypes as C

import torch

from . import _lib


# --------------------------------------------------------------------------------------------- HIP kernels
def _rows2d(t, name):
    """(rows, channels, row stride) of a (..., channels) tensor whose leading dimensions collapse to one stride."""
    if t.stride(-1) != 1 and t.shape[-1] > 1:
        raise ValueError(f"{name}: innermost dimension must be contiguous")
    ch = t.shape[-1]
    rows = t.numel() // ch if ch else 0
    if t.dim() == 1:
        return 1, ch, ch
    sr = t.stride(-2)
    # the leading dimensions must be walkable with the one row stride (true for contiguous tensors and column slices of them)
    exp = sr
    for k in range(t.dim() - 2, -1, -1):
        if t.shape[k] != 1 and t.stride(k) != exp:
            raise ValueError(f"{name}: rows are not evenly strided (shape {tuple(t.shape)}, strides {t.stride()})")
        exp *= t.shape[k]
    return rows, ch, sr


def _vec_ok(t):
    """True if the rows of ``t`` can be read as 16-byte vectors in place."""
    _, _, sr = _rows2d(t, "tensor")
    return t.data_ptr() % 16 == 0 and (sr * t.element_size()) % 16 == 0


def softplus_bias_hip(dt, dt_bias):
    """softplus(dt + dt_bias), threshold form; dt (..., h) may be a column slice; result contiguous, dtype of dt."""
    _lib.require_gpu(dt, dt_bias)
    lib = _lib.load()
    rows, h, sr = _rows2d(dt, "dt")
    out = torch.empty(dt.shape, dtype=dt.dtype, device=dt.device)
    bias = dt_bias.detach().float().contiguous()
    rc = lib.m2_softplus_bias_fwd(_lib.ptr(dt), sr, _lib.ptr(bias), _lib.ptr(out), h, rows, h, _lib.dtype_code(dt.dtype),
                                  _lib.stream_ptr(dt.device))
    _lib.check(rc, "m2_softplus_bias_fwd")
    return out


def softplus_bias_bwd_hip(dt, dt_bias, d_out, out_d_in=None):
    """Returns (d_in, d_bias fp32 (h)); d_in is written into ``out_d_in`` (a view with the dtype of dt) when given."""
    _lib.require_gpu(dt, dt_bias, d_out)
    lib = _lib.load()
    rows, h, sr = _rows2d(dt, "dt")
    if d_out.dtype != dt.dtype or d_out.stride(-1) != 1:
        d_out = d_out.to(dt.dtype).contiguous()
    _, _, dosr = _rows2d(d_out, "d_out")
    d_in = out_d_in if out_d_in is not None else torch.empty(dt.shape, dtype=dt.dtype, device=dt.device)
    if d_in.dtype != dt.dtype or d_in.shape != dt.shape:
        raise ValueError("softplus_bias_bwd: out_d_in must have the shape and dtype of dt")
    _, _, disr = _rows2d(d_in, "out_d_in")
    bias = dt_bias.detach().float().contiguous()
    d_bias = torch.empty(h, dtype=torch.float32, device=dt.device)
    nbytes = lib.m2_softplus_bias_bwd_workspace_bytes(rows, h)
    ws = _lib.Workspace.get(nbytes, dt.device)
    rc = lib.m2_softplus_bias_bwd(_lib.ptr(dt), sr, _lib.ptr(bias), _lib.ptr(d_out), dosr, _lib.ptr(d_in), disr, _lib.ptr(d_bias),
                                  _lib.ptr(ws), ws.numel(), rows, h, _lib.dtype_code(dt.dtype), _lib.stream_ptr(dt.device))
    _lib.check(rc, "m2_softplus_bias_bwd")
    return d_in, d_bias


def _norm_params(x, z, weight, n_groups, eps):
    p = _lib.RmsnormParams()
    # rows that cannot be read as 16-byte vectors where they lie (odd column offsets or row strides) are copied once
    if not _vec_ok(x):
        x = x.contiguous()
    rows, d, xsr = _rows2d(x, "x")
    p.x = _lib.ptr(x); p.x_stride_row = xsr
    keep = [x]
    if z is not None:
        if z.shape != x.shape or z.dtype != x.dtype:
            raise ValueError("rmsnorm_gated: z must have the shape and dtype of x")
        if not _vec_ok(z):
            z = z.contiguous()
        _, _, zsr = _rows2d(z, "z")
        p.z = _lib.ptr(z); p.z_stride_row = zsr
        keep.append(z)
    p.rows, p.channels, p.n_groups = rows, d, n_groups
    p.dtype = _lib.dtype_code(x.dtype)
    p.eps = float(eps)
    w32 = _lib.f32_param(weight)
    p.weight = _lib.ptr(w32)
    keep.append(w32)
    return p, keep


def rmsnorm_gated_hip(x, z, weight, n_groups, eps, out_dtype=None):
    """out = weight * h * rsqrt(mean_group(h^2) + eps), h = x * silu(z); out in ``out_dtype`` (fp32 or the dtype of x)."""
    _lib.require_gpu(x, z, weight)
    lib = _lib.load()
    out_dtype = torch.float32 if out_dtype is None else out_dtype
    if out_dtype not in (torch.float32, x.dtype):
        raise ValueError("rmsnorm_gated: out_dtype must be float32 or the dtype of x")
    p, keep = _norm_params(x, z, weight, n_groups, eps)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    p.out = _lib.ptr(out); p.out_stride_row = x.shape[-1]
    p.out_f32 = 1 if out_dtype == torch.float32 else 0
    _lib.check(lib.m2_rmsnorm_gated_fwd(C.byref(p), _lib.stream_ptr(x.device)), "m2_rmsnorm_gated_fwd")
    return out


def rmsnorm_gated_bwd_hip(x, z, weight, d_out, n_groups, eps, out_dz=None):
    """Returns (dx, dw fp32); dz is written into ``out_dz`` (a view with the dtype of x) or a fresh tensor."""
    _lib.require_gpu(x, z, weight, d_out)
    lib = _lib.load()
    if d_out.dtype != x.dtype or d_out.stride(-1) != 1 or not _vec_ok(d_out):
        d_out = d_out.to(x.dtype).contiguous()
    p, keep = _norm_params(x, z, weight, n_groups, eps)
    _, _, gsr = _rows2d(d_out, "d_out")
    p.d_out = _lib.ptr(d_out); p.d_out_stride_row = gsr
    dx = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    p.dx = _lib.ptr(dx); p.dx_stride_row = x.shape[-1]
    dz = None
    if z is not None:
        if out_dz is not None and (out_dz.dtype != x.dtype or out_dz.shape != x.shape):
            raise ValueError("rmsnorm_gated_bwd: out_dz must have the shape and dtype of x")
        dz = out_dz if (out_dz is not None and _vec_ok(out_dz)) else torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _, _, dzsr = _rows2d(dz, "out_dz")
        p.dz = _lib.ptr(dz); p.dz_stride_row = dzsr
    dw = torch.empty(x.shape[-1], dtype=torch.float32, device=x.device)
    p.d_weight = _lib.ptr(dw)
    nbytes = lib.m2_rmsnorm_gated_bwd_workspace_bytes(p.rows, p.channels, n_groups, p.dtype)
    ws = _lib.Workspace.get(nbytes, x.device)
    p.workspace = _lib.ptr(ws); p.workspace_bytes = ws.numel()
    _lib.check(lib.m2_rmsnorm_gated_bwd(C.byref(p), _lib.stream_ptr(x.device)), "m2_rmsnorm_gated_bwd")
    if out_dz is not None and dz is not out_dz:
        out_dz.copy_(dz)
        dz = out_dz
    return dx, dw, dz


def add_rmsnorm_ok(channels, out_dtype):
    """True if ``add_rmsnorm_`` takes rows of this width: a multiple of 4, at most 8192 channels, fp32 or bf16 output."""
    return channels % 4 == 0 and 0 < channels <= 8192 and out_dtype in (torch.float32, torch.bfloat16)


def add_rmsnorm_(residual, delta, weight, eps, out_dtype):
    """``residual += delta`` in place (fp32), then RMSNorm of the sum, in one kernel (inference; the block boundary of the
    token-by-token loop, ``modeling_mamba2.py:133-140`` + ``:94-103``).  ``delta`` (dtype ``out_dtype``) may be None.
    Returns weight * residual * rsqrt(mean(residual^2) + eps) in ``out_dtype``."""
    _lib.require_gpu(residual, delta, weight)
    lib = _lib.load()
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise ValueError("add_rmsnorm_: the residual stream must be contiguous float32")
    rows, d, rsr = _rows2d(residual, "residual")
    dsr = 0
    if delta is not None:
        if delta.shape != residual.shape or delta.dtype != out_dtype:
            raise ValueError("add_rmsnorm_: delta must have the residual's shape and the output dtype")
        if delta.stride(-1) != 1:
            delta = delta.contiguous()
        _, _, dsr = _rows2d(delta, "delta")
    out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
    w32 = _lib.f32_param(weight)
    rc = lib.m2_add_rmsnorm(_lib.ptr(residual), rsr, _lib.ptr(delta), dsr, _lib.ptr(w32), _lib.ptr(out), d, rows, d, float(eps),
                            _lib.dtype_code(out_dtype), _lib.stream_ptr(residual.device))
    _lib.check(rc, "m2_add_rmsnorm")
    return out


# --------------------------------------------------------------------------------------------- autograd form
def norm_kernel_ok(x, n_groups):
    """True if the HIP norm kernels take this shape: group width a multiple of the vector width and within a row's registers."""
    if x.dtype not in (torch.float32, torch.bfloat16) or n_groups < 1 or x.shape[-1] % n_groups:
        return False
    gw = x.shape[-1] // n_groups
    vec = 8 if x.dtype == torch.bfloat16 else 4
    return gw % vec == 0 and 0 < gw <= 8192


class RmsnormGated(torch.autograd.Function):
    """Gated grouped RMSNorm on the HIP kernels, forward and backward (z may be None: plain RMSNorm)."""

    @staticmethod
    def forward(ctx, x, z, weight, n_groups, eps, out_dtype):
        ctx.save_for_backward(x, z, weight)
        ctx.n_groups, ctx.eps = n_groups, eps
        return rmsnorm_gated_hip(x, z, weight, n_groups, eps, out_dtype=out_dtype)

    @staticmethod
    def backward(ctx, d_out):
        x, z, weight = ctx.saved_tensors
        dx, dw, dz = rmsnorm_gated_bwd_hip(x, z, weight, d_out, ctx.n_groups, ctx.eps)
        return dx, dz, dw.to(weight.dtype), None, None, None


def rmsnorm_gated_fn(x, z, weight, n_groups, eps, out_dtype=None):
    """Differentiable gated grouped RMSNorm; output fp32 unless ``out_dtype`` says the dtype of x.
    Raises ValueError for shapes outside the kernels' limits."""
    _lib.require_gpu(x, z, weight)
    if not norm_kernel_ok(x, n_groups):
        raise ValueError(f"rmsnorm_gated: {x.shape[-1]} channels in {n_groups} groups, dtype {x.dtype}: a group must be a "
                         "multiple of 16 bytes and at most 8192 channels wide, in float32 or bfloat16")
    if z is not None and z.dtype != x.dtype:
        raise ValueError("rmsnorm_gated: z must have the dtype of x")
    return RmsnormGated.apply(x, z, weight, n_groups, eps, out_dtype)
