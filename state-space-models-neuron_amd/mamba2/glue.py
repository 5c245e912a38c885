"""Elementwise glue of the mixer core: softplus(dt + dt_bias) and the gated, grouped RMSNorm, forward and
backward (``mamba2/fused_kernel.py:33-73,76-175``; torch twins ``mamba2/mamba2_mixer.py:36-38,88-105``).

These run as torch device ops on the caller's stream (elementwise / small reductions, no host round trips);
the SSD scan, conv and decode kernels are the hand-written HIP part of the path.
"""
import torch
import torch.nn.functional as F

SOFTPLUS_THRESHOLD = 10.0      # mamba2_mixer.py:36


def softplus_bias(dt, dt_bias):
    """softplus(dt + dt_bias) with the reference's threshold form; result in the dtype of dt."""
    v = dt.float() + dt_bias.float()
    return torch.where(v < SOFTPLUS_THRESHOLD, torch.log1p(torch.exp(torch.clamp(v, max=SOFTPLUS_THRESHOLD))), v).to(dt.dtype)


def softplus_bias_bwd(dt, dt_bias, d_out, out_d_in=None):
    """d_in = d_out * sigmoid(dt + dt_bias) (1 above the threshold); returns d_bias (h) fp32 (fused_kernel.py:68-72)."""
    v = dt.float() + dt_bias.float()
    d_in = d_out.float() * torch.where(v < SOFTPLUS_THRESHOLD, torch.sigmoid(v), torch.ones_like(v))
    if out_d_in is not None:
        out_d_in.copy_(d_in)
    return d_in.sum(dim=tuple(range(d_in.dim() - 1)))


def rmsnorm_gated(x, z, weight, n_groups, eps, out_dtype=None):
    """h = x * silu(z); per group of d/g contiguous channels out = h * rsqrt(mean h^2 + eps) * w, in fp32."""
    h = x.float()
    if z is not None:
        h = h * F.silu(z.float())
    shp = h.shape
    hg = h.reshape(*shp[:-1], n_groups, shp[-1] // n_groups)
    hg = hg * torch.rsqrt(hg.pow(2).mean(-1, keepdim=True) + eps)
    out = weight.float() * hg.reshape(shp)
    return out if out_dtype is None else out.to(out_dtype)


def rmsnorm_gated_bwd(x, z, weight, d_out, n_groups, eps, out_dz=None):
    """Returns (dx, dw fp32); dz is written into ``out_dz`` (fused_kernel.py:159-171)."""
    xf, zf, g = x.float(), z.float(), d_out.float()
    sig = torch.sigmoid(zf)
    gate = zf * sig
    h = xf * gate
    shp = h.shape
    G = n_groups
    hg = h.reshape(*shp[:-1], G, shp[-1] // G)
    var = hg.pow(2).mean(-1, keepdim=True) + eps
    rinv = torch.rsqrt(var)
    gw = (g * weight.float()).reshape(hg.shape)
    cf = (hg * gw).mean(-1, keepdim=True) / var
    d_h = (rinv * (gw - cf * hg)).reshape(shp)
    dw = (g * (hg * rinv).reshape(shp)).sum(dim=tuple(range(g.dim() - 1)))
    dx = (d_h * gate).to(x.dtype)
    dz = d_h * xf * (sig * (1 + zf * (1 - sig)))
    if out_dz is not None:
        out_dz.copy_(dz)
    return dx, dw
