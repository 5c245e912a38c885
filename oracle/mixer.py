"""Mixer-core glue oracle.  TEST INFRASTRUCTURE ONLY.

* ``softplus_ref``           -- ``mamba2/mamba2_mixer.py:36-38`` (threshold 10) /
                                ``mamba2/fused_kernel.py:33-47`` (softplus(dt + dt_bias)).
* ``rmsnorm_gated_ref``      -- ``mamba2/mamba2_mixer.py:88-105`` / ``fused_kernel.py:76-103``:
                                h = x * silu(z); per group of d_inner/g contiguous channels
                                out = h * rsqrt(mean(h^2) + eps) * w, computed in fp32.
* ``fused_core_ref``         -- the pipeline of ``fused_kernel.py:252-282``:
                                split [z | xBC | dt] -> conv+SiLU -> softplus(dt + bias) -> SSD -> norm.

Pins (tests/test_oracle_mixer.py): softplus vs ``F.softplus``; the norm vs a
per-group explicit loop and vs HF transformers' ``MambaRMSNormGated`` when
g = 1 (HF normalises across all of d_inner); the pipeline is a composition of
pinned parts and is compared with HF's torch ``Mamba2Mixer`` path for g = 1 via
golden vectors.
"""
import torch
import torch.nn.functional as F

from .conv import conv1d_ref
from .ssd import ssd_chunked_ref


def softplus_ref(x, threshold=10.0):
    return torch.where(x < threshold, torch.log1p(torch.exp(torch.clamp(x, max=threshold))), x)


def rmsnorm_gated_ref(x, z, weight, n_groups=1, eps=1e-5):
    """x, z: (..., d_inner); weight (d_inner).  fp32 (or fp64 if x is fp64) output."""
    ct = torch.float64 if x.dtype == torch.float64 else torch.float32
    h = x.to(ct)
    if z is not None:
        h = h * F.silu(z.to(ct))
    shp = h.shape
    hg = h.reshape(*shp[:-1], n_groups, shp[-1] // n_groups)
    var = hg.pow(2).mean(-1, keepdim=True)
    hg = hg * torch.rsqrt(var + eps)
    return weight.to(ct) * hg.reshape(shp)


def fused_core_ref(zxBCdt, A, D, conv_w, conv_b, dt_bias, norm_w, n_groups, d_state, d_inner, d_head,
                   chunk=128, eps=1e-5, handover=None):
    """zxBCdt (b, l, 2*d_inner + 2*g*n + h) -> norm_out (b, l, d_inner).
    Split order [z | xBC | dt] (``mamba2_mixer.py:265``), xBC order [x | B | C]
    (``mamba2_kernel.py:109-115,151``).

    ``handover`` (optional callable) is applied to every tensor one stage stores for the next
    (conv output, scan output, norm output); tests pass a round-to-bfloat16 to model what storing
    those tensors in the activation dtype, as the reference does, costs in accuracy."""
    if handover is None:
        handover = lambda t: t
    b, l, _ = zxBCdt.shape
    h = d_inner // d_head
    d_conv = d_inner + 2 * n_groups * d_state
    z, xBC, dt = torch.split(zxBCdt, [d_inner, d_conv, h], dim=-1)
    xBC = handover(conv1d_ref(xBC, conv_w, conv_b, "silu", channels_last=True))
    dt = softplus_ref(dt + dt_bias)
    x, Bm, Cm = torch.split(xBC, [d_inner, n_groups * d_state, n_groups * d_state], dim=-1)
    y, _ = ssd_chunked_ref(dt, A.to(x.dtype), x.reshape(b, l, h, d_head),
                           Bm.reshape(b, l, n_groups, d_state), Cm.reshape(b, l, n_groups, d_state),
                           D.to(x.dtype) if D is not None else None, chunk=chunk)
    return handover(rmsnorm_gated_ref(handover(y).reshape(b, l, d_inner), z, norm_w, n_groups, eps))
