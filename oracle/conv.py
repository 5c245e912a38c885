"""Causal depthwise conv1d (+activation) oracle.  TEST INFRASTRUCTURE ONLY.

Semantics (``mamba2/conv1d_grouped.py:69-81``): for weight (C, 1, k), bias (C),
    y[b, t, c] = act(bias[c] + sum_{i<k} w[c, 0, i] * x[b, t - (k-1) + i, c]),  x[t<0] = 0
i.e. ``nn.Conv1d(C, C, k, groups=C, padding=k-1)(x)[..., :L]``.

Pins (tests/test_oracle_conv.py): ``conv1d_ref`` is the library routine
``F.conv1d`` the reference's own parity script uses (``conv1d_grouped.py:349-367``);
it is cross-checked with a brute-force tap loop, with an impulse-response test
(an impulse at t0 in channel c yields w[c, k-1-d] at t0+d) and with HF
transformers' ``causal_conv1d_fn`` goldens.  Gradients come from autograd.
The reference's own backward kernel zero-pads the pre-activation gradient per
128-token tile (``conv1d_grouped.py:173-176``), which drops the cross-tile
contribution to dx; the oracle deliberately does NOT reproduce that defect.
"""
import torch
import torch.nn.functional as F


def _act(z, activation):
    if activation is None or activation == "identity":
        return z
    if activation in ("silu", "swish"):
        return F.silu(z)
    if activation == "relu":
        return F.relu(z)
    raise ValueError(f"Invalid activation {activation}")


def conv1d_ref(x, weight, bias=None, activation=None, channels_last=True):
    """x: (b, l, C) if channels_last else (b, C, l).  weight: (C, 1, k).  Same layout out."""
    C, _, k = weight.shape
    xc = x.transpose(1, 2) if channels_last else x
    L = xc.shape[-1]
    y = F.conv1d(xc, weight, bias, padding=k - 1, groups=C)[..., :L]
    y = _act(y, activation)
    return y.transpose(1, 2) if channels_last else y


def conv1d_bruteforce(x, weight, bias=None, activation=None):
    """Explicit tap loop on (b, l, C); independent of F.conv1d."""
    b, l, C = x.shape
    k = weight.shape[-1]
    y = torch.zeros_like(x)
    for i in range(k):
        shift = k - 1 - i
        if shift >= l:
            continue
        y[:, shift:, :] += x[:, : l - shift, :] * weight[:, 0, i][None, None, :]
    if bias is not None:
        y = y + bias[None, None, :]
    return _act(y, activation)


def conv1d_grads_ref(x, weight, bias, dy, activation="silu", channels_last=True):
    """(y, dx, dw, db) by autograd through ``conv1d_ref``."""
    xl = x.detach().clone().requires_grad_(True)
    wl = weight.detach().clone().requires_grad_(True)
    bl = bias.detach().clone().requires_grad_(True) if bias is not None else None
    y = conv1d_ref(xl, wl, bl, activation, channels_last)
    wrt = [xl, wl] + ([bl] if bl is not None else [])
    g = torch.autograd.grad((y * dy).sum(), wrt)
    return y.detach(), g[0], g[1], (g[2] if bl is not None else None)


def make_conv_inputs(b, l, C, k=4, seed=0, dtype=torch.float32, device="cpu"):
    """x, dy ~ N(0,1); w, bias ~ U(-1/2, 1/2); drawn in fp32 then rounded to ``dtype``."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(b, l, C, generator=gen)
    dy = torch.randn(b, l, C, generator=gen)
    w = torch.rand(C, 1, k, generator=gen) - 0.5
    bias = torch.rand(C, generator=gen) - 0.5
    cast = lambda t: t.to(dtype).to(device)
    return {"x": cast(x), "dy": cast(dy), "w": cast(w), "bias": cast(bias)}
