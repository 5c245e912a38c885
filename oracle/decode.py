"""Single-token recurrent decode step oracle.  TEST INFRASTRUCTURE ONLY.

Follows ``mamba2/mamba2_kernel_inference.py``:
  conv state shift + 1-token conv + SiLU on all of [x | B | C]   (``:13-23``, default
      activation 'silu' ``:14``; B ``:69``, C ``:75``, x ``:87-90``)
  dA = exp(A * dt)                                               (``:81``)
  S' = S * dA + (dt * x) (x) B                                   (``:95-97``)
  y  = S' . C + D * x                                            (``:101-102``)

The conv state is (b, C, W).  The reference keeps W = k columns and shifts
``new[:, :k-1] = old[:, 1:]; new[:, k-1] = x`` (``:18-19``); a W = k-1 state
(the minimal history) is handled the same way: shift left by one, append x,
and the taps are the last k-1 OLD columns followed by x.

Pins (tests/test_oracle_decode.py): l decode steps from a zero state equal
``conv1d_ref`` + ``ssd_recurrent_ref`` on the same l tokens (y, final S, and
conv state == last W inputs) -- the check the reference's own test intends
(``tests/mamba2_kernel_test_no_tp.py:203-268``); zero in -> zero out
(``:62-105``); batch-row consistency (``:108-148``); and HF transformers'
``mamba2_selective_state_update`` goldens for the SSM part.
"""
import torch
import torch.nn.functional as F


def decode_step_ref(xBC, conv_state, conv_weight, conv_bias, S, dt, A, D=None, n_groups=1,
                    activation="silu"):
    """xBC (b,1,Cx); conv_state (b,Cx,W); conv_weight (Cx,k); conv_bias (Cx) or None;
    S (b,h,p,n); dt (b,1,h); A (h); D (h) or None.
    Returns (y (b,1,h*p), new_conv_state, new_S) -- fresh tensors."""
    b, h, p, n = S.shape
    k = conv_weight.shape[-1]
    W = conv_state.shape[-1]
    d_inner = h * p
    gn = n_groups * n
    assert xBC.shape[1] == 1 and xBC.shape[2] == d_inner + 2 * gn
    assert W >= k - 1
    xin = xBC[:, 0, :]                                                   # (b, Cx)
    new_conv = torch.cat([conv_state[:, :, 1:], xin[:, :, None]], dim=-1)  # (b, Cx, W)
    taps = torch.cat([conv_state[:, :, W - (k - 1):], xin[:, :, None]], dim=-1)  # (b, Cx, k)
    z = (taps * conv_weight[None]).sum(-1)
    if conv_bias is not None:
        z = z + conv_bias[None]
    if activation in ("silu", "swish"):
        z = F.silu(z)
    elif activation is not None:
        raise ValueError(activation)
    x = z[:, :d_inner].reshape(b, h, p)
    Bv = z[:, d_inner:d_inner + gn].reshape(b, n_groups, n).repeat_interleave(h // n_groups, dim=1)
    Cv = z[:, d_inner + gn:].reshape(b, n_groups, n).repeat_interleave(h // n_groups, dim=1)
    dtv = dt[:, 0, :]                                                    # (b, h)
    dA = torch.exp(A[None] * dtv)
    newS = S * dA[:, :, None, None] + (dtv[:, :, None] * x)[..., None] * Bv[:, :, None, :]
    y = torch.einsum("bhpn,bhn->bhp", newS, Cv)
    if D is not None:
        y = y + D[None, :, None] * x
    return y.reshape(b, 1, d_inner), new_conv, newS


def make_decode_inputs(b, h, p, n, g, k=4, W=3, seed=0, act_dtype=torch.float32, device="cpu"):
    """State ~ N(0, 0.1) fp32, conv state ~ N(0,1), token inputs as for the scan:
    xBC ~ N(0,1) (B, C slices scaled by 1/sqrt(n)), dt = exp(U(log 1e-3, log 1e-1)),
    A = -exp(U(0, log 16)), D = 1, conv w, bias ~ U(-1/2, 1/2)."""
    import math
    gen = torch.Generator(device="cpu").manual_seed(seed)
    d_inner = h * p
    Cx = d_inner + 2 * g * n
    xBC = torch.randn(b, 1, Cx, generator=gen)
    xBC[:, :, d_inner:] /= math.sqrt(n)
    conv_state = torch.randn(b, Cx, W, generator=gen)
    S = 0.1 * torch.randn(b, h, p, n, generator=gen)
    dt = torch.exp(torch.empty(b, 1, h).uniform_(math.log(1e-3), math.log(1e-1), generator=gen))
    A = -torch.exp(torch.empty(h).uniform_(0.0, math.log(16.0), generator=gen))
    D = torch.ones(h)
    w = torch.rand(Cx, k, generator=gen) - 0.5
    bias = torch.rand(Cx, generator=gen) - 0.5
    cast = lambda t: t.to(act_dtype).to(device)
    return {"xBC": cast(xBC), "conv_state": cast(conv_state), "conv_weight": cast(w),
            "conv_bias": cast(bias), "S": S.to(device), "dt": cast(dt), "A": A.to(device),
            "D": D.to(device)}
