"""GPU: m2_decode_step_static (the decode step whose scratch lives inside the library, for callers that cannot allocate)
against m2_decode_step, through the C ABI: bit-identical outputs on two calls in a row, the second with a smaller input;
sizes beyond the built-in scratch are refused."""
import ctypes

import pytest
import torch

from oracle.decode import decode_step_ref, make_decode_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _params(_lib, q, y, workspace=None):
    b, h, p, n = q["S"].shape
    Cx = q["xBC"].shape[-1]
    g = (Cx - h * p) // (2 * n)
    P = _lib.DecodeParams()
    P.xBC, P.conv_state, P.conv_w, P.conv_b = (_lib.ptr(q[k]) for k in ("xBC", "conv_state", "conv_weight", "conv_bias"))
    P.S, P.dt, P.A, P.D, P.y = _lib.ptr(q["S"]), _lib.ptr(q["dt"]), _lib.ptr(q["A"]), _lib.ptr(q["D"]), _lib.ptr(y)
    if workspace is not None:
        P.workspace, P.workspace_bytes = _lib.ptr(workspace), workspace.numel()
    P.batch, P.nheads, P.headdim, P.dstate, P.ngroups = b, h, p, n, g
    P.k, P.W = q["conv_weight"].shape[-1], q["conv_state"].shape[-1]
    P.xBC_stride_b, P.dt_stride_b, P.y_stride_b = q["xBC"].stride(0), q["dt"].stride(0), y.stride(0)
    P.dtype, P.param_dtype = _lib.dtype_code(q["xBC"].dtype), _lib.dtype_code(q["conv_weight"].dtype)
    P.activation = _lib.ACT["silu"]
    return P


def _both(lib, _lib, shape, seed):
    b, h, p, n, g = shape
    q = make_decode_inputs(b, h, p, n, g, k=4, W=3, seed=seed, act_dtype=torch.bfloat16, device=DEV)
    host = {k: v.cpu() for k, v in q.items()}
    qa = {k: v.clone() for k, v in q.items()}
    qb = {k: v.clone() for k, v in q.items()}
    ya = torch.empty(b, 1, h * p, dtype=torch.bfloat16, device=DEV)
    yb = torch.full_like(ya, 7.0)
    ws = torch.empty(lib.m2_decode_workspace_bytes(b, h, p, n, g), dtype=torch.uint8, device=DEV)
    st = _lib.stream_ptr()
    assert lib.m2_decode_step(ctypes.byref(_params(_lib, qa, ya, ws)), st) == 0, lib.m2_last_error()
    assert lib.m2_decode_step_static(ctypes.byref(_params(_lib, qb, yb)), st) == 0, lib.m2_last_error()
    torch.cuda.synchronize()
    # the same kernels on the same inputs: bit-identical outputs and states
    assert torch.equal(ya, yb)
    assert torch.equal(qa["S"], qb["S"]) and torch.equal(qa["conv_state"], qb["conv_state"])
    # and the entry point is right, not only consistent: against the fp64 oracle
    y_ref, cs_ref, S_ref = decode_step_ref(*(host[k].double() for k in ("xBC", "conv_state", "conv_weight", "conv_bias", "S", "dt", "A", "D")),
                                           n_groups=g)
    assert torch.equal(qb["conv_state"].cpu().double(), cs_ref)
    assert ((qb["S"].cpu().double() - S_ref).abs().max() / S_ref.abs().max()).item() < 1e-4
    rms = y_ref.pow(2).mean().sqrt()
    floor = ((y_ref.to(torch.bfloat16).double() - y_ref).abs().max() / rms).item()
    assert ((yb.cpu().double() - y_ref).abs().max() / rms).item() < 2e-2 + floor


def test_decode_step_static_matches_decode_step_twice(lib):
    from mamba2 import _lib
    _both(lib, _lib, (16, 8, 64, 128, 1), seed=21)       # 16 x 768 floats of scratch
    _both(lib, _lib, (3, 4, 64, 64, 2), seed=22)         # smaller: the scratch still holds the previous call's values


def test_decode_step_static_through_wrapper_and_limit(lib):
    from mamba2 import _lib
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    q = make_decode_inputs(4, 4, 64, 128, 2, k=4, W=3, seed=23, act_dtype=torch.bfloat16, device=DEV)
    args = lambda d: (d["xBC"], d["conv_state"], d["conv_weight"], d["conv_bias"], d["S"], d["dt"], d["A"], d["D"])
    qa = {k: v.clone() for k, v in q.items()}
    qb = {k: v.clone() for k, v in q.items()}
    ya, _, _ = mamba2_kernel_inference(*args(qa), n_groups=2)
    out = torch.empty_like(ya)
    yb, _, _ = mamba2_kernel_inference(*args(qb), n_groups=2, out=out, static_scratch=True)
    assert yb.data_ptr() == out.data_ptr() and torch.equal(ya, yb) and torch.equal(qa["S"], qb["S"])
    # beyond the built-in scratch (batch x channels > 2^20): refused before anything is launched
    P = _lib.DecodeParams()
    P.batch, P.nheads, P.headdim, P.dstate, P.ngroups, P.k, P.W, P.dtype, P.param_dtype = 256, 80, 64, 128, 1, 4, 3, 1, 1
    assert lib.m2_decode_step_static(ctypes.byref(P), None) == -4
    assert b"exceed the built-in scratch" in lib.m2_last_error()
