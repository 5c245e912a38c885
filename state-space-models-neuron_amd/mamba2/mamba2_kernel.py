"""SSD chunked scan: ``Mamba2Kernel`` / ``mamba2_kernel`` with the reference's call signature
(``mamba2/mamba2_kernel.py:488-519``), computed by the gfx950 HIP kernels.

    mamba2_kernel(dt[b,l,h], A[h], X[b,l,h,p], B[b,l,g,n], C[b,l,g,n], D[h]) -> Y[b,l,h,p]

Extensions (keyword-only, default off): ``initial_state`` (b,h,p,n) fp32 and
``return_final_state`` -> (Y, S[b,h,p,n] fp32).  X, B, C may be strided views into a packed
[x | B | C] buffer as long as their innermost dimension is contiguous.
"""
import os

import torch

from . import _lib
from ._lib import SsdParams, ptr


def _strides3(t):
    return t.stride(0), t.stride(1), t.stride(2)


def _check_inner(name, t):
    if t.stride(-1) != 1 and t.shape[-1] > 1:
        raise ValueError(f"{name}: innermost dimension must be contiguous (stride {t.stride(-1)})")


def _fill_common(p, dt, A, X, B, C, D, dt_bias=None):
    b, l, h, hd = X.shape
    p.dt_bias = ptr(dt_bias)
    g, n = B.shape[2], B.shape[3]
    p.x, p.dt, p.A, p.B, p.C, p.D = ptr(X), ptr(dt), ptr(A), ptr(B), ptr(C), ptr(D)
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups = b, l, h, hd, n, g
    p.x_stride_b, p.x_stride_l, p.x_stride_h = _strides3(X)
    p.dt_stride_b, p.dt_stride_l = dt.stride(0), dt.stride(1)
    p.B_stride_b, p.B_stride_l, p.B_stride_g = _strides3(B)
    p.C_stride_b, p.C_stride_l, p.C_stride_g = _strides3(C)
    p.dtype = _lib.dtype_code(X.dtype)
    p.dt_dtype = _lib.dtype_code(dt.dtype)


def _validate(dt, A, X, B, C, D, initial_state):
    if X.dim() != 4 or B.dim() != 4 or C.dim() != 4 or dt.dim() != 3:
        raise ValueError("expected dt (b,l,h), X (b,l,h,p), B/C (b,l,g,n)")
    b, l, h, hd = X.shape
    if dt.shape != (b, l, h):
        raise ValueError(f"dt shape {tuple(dt.shape)} != {(b, l, h)}")
    if B.shape != C.shape or B.shape[:2] != (b, l):
        raise ValueError(f"B {tuple(B.shape)} / C {tuple(C.shape)} do not match X {tuple(X.shape)}")
    if h % B.shape[2] != 0:
        raise ValueError(f"n_heads {h} not divisible by n_groups {B.shape[2]}")
    if A.shape != (h,) or (D is not None and D.shape != (h,)):
        raise ValueError("A and D must have shape (n_heads,)")
    if B.dtype != X.dtype or C.dtype != X.dtype:
        raise ValueError("X, B and C must share one dtype")
    if dt.dtype not in (X.dtype, torch.float32):
        raise ValueError("dt must be float32 or have the dtype of X")
    for name, t in (("X", X), ("B", B), ("C", C), ("dt", dt)):
        _check_inner(name, t)
    if initial_state is not None and initial_state.shape != (b, h, hd, B.shape[3]):
        raise ValueError("initial_state must have shape (b, h, p, n)")
    _lib.require_gpu(dt, A, X, B, C, D, initial_state)


def _bias32(dt_bias, h):
    if dt_bias is None:
        return None
    if dt_bias.shape != (h,):
        raise ValueError("dt_bias must have shape (n_heads,)")
    _lib.require_gpu(dt_bias)
    return dt_bias.detach().float().contiguous()


def alloc_chunk_states(dt, A, X, B, C):
    """Carry-over buffer from ``ssd_forward(..., chunk_states=buf)`` to ``ssd_backward(..., chunk_states=buf)``
    (opaque bytes): the SSM state entering each 128-token chunk -- the first b*ceil(l/128)*h*p*n elements, in
    X's dtype -- followed by the decay tables and the per-chunk operand tiles."""
    lib = _lib.load()
    p = SsdParams()
    _fill_common(p, dt, A, X, B, C, None)
    return torch.empty(lib.m2_ssd_chunk_states_bytes(p), dtype=torch.uint8, device=X.device)


def ssd_forward(dt, A, X, B, C, D=None, initial_state=None, want_final_state=False, chunk_states=None, dt_bias=None):
    """Raw forward through the C ABI.  Returns (Y, final_state or None).
    With ``dt_bias`` (h), ``dt`` is the raw projection output and the step size is softplus(dt + dt_bias), applied inside."""
    _validate(dt, A, X, B, C, D, initial_state)
    lib = _lib.load()
    b, l, h, hd = X.shape
    n = B.shape[3]
    A32 = A.detach().float().contiguous()
    D32 = D.detach().float().contiguous() if D is not None else None
    S0 = initial_state.detach().float().contiguous() if initial_state is not None else None
    Y = torch.empty((b, l, h, hd), dtype=X.dtype, device=X.device)
    S = torch.empty((b, h, hd, n), dtype=torch.float32, device=X.device) if want_final_state else None
    p = SsdParams()
    bias32 = _bias32(dt_bias, h)
    _fill_common(p, dt, A32, X, B, C, D32, bias32)
    p.initial_state, p.final_state, p.y = ptr(S0), ptr(S), ptr(Y)
    p.chunk_states = _chunk_states_ptr(lib, p, chunk_states)
    p.y_stride_b, p.y_stride_l, p.y_stride_h = _strides3(Y)
    nbytes = lib.m2_ssd_fwd_workspace_bytes(p)
    ws = _lib.Workspace.get(nbytes, X.device)
    p.workspace, p.workspace_bytes = ptr(ws), ws.numel()
    with torch.cuda.device(X.device):
        _lib.check(lib.m2_ssd_fwd(p, _lib.stream_ptr(X.device)), "m2_ssd_fwd")
    return Y, S


def _chunk_states_ptr(lib, p, chunk_states):
    if chunk_states is None:
        return None
    need = lib.m2_ssd_chunk_states_bytes(p)
    if not chunk_states.is_contiguous() or chunk_states.numel() * chunk_states.element_size() != need:
        raise ValueError(f"chunk_states must be a contiguous buffer of {need} bytes (see alloc_chunk_states)")
    return ptr(chunk_states)


def ssd_backward(dt, A, X, B, C, D, dY, initial_state=None, d_final_state=None, want_dinitial=False,
                 out_dX=None, out_dB=None, out_dC=None, chunk_states=None, dt_bias=None, out_ddt=None):
    """Raw backward through the C ABI.
    Returns (ddt, dA fp32 (h), dX, dB, dC, dD fp32 (h) or None, d_initial_state or None), and as an eighth element
    d_dt_bias fp32 (h) when ``dt_bias`` is given (``dt`` is then the raw projection output and ddt its gradient).
    ``out_dX/out_dB/out_dC/out_ddt`` let the caller provide (strided) destinations, e.g. views of a packed
    [dx | dB | dC] buffer.  ``chunk_states``: what the forward wrote for the same inputs (skips the recompute)."""
    lib = _lib.load()
    b, l, h, hd = X.shape
    g, n = B.shape[2], B.shape[3]
    dev = X.device
    A32 = A.detach().float().contiguous()
    D32 = D.detach().float().contiguous() if D is not None else None
    S0 = initial_state.detach().float().contiguous() if initial_state is not None else None
    dSf = d_final_state.detach().float().contiguous() if d_final_state is not None else None
    if dY.stride(-1) != 1 or dY.dtype != X.dtype:
        dY = dY.to(X.dtype).contiguous()
    esz = dY.element_size()
    if any((s * esz) % 16 for s in dY.stride()[:3]) or dY.data_ptr() % 16:
        dY = dY.contiguous()
    if out_ddt is not None and (out_ddt.shape != (b, l, h) or out_ddt.dtype != dt.dtype or out_ddt.stride(-1) != 1):
        raise ValueError("out_ddt must have the shape and dtype of dt, heads contiguous")
    ddt = out_ddt if out_ddt is not None else torch.empty((b, l, h), dtype=dt.dtype, device=dev)
    bias32 = _bias32(dt_bias, h)
    d_bias = torch.empty((h,), dtype=torch.float32, device=dev) if dt_bias is not None else None
    dX = out_dX if out_dX is not None else torch.empty((b, l, h, hd), dtype=X.dtype, device=dev)
    dB = out_dB if out_dB is not None else torch.empty((b, l, g, n), dtype=B.dtype, device=dev)
    dC = out_dC if out_dC is not None else torch.empty((b, l, g, n), dtype=C.dtype, device=dev)
    dA = torch.empty((h,), dtype=torch.float32, device=dev)
    dD = torch.empty((h,), dtype=torch.float32, device=dev) if D is not None else None
    dS0 = torch.empty((b, h, hd, n), dtype=torch.float32, device=dev) if want_dinitial else None
    p = SsdParams()
    _fill_common(p, dt, A32, X, B, C, D32, bias32)
    p.d_dt_bias = ptr(d_bias)
    p.initial_state, p.dy, p.d_final_state = ptr(S0), ptr(dY), ptr(dSf)
    p.chunk_states = _chunk_states_ptr(lib, p, chunk_states)
    p.dx, p.ddt, p.dA, p.dB, p.dC, p.dD, p.d_initial_state = ptr(dX), ptr(ddt), ptr(dA), ptr(dB), ptr(dC), ptr(dD), ptr(dS0)
    p.dy_stride_b, p.dy_stride_l, p.dy_stride_h = _strides3(dY)
    p.dx_stride_b, p.dx_stride_l, p.dx_stride_h = _strides3(dX)
    p.ddt_stride_b, p.ddt_stride_l = ddt.stride(0), ddt.stride(1)
    p.dB_stride_b, p.dB_stride_l, p.dB_stride_g = _strides3(dB)
    p.dC_stride_b, p.dC_stride_l, p.dC_stride_g = _strides3(dC)
    nbytes = lib.m2_ssd_bwd_workspace_bytes(p)
    ws = _lib.Workspace.get(nbytes, dev)
    p.workspace, p.workspace_bytes = ptr(ws), ws.numel()
    with torch.cuda.device(dev):
        _lib.check(lib.m2_ssd_bwd(p, _lib.stream_ptr(dev)), "m2_ssd_bwd")
    if dt_bias is not None:
        return ddt, dA, dX, dB, dC, dD, dS0, d_bias
    return ddt, dA, dX, dB, dC, dD, dS0


# The reference saves only the inputs and recomputes the chunk states in the backward
# (``mamba2/mamba2_kernel.py:492,363-367``) because its device memory is scarce.  With 288 GB of HBM the
# states entering each chunk (as many bytes as X) are kept instead, which removes two kernels and
# ~0.5 GB of traffic from the backward at the 2.7B shape.  M2_SSD_SAVE_STATES=0 restores recompute.
SAVE_CHUNK_STATES = os.environ.get("M2_SSD_SAVE_STATES", "1") != "0"


class Mamba2Kernel(torch.autograd.Function):
    """forward(ctx, dt, A, X, B, C, D) -> Y; backward -> (ddt, dA, dX, dB, dC, dD)
    (``mamba2/mamba2_kernel.py:490,498,515``).  Two optional trailing arguments carry the
    extensions: ``initial_state`` and ``return_final_state``."""

    @staticmethod
    def forward(ctx, dt, A, X, B, C, D, initial_state=None, return_final_state=False):
        needs_grad = any(ctx.needs_input_grad[:7])
        states = alloc_chunk_states(dt, A, X, B, C) if (SAVE_CHUNK_STATES and needs_grad and X.numel() > 0) else None
        Y, S = ssd_forward(dt, A, X, B, C, D, initial_state, return_final_state, chunk_states=states)
        ctx.chunk_states = states
        ctx.save_for_backward(dt, A, X, B, C, D, initial_state)
        ctx.return_final_state = return_final_state
        if return_final_state:
            return Y, S
        return Y

    @staticmethod
    def backward(ctx, d_output, *rest):
        dt, A, X, B, C, D, initial_state = ctx.saved_tensors
        dS = rest[0] if (ctx.return_final_state and rest and rest[0] is not None) else None
        want_dinit = initial_state is not None and ctx.needs_input_grad[6]
        ddt, dA, dX, dB, dC, dD, dS0 = ssd_backward(dt, A, X, B, C, D, d_output, initial_state, dS, want_dinit,
                                                     chunk_states=ctx.chunk_states)
        ctx.chunk_states = None
        dA = dA.to(A.dtype)
        dD = dD.to(D.dtype) if D is not None else None
        return ddt, dA, dX, dB, dC, dD, dS0, None


def mamba2_kernel(dt, A, X, B, C, D, *, initial_state=None, return_final_state=False):
    return Mamba2Kernel.apply(dt, A, X, B, C, D, initial_state, return_final_state)
