"""Single-token decode step with the reference's signature
(``mamba2/mamba2_kernel_inference.py:107-122``), computed by the gfx950 HIP kernels.

    mamba2_kernel_inference(xBC[b,1,Cx], conv_state[b,Cx,W], conv_weight[Cx,k], conv_bias[Cx],
                            S[b,h,p,n], dt[b,1,h], logA[h], D[h]=None, n_groups=1)
        -> (Y[b,1,h*p], conv_state, S)

Unlike the reference, which writes fresh output tensors, ``conv_state`` and ``S`` are updated IN
PLACE and the same tensors are returned, which is compatible with the caller's re-binding of the
cache entries (``mamba2/mamba2_mixer.py:275-276``).  W may be k-1 or k columns.  The SSM state must
be float32.  ``xBC`` and ``dt`` may be column slices of the packed projection output.  With the keyword
``dt_bias`` (h), ``dt`` is the raw projection output and the kernel applies softplus(dt + dt_bias) itself
(the caller's ``softplus`` pass of ``mamba2_mixer.py:268`` is then not needed).  ``out`` takes a preallocated Y;
``static_scratch=True`` runs the step through ``m2_decode_step_static``, whose scratch lives inside the library (nothing
is allocated for it; batch x channels is limited, and calls that overlap on one GPU must not use it at the same time).
"""
import torch

from . import _lib
from ._lib import DecodeParams, ptr


def mamba2_kernel_inference(xBC_tensor, conv_state_tensor, conv_weight_tensor, conv_bias_tensor, S_tensor, dt_tensor,
                            logA_tensor, D_tensor=None, n_groups=1, activation="silu", dt_bias=None, out=None, static_scratch=False):
    batch_size, n_heads, d_head, d_state = S_tensor.shape
    seq_len = xBC_tensor.shape[1]
    assert seq_len == 1
    d_inner = n_heads * d_head
    d_xBC = xBC_tensor.shape[-1]
    assert d_xBC == d_inner + 2 * n_groups * d_state, f"Expected d_xBC {d_inner + 2 * n_groups * d_state}, got {d_xBC}"
    assert n_heads % n_groups == 0, "Number of heads must be divisible by number of groups"
    assert dt_tensor.shape == (batch_size, 1, n_heads)
    k = conv_weight_tensor.shape[-1]
    W = conv_state_tensor.shape[-1]
    if S_tensor.dtype != torch.float32:
        raise ValueError("the SSM state must be float32")
    if conv_state_tensor.dtype != xBC_tensor.dtype or dt_tensor.dtype != xBC_tensor.dtype:
        raise ValueError("xBC, conv_state and dt must share one dtype")
    if not (S_tensor.is_contiguous() and conv_state_tensor.is_contiguous()):
        raise ValueError("S and conv_state must be contiguous (they are updated in place)")
    if xBC_tensor.stride(-1) != 1 or dt_tensor.stride(-1) != 1:
        raise ValueError("xBC and dt must be contiguous in their last dimension")
    _lib.require_gpu(xBC_tensor, conv_state_tensor, conv_weight_tensor, conv_bias_tensor, S_tensor, dt_tensor, logA_tensor, D_tensor,
                     dt_bias)
    if dt_bias is not None and dt_bias.shape != (n_heads,):
        raise ValueError("dt_bias must have shape (n_heads,)")
    lib = _lib.load()
    dev = xBC_tensor.device
    w = conv_weight_tensor.detach().reshape(d_xBC, k).contiguous()
    bias = conv_bias_tensor.detach().contiguous() if conv_bias_tensor is not None else None
    A32 = logA_tensor.detach().float().contiguous()
    D32 = D_tensor.detach().float().contiguous() if D_tensor is not None else None
    bias32 = dt_bias.detach().float().contiguous() if dt_bias is not None else None
    if out is not None and (out.shape != (batch_size, seq_len, d_inner) or out.dtype != xBC_tensor.dtype or out.stride(-1) != 1
                            or out.device != dev):
        raise ValueError("out must be (batch, 1, n_heads * d_head) in the dtype of xBC, on its device")
    out_Y = out if out is not None else torch.empty((batch_size, seq_len, d_inner), device=dev, dtype=xBC_tensor.dtype)
    p = DecodeParams()
    if not static_scratch:
        nbytes = lib.m2_decode_workspace_bytes(batch_size, n_heads, d_head, d_state, n_groups)
        ws = _lib.Workspace.get(nbytes, dev)
        p.workspace, p.workspace_bytes = ptr(ws), ws.numel()
    p.xBC, p.conv_state, p.conv_w, p.conv_b = ptr(xBC_tensor), ptr(conv_state_tensor), ptr(w), ptr(bias)
    p.S, p.dt, p.A, p.D, p.y = ptr(S_tensor), ptr(dt_tensor), ptr(A32), ptr(D32), ptr(out_Y)
    p.batch, p.nheads, p.headdim, p.dstate, p.ngroups = batch_size, n_heads, d_head, d_state, n_groups
    p.k, p.W = k, W
    p.xBC_stride_b, p.dt_stride_b, p.y_stride_b = xBC_tensor.stride(0), dt_tensor.stride(0), out_Y.stride(0)
    p.dtype, p.param_dtype = _lib.dtype_code(xBC_tensor.dtype), _lib.dtype_code(w.dtype)
    p.activation = _lib.ACT[activation]
    p.dt_bias = ptr(bias32)
    with torch.cuda.device(dev):
        if static_scratch:
            _lib.check(lib.m2_decode_step_static(p, _lib.stream_ptr(dev)), "m2_decode_step_static")
        else:
            _lib.check(lib.m2_decode_step(p, _lib.stream_ptr(dev)), "m2_decode_step")
    return out_Y, conv_state_tensor, S_tensor
