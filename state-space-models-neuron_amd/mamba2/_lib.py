"""ctypes binding of libmamba2_hip.so (the C ABI declared in include/mamba2_hip.h).

The structures below mirror the C structs field for field.  ``load()`` raises if
the library is missing: there is no CPU or PyTorch fallback in this package.
"""
import ctypes as C
import weakref
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmamba2_hip.so")

M2_F32, M2_BF16 = 0, 1
ACT = {None: 0, "identity": 0, "silu": 1, "swish": 1, "relu": 2}
CHUNK = 128

_i64, _i32, _vp, _sz = C.c_int64, C.c_int32, C.c_void_p, C.c_size_t


class Conv1dParams(C.Structure):
    _fields_ = [("x", _vp), ("w", _vp), ("bias", _vp), ("dy", _vp), ("y", _vp), ("dx", _vp), ("dw", _vp), ("db", _vp),
                ("workspace", _vp), ("workspace_bytes", _sz),
                ("batch", _i64), ("seqlen", _i64), ("channels", _i64), ("k", _i32),
                ("x_stride_b", _i64), ("x_stride_l", _i64), ("x_stride_c", _i64),
                ("y_stride_b", _i64), ("y_stride_l", _i64), ("y_stride_c", _i64),
                ("dx_stride_b", _i64), ("dx_stride_l", _i64), ("dx_stride_c", _i64),
                ("dtype", _i32), ("param_dtype", _i32), ("activation", _i32)]


class SsdParams(C.Structure):
    _fields_ = [("x", _vp), ("dt", _vp), ("A", _vp), ("B", _vp), ("C", _vp), ("D", _vp),
                ("initial_state", _vp), ("final_state", _vp), ("chunk_states", _vp), ("y", _vp),
                ("dy", _vp), ("d_final_state", _vp),
                ("dx", _vp), ("ddt", _vp), ("dA", _vp), ("dB", _vp), ("dC", _vp), ("dD", _vp), ("d_initial_state", _vp),
                ("workspace", _vp), ("workspace_bytes", _sz),
                ("batch", _i64), ("seqlen", _i64), ("nheads", _i64), ("headdim", _i64), ("dstate", _i64), ("ngroups", _i64),
                ("x_stride_b", _i64), ("x_stride_l", _i64), ("x_stride_h", _i64),
                ("dt_stride_b", _i64), ("dt_stride_l", _i64),
                ("B_stride_b", _i64), ("B_stride_l", _i64), ("B_stride_g", _i64),
                ("C_stride_b", _i64), ("C_stride_l", _i64), ("C_stride_g", _i64),
                ("y_stride_b", _i64), ("y_stride_l", _i64), ("y_stride_h", _i64),
                ("dy_stride_b", _i64), ("dy_stride_l", _i64), ("dy_stride_h", _i64),
                ("dx_stride_b", _i64), ("dx_stride_l", _i64), ("dx_stride_h", _i64),
                ("ddt_stride_b", _i64), ("ddt_stride_l", _i64),
                ("dB_stride_b", _i64), ("dB_stride_l", _i64), ("dB_stride_g", _i64),
                ("dC_stride_b", _i64), ("dC_stride_l", _i64), ("dC_stride_g", _i64),
                ("dtype", _i32), ("dt_dtype", _i32),
                ("dt_bias", _vp), ("d_dt_bias", _vp)]


class DecodeParams(C.Structure):
    _fields_ = [("xBC", _vp), ("conv_state", _vp), ("conv_w", _vp), ("conv_b", _vp),
                ("S", _vp), ("dt", _vp), ("A", _vp), ("D", _vp), ("y", _vp),
                ("workspace", _vp), ("workspace_bytes", _sz),
                ("batch", _i64), ("nheads", _i64), ("headdim", _i64), ("dstate", _i64), ("ngroups", _i64),
                ("k", _i32), ("W", _i32),
                ("xBC_stride_b", _i64), ("dt_stride_b", _i64), ("y_stride_b", _i64),
                ("dtype", _i32), ("param_dtype", _i32), ("activation", _i32), ("dt_bias", _vp)]


class RmsnormParams(C.Structure):
    _fields_ = [("x", _vp), ("z", _vp), ("weight", _vp), ("out", _vp), ("d_out", _vp), ("dx", _vp), ("dz", _vp), ("d_weight", _vp),
                ("workspace", _vp), ("workspace_bytes", _sz),
                ("rows", _i64), ("channels", _i64),
                ("x_stride_row", _i64), ("z_stride_row", _i64), ("out_stride_row", _i64), ("d_out_stride_row", _i64),
                ("dx_stride_row", _i64), ("dz_stride_row", _i64),
                ("n_groups", _i32), ("dtype", _i32), ("out_f32", _i32), ("eps", C.c_float)]


# name -> (restype, argtypes); every symbol the header declares
SYMBOLS = {
    "m2_abi_version": (C.c_int, []),
    "m2_last_error": (C.c_char_p, []),
    "m2_struct_layout": (C.c_int, [_i32, C.POINTER(_i64), _i32]),
    "m2_conv1d_fwd": (C.c_int, [C.POINTER(Conv1dParams), _vp]),
    "m2_conv1d_bwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "m2_conv1d_bwd": (C.c_int, [C.POINTER(Conv1dParams), _vp]),
    "m2_ssd_chunk_states_bytes": (_sz, [C.POINTER(SsdParams)]),
    "m2_ssd_fwd_workspace_bytes": (_sz, [C.POINTER(SsdParams)]),
    "m2_ssd_fwd": (C.c_int, [C.POINTER(SsdParams), _vp]),
    "m2_ssd_bwd_workspace_bytes": (_sz, [C.POINTER(SsdParams)]),
    "m2_ssd_bwd": (C.c_int, [C.POINTER(SsdParams), _vp]),
    "m2_decode_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64]),
    "m2_decode_step": (C.c_int, [C.POINTER(DecodeParams), _vp]),
    "m2_decode_step_static": (C.c_int, [C.POINTER(DecodeParams), _vp]),
    "m2_softplus_bias_fwd": (C.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _i64, _i32, _vp]),
    "m2_softplus_bias_bwd_workspace_bytes": (_sz, [_i64, _i64]),
    "m2_softplus_bias_bwd": (C.c_int, [_vp, _i64, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _sz, _i64, _i64, _i32, _vp]),
    "m2_rmsnorm_gated_fwd": (C.c_int, [C.POINTER(RmsnormParams), _vp]),
    "m2_rmsnorm_gated_bwd_workspace_bytes": (_sz, [_i64, _i64, _i32, _i32]),
    "m2_rmsnorm_gated_bwd": (C.c_int, [C.POINTER(RmsnormParams), _vp]),
    "m2_add_rmsnorm": (C.c_int, [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _i64, _i64, C.c_float, _i32, _vp]),
    "m2_mfma_selftest": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp]),
    "m2_stream_copy": (C.c_int, [_vp, _vp, _sz, _vp]),
    "m2_tile_walk": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _i64, C.c_int32, _vp]),
}

_lib = None


def load(path=None):
    """Load the library once.  Raises RuntimeError when it has not been built.  ``path`` names another build of the same
    ABI (it must be given on the first call of the process: the library that is loaded first stays)."""
    global _lib
    if _lib is not None:
        if path is not None and os.path.abspath(path) != _lib._name:
            raise RuntimeError(f"{_lib._name} is already loaded; cannot switch to {path}")
        return _lib
    path = os.path.abspath(path) if path is not None else LIB_PATH
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: build it with `python state-space-models-neuron_amd/build.py` "
            "(there is no fallback path; the HIP extension is required)")
    lib = C.CDLL(path)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().m2_last_error().decode("utf-8", "replace")
        if rc in (-1, -2, -3, -6):
            raise ValueError(f"{what}: {msg} (code {rc})")
        raise RuntimeError(f"{what}: {msg} (code {rc})")


def dtype_code(t):
    if t == torch.float32:
        return M2_F32
    if t == torch.bfloat16:
        return M2_BF16
    raise ValueError(f"unsupported dtype {t}: the HIP kernels take float32 or bfloat16")


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def stream_ptr(device=None):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("mamba2 HIP kernels need tensors on a GPU device (got %s); there is no CPU path" % t.device)


_f32_copies = {}          # id(tensor) -> (weak reference, key, fp32 copy); entries go when the tensor does


def f32_param(t):
    """fp32 contiguous values of a parameter-like tensor.  fp32 tensors are returned as they are.  For others (a model
    held in bfloat16) the converted copy is kept while autograd is off (inference loops call the same kernels thousands
    of times per second) and rebuilt when the tensor was written through autograd-visible in-place ops, moved or retyped;
    writes through ``.data`` are not seen."""
    if t.dtype == torch.float32:
        return t.detach().contiguous()
    if torch.is_grad_enabled():
        return t.detach().float().contiguous()
    key = (t.data_ptr(), t._version, t.dtype, tuple(t.shape))
    ident = id(t)                     # the caller's tensor object (a module's Parameter lives as long as the module)
    hit = _f32_copies.get(ident)
    if hit is None or hit[0]() is not t or hit[1] != key:
        hit = (weakref.ref(t, lambda _, i=ident: _f32_copies.pop(i, None)), key, t.detach().float().contiguous())
        _f32_copies[ident] = hit
    return hit[2]


class Workspace:
    """Caller-owned scratch memory, cached per (device, stream) and grown on demand.

    The kernels of one call are stream-ordered, and the next call on the same stream may
    overwrite the scratch, so one buffer per stream is enough.
    """
    _bufs = {}

    @classmethod
    def get(cls, nbytes, device):
        key = (device.index if device.index is not None else torch.cuda.current_device(),
               torch.cuda.current_stream(device).cuda_stream)
        buf = cls._bufs.get(key)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
            cls._bufs[key] = buf
        return buf
