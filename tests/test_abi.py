"""CPU: the C-ABI library loads and exports every symbol the header declares; argument validation
that happens before any device call; the Python layer refuses CPU tensors (no fallback path)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    txt = open(os.path.join(ROOT, "include", "mamba2_hip.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(m2_[a-z0-9_]+)\s*\(", txt)))


def test_header_symbols_exported_and_bound(lib):
    from mamba2 import _lib
    syms = _header_symbols()
    assert len(syms) >= 13
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in the header but not exported"
        assert s in _lib.SYMBOLS, f"{s} has no ctypes prototype"
    assert sorted(_lib.SYMBOLS) == syms
    assert lib.m2_abi_version() == 4


def test_struct_sizes_match_header():
    # field counts guard against drift between the header and the ctypes mirror
    from mamba2 import _lib
    txt = open(os.path.join(ROOT, "include", "mamba2_hip.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    for cname, pyc in (("m2_conv1d_params", _lib.Conv1dParams), ("m2_ssd_params", _lib.SsdParams), ("m2_decode_params", _lib.DecodeParams),
                       ("m2_rmsnorm_params", _lib.RmsnormParams)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), txt, flags=re.S).group(1)
        names = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            parts = decl.split(",")
            first = parts[0].split()[-1].lstrip("*")
            names.append(first)
            names += [q.strip().lstrip("*") for q in parts[1:]]
        assert names == [f[0] for f in pyc._fields_], cname


def test_struct_layout_matches_library(lib):
    # size and every field offset of the ctypes mirrors against what the compiled library reports
    from mamba2 import _lib
    for which, pyc in enumerate((_lib.Conv1dParams, _lib.SsdParams, _lib.DecodeParams, _lib.RmsnormParams)):
        buf = (ctypes.c_int64 * 128)()
        n = lib.m2_struct_layout(which, buf, 128)
        assert n == 1 + len(pyc._fields_), pyc.__name__
        assert buf[0] == ctypes.sizeof(pyc), pyc.__name__
        for i, (fname, _) in enumerate(pyc._fields_):
            assert buf[1 + i] == getattr(pyc, fname).offset, f"{pyc.__name__}.{fname}"
    assert lib.m2_struct_layout(9, (ctypes.c_int64 * 4)(), 4) == -1


def test_validation_before_any_device_call(lib):
    from mamba2 import _lib
    p = _lib.Conv1dParams()
    p.batch, p.seqlen, p.channels, p.k = 1, 8, 8, 9
    assert lib.m2_conv1d_fwd(ctypes.byref(p), None) == -1
    assert b"kernel size" in lib.m2_last_error()
    p.k, p.dtype = 4, 7
    assert lib.m2_conv1d_fwd(ctypes.byref(p), None) == -2
    s = _lib.SsdParams()
    s.batch, s.seqlen, s.nheads, s.headdim, s.dstate, s.ngroups = 1, 128, 2, 48, 64, 1
    assert lib.m2_ssd_fwd(ctypes.byref(s), None) == -1 and b"headdim" in lib.m2_last_error()
    s.headdim, s.ngroups, s.nheads = 64, 2, 3
    assert lib.m2_ssd_fwd(ctypes.byref(s), None) == -1 and b"divisible" in lib.m2_last_error()
    s.nheads = 4
    assert lib.m2_ssd_fwd(ctypes.byref(s), None) == -6          # NULL inputs
    d = _lib.DecodeParams()
    d.batch, d.nheads, d.headdim, d.dstate, d.ngroups, d.k, d.W = 1, 2, 4, 8, 1, 4, 2
    assert lib.m2_decode_step(ctypes.byref(d), None) == -1 and b"conv state width" in lib.m2_last_error()
    assert lib.m2_ssd_fwd(None, None) == -6
    # workspace sizing is pure host arithmetic
    s.batch, s.seqlen, s.nheads, s.headdim, s.dstate, s.ngroups, s.dtype = 4, 2048, 80, 64, 128, 1, 1
    fw, bw = lib.m2_ssd_fwd_workspace_bytes(ctypes.byref(s)), lib.m2_ssd_bwd_workspace_bytes(ctypes.byref(s))
    tiles = 4 * 16 * 80 * 64 * 128
    assert fw >= tiles * 2 and bw >= fw + tiles * 2      # bf16: the states entering the chunks (+ their gradients)
    s.dtype = 0
    assert lib.m2_ssd_fwd_workspace_bytes(ctypes.byref(s)) >= tiles * 8      # fp32: per-chunk contributions and states
    # mixer glue
    n = _lib.RmsnormParams()
    n.rows, n.channels, n.n_groups, n.dtype = 4, 96, 5, 1
    assert lib.m2_rmsnorm_gated_fwd(ctypes.byref(n), None) == -1             # channels not divisible by the groups
    n.n_groups = 8
    assert lib.m2_rmsnorm_gated_fwd(ctypes.byref(n), None) == -1 and b"multiple of 8" in lib.m2_last_error()
    n.channels, n.n_groups = 128, 2
    assert lib.m2_rmsnorm_gated_fwd(ctypes.byref(n), None) == -6             # NULL tensors
    assert lib.m2_rmsnorm_gated_bwd(ctypes.byref(n), None) == -6
    n.dtype = 5
    assert lib.m2_rmsnorm_gated_fwd(ctypes.byref(n), None) == -2
    assert lib.m2_softplus_bias_fwd(None, 8, None, None, 8, 4, 0, 1, None) == -1      # no heads
    assert lib.m2_softplus_bias_fwd(None, 8, None, None, 8, 4, 8, 1, None) == -6
    assert lib.m2_softplus_bias_fwd(None, 8, None, None, 8, 0, 8, 1, None) == 0       # no rows: nothing to do
    # one partial row of dw per workgroup of the backward (up to one per wave), one partial row of d_bias per 16 rows
    assert lib.m2_rmsnorm_gated_bwd_workspace_bytes(8192, 5120, 1, 1) >= 512 * 5120 * 4
    assert lib.m2_softplus_bias_bwd_workspace_bytes(8192, 80) >= (8192 // 16) * 80 * 4


def test_python_layer_has_no_cpu_fallback():
    from mamba2.conv1d_grouped import nki_conv1d
    from mamba2.mamba2_kernel import mamba2_kernel
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    with pytest.raises(RuntimeError, match="no CPU path"):
        nki_conv1d(torch.zeros(1, 8, 16), torch.zeros(8, 1, 4), None, "silu")
    with pytest.raises(RuntimeError, match="no CPU path"):
        mamba2_kernel(torch.zeros(1, 128, 2), torch.zeros(2), torch.zeros(1, 128, 2, 64), torch.zeros(1, 128, 1, 64),
                      torch.zeros(1, 128, 1, 64), torch.zeros(2))
    from mamba2 import glue
    with pytest.raises(RuntimeError, match="no CPU path"):
        glue.rmsnorm_gated_hip(torch.zeros(2, 64), None, torch.ones(64), 1, 1e-5)
    with pytest.raises(RuntimeError, match="no CPU path"):
        glue.softplus_bias_hip(torch.zeros(2, 3, 8), torch.zeros(8))
    with pytest.raises(RuntimeError, match="no CPU path"):
        mamba2_kernel_inference(torch.zeros(1, 1, 40), torch.zeros(1, 40, 3), torch.zeros(40, 4), torch.zeros(40),
                                torch.zeros(1, 2, 4, 16), torch.zeros(1, 1, 2), torch.zeros(2), torch.zeros(2))


def test_missing_library_fails_loudly(monkeypatch):
    from mamba2 import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmamba2_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "one GPU only" in r.stderr and r.stdout.strip() == ""


def test_f32_param_copy_is_kept_only_without_autograd():
    from mamba2 import _lib
    w = torch.nn.Parameter(torch.randn(8).bfloat16())
    with torch.no_grad():
        a, b = _lib.f32_param(w), _lib.f32_param(w)
        assert a is b and torch.equal(a, w.float())
        w.mul_(2)                                   # an in-place update (optimizer step, load_state_dict) is seen
        c = _lib.f32_param(w)
        assert c is not a and torch.equal(c, w.float())
    assert _lib.f32_param(w) is not c               # autograd on: converted per call
    f = torch.nn.Parameter(torch.randn(8))
    assert _lib.f32_param(f).data_ptr() == f.data_ptr()
