"""GPU: SSD chunked scan forward/backward parity against the fp64 CPU oracle (through the C ABI)."""
import pytest
import torch

from conftest import rel_err, rel_rms_err
from oracle.ssd import make_ssd_inputs, ssd_chunked_ref, ssd_grads_ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tol(dtype):
    return (1e-4, rel_err) if dtype == torch.float32 else (2e-2, rel_rms_err)


def _dev(d):
    return {k: v.to(DEV) for k, v in d.items()}


def _f64(d):
    return {k: v.double() for k, v in d.items()}


CASES = [
    # b, l, h, p, n, g
    (1, 256, 8, 64, 64, 1),      # the fp32 correctness configuration
    (2, 384, 4, 64, 128, 2),
    (1, 200, 2, 128, 64, 1),     # ragged length, p = 128
    (2, 128, 4, 128, 128, 4),
    (1, 77, 2, 64, 128, 1),      # shorter than one chunk
    (1, 640, 2, 128, 128, 2),    # p = 128 over an odd number of chunks (the state pass peels one off)
    (1, 512, 4, 128, 64, 1),     # p = 128, n = 64 over an even number
    (2, 896, 4, 64, 64, 2),      # n = 64: two-wave state pass, seven chunks
    (2, 2000, 8, 64, 64, 8),     # 256 (batch, chunk, group) triples: the group finish takes both sides per workgroup; ragged
    (3, 1, 2, 64, 128, 1),       # a single token
    (2, 17, 5, 64, 64, 1),       # 17 tokens, an odd head count in one group
    (1, 300, 10, 64, 128, 2),    # five heads per group
    (3, 129, 10, 128, 128, 2),   # one token into the second chunk, p = 128
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b,l,h,p,n,g", CASES)
def test_ssd_forward(dtype, b, l, h, p, n, g):
    from mamba2.mamba2_kernel import mamba2_kernel
    d = make_ssd_inputs(b, l, h, p, n, g, seed=l, dtype=dtype)
    r = _f64(d)
    y_ref, S_ref = ssd_chunked_ref(r["dt"], r["A"], r["X"], r["B"], r["C"], r["D"], chunk=64)
    dd = _dev(d)
    y, S = mamba2_kernel(dd["dt"], dd["A"], dd["X"], dd["B"], dd["C"], dd["D"], return_final_state=True)
    tol, metric = _tol(dtype)
    assert y.dtype == dtype and S.dtype == torch.float32
    assert metric(y, y_ref) < tol, "y"
    assert metric(S, S_ref) < tol, "final state"
    # without the final state the scan takes the one-tile form of the state pass (bf16 operand rounding of the decay-scaled
    # rows): the states entering the chunks differ in their last bit here and there, y stays within the same bar
    y2 = mamba2_kernel(dd["dt"], dd["A"], dd["X"], dd["B"], dd["C"], dd["D"])
    assert metric(y2, y_ref) < tol, "y without the final state"
    assert (y2.float() - y.float()).abs().max() <= 2 ** -6 * y.float().abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_forward_initial_state_no_D_fp32_dt(dtype):
    from mamba2.mamba2_kernel import mamba2_kernel
    b, l, h, p, n, g = 2, 300, 4, 64, 64, 2
    d = make_ssd_inputs(b, l, h, p, n, g, seed=9, dtype=dtype)
    d["dt"] = d["dt"].float()                                  # fp32 dt next to bf16 activations
    S0 = 0.1 * torch.randn(b, h, p, n, generator=torch.Generator().manual_seed(3))
    r = _f64(d)
    y_ref, S_ref = ssd_chunked_ref(r["dt"], r["A"], r["X"], r["B"], r["C"], None, initial_state=S0.double(), chunk=128)
    dd = _dev(d)
    y, S = mamba2_kernel(dd["dt"], dd["A"], dd["X"], dd["B"], dd["C"], None, initial_state=S0.to(DEV), return_final_state=True)
    if dtype == torch.float32:
        assert rel_err(y, y_ref) < 1e-4 and rel_err(S, S_ref) < 1e-4
    else:
        # without the D x skip the outputs are heavy-tailed (max |y| ~ 25 RMS here: a few tokens with large steps tower over
        # the rest): raw figure against 2e-2 + the bf16 storage floor, with a relative L2 error under 1e-2
        assert rel_rms_err(y, y_ref, name="y (no D, initial state)") < 2e-2
        assert rel_rms_err(S, S_ref, name="final state (initial state)") < 2e-2


def test_ssd_packed_views():
    # x, B, C as views into one packed [x | B | C] buffer, as the mixer passes them (mamba2_kernel.py:109-115,151)
    from mamba2.mamba2_kernel import mamba2_kernel
    b, l, h, p, n, g = 2, 256, 4, 64, 64, 2
    d = make_ssd_inputs(b, l, h, p, n, g, seed=2, dtype=torch.bfloat16)
    packed = torch.cat([d["X"].reshape(b, l, -1), d["B"].reshape(b, l, -1), d["C"].reshape(b, l, -1)], dim=-1).to(DEV)
    X = packed[..., :h * p].unflatten(-1, (h, p))
    Bm = packed[..., h * p:h * p + g * n].unflatten(-1, (g, n))
    Cm = packed[..., h * p + g * n:].unflatten(-1, (g, n))
    assert not X.is_contiguous()
    dd = _dev(d)
    y = mamba2_kernel(dd["dt"], dd["A"], X, Bm, Cm, dd["D"])
    y2 = mamba2_kernel(dd["dt"], dd["A"], dd["X"], dd["B"], dd["C"], dd["D"])
    assert torch.equal(y, y2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b,l,h,p,n,g", [(2, 255, 6, 64, 128, 2), (1, 511, 3, 128, 64, 1)])
def test_ssd_packed_views_with_pad_columns_fwd_bwd(dtype, b, l, h, p, n, g):
    # x, B, C (and their gradients) as column slices of buffers that are 8 columns wider than [x | B | C]: row pitches that
    # are not the packed width, every gradient written in place, the pad columns left alone; initial state and the
    # gradient of the final state included
    from mamba2.mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward
    d = make_ssd_inputs(b, l, h, p, n, g, seed=b + l, dtype=dtype)
    gen = torch.Generator().manual_seed(l)
    # (states of the size the scan itself builds up: larger ones make the first chunk's gradients tower over the rest)
    S0, dSf = 0.02 * torch.randn(b, h, p, n, generator=gen), 0.02 * torch.randn(b, h, p, n, generator=gen)
    r = _f64(d)
    ref = ssd_grads_ref(r["dt"], r["A"], r["X"], r["B"], r["C"], r["D"], r["dy"], chunk=64, initial_state=S0.double(), d_final_state=dSf.double())
    dv = _dev(d)
    W = h * p + 2 * g * n + 8

    def views(buf):
        return (buf[..., :h * p].unflatten(-1, (h, p)), buf[..., h * p:h * p + g * n].unflatten(-1, (g, n)),
                buf[..., h * p + g * n:h * p + 2 * g * n].unflatten(-1, (g, n)))

    buf = torch.zeros(b, l, W, dtype=dtype, device=DEV)
    X, Bm, Cm = views(buf)
    X.copy_(dv["X"]); Bm.copy_(dv["B"]); Cm.copy_(dv["C"])
    gbuf = torch.full((b, l, W), 3.0, dtype=dtype, device=DEV)
    dXv, dBv, dCv = views(gbuf)
    st = alloc_chunk_states(dv["dt"], dv["A"], X, Bm, Cm)
    y, S = ssd_forward(dv["dt"], dv["A"], X, Bm, Cm, dv["D"], initial_state=S0.to(DEV), want_final_state=True, chunk_states=st)
    out = ssd_backward(dv["dt"], dv["A"], X, Bm, Cm, dv["D"], dv["dy"], initial_state=S0.to(DEV), d_final_state=dSf.to(DEV),
                       want_dinitial=True, chunk_states=st, out_dX=dXv, out_dB=dBv, out_dC=dCv)
    got = {"y": y, "final_state": S, "ddt": out[0], "dA": out[1], "dX": dXv, "dB": dBv, "dC": dCv, "dD": out[5], "dinitial_state": out[6]}
    tol, metric = _tol(dtype)
    for k, v in got.items():
        e = metric(v, ref[k])
        assert e < tol, f"{k}: {e}"
    assert torch.equal(gbuf[..., W - 8:], torch.full((b, l, 8), 3.0, dtype=dtype, device=DEV))


def test_ssd_special_cases():
    from mamba2.mamba2_kernel import mamba2_kernel
    b, l, h, p, n, g = 3, 256, 4, 64, 64, 1
    d = _dev(make_ssd_inputs(1, l, h, p, n, g, seed=6))
    rep = lambda t: t.repeat(b, *([1] * (t.dim() - 1)))
    # batch-row consistency
    y, S = mamba2_kernel(rep(d["dt"]), d["A"], rep(d["X"]), rep(d["B"]), rep(d["C"]), d["D"], return_final_state=True)
    assert torch.equal(y[0], y[1]) and torch.equal(y[0], y[2]) and torch.equal(S[0], S[2])
    # zero in -> zero out;  B = C = 0 -> y = D x
    z = torch.zeros_like(d["X"])
    y, S = mamba2_kernel(d["dt"], d["A"], z, d["B"], d["C"], d["D"], return_final_state=True)
    assert y.abs().max() == 0 and S.abs().max() == 0
    zb = torch.zeros_like(d["B"])
    y = mamba2_kernel(d["dt"], d["A"], d["X"], zb, zb, d["D"])
    assert torch.allclose(y, d["D"][None, None, :, None] * d["X"], atol=1e-6)
    # empty
    y, S = mamba2_kernel(d["dt"][:, :0], d["A"], d["X"][:, :0], d["B"][:, :0], d["C"][:, :0], d["D"], return_final_state=True)
    assert y.shape == (1, 0, h, p) and S.abs().max() == 0


def test_ssd_rejects_unsupported():
    from mamba2.mamba2_kernel import mamba2_kernel
    d = _dev(make_ssd_inputs(1, 128, 2, 32, 64, 1, seed=0))
    with pytest.raises(ValueError, match="headdim"):
        mamba2_kernel(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"])
    d = make_ssd_inputs(1, 128, 2, 64, 64, 1, seed=0)
    with pytest.raises(RuntimeError, match="no CPU path"):
        mamba2_kernel(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"])


def test_ssd_rejects_token_strides_beyond_the_offset_arithmetic():
    """The kernels form row offsets inside a chunk with 24-bit multiplies and 32-bit sums: a token stride of 2^21 elements or
    more is refused by the library before anything is launched (checked straight through the C ABI: no tensor has such a stride)."""
    from mamba2 import _lib
    from mamba2._lib import SsdParams, ptr
    from mamba2.mamba2_kernel import _fill_common, _strides3
    d = _dev(make_ssd_inputs(1, 128, 2, 64, 64, 1, seed=0, dtype=torch.bfloat16))
    lib = _lib.load()
    Y = torch.empty_like(d["X"])
    p = SsdParams()
    _fill_common(p, d["dt"], d["A"].float(), d["X"], d["B"], d["C"], None)
    p.y = ptr(Y)
    p.y_stride_b, p.y_stride_l, p.y_stride_h = _strides3(Y)
    ws = torch.empty(lib.m2_ssd_fwd_workspace_bytes(p), dtype=torch.uint8, device=DEV)
    p.workspace, p.workspace_bytes = ptr(ws), ws.numel()
    p.x_stride_l = 1 << 21
    rc = lib.m2_ssd_fwd(p, _lib.stream_ptr(torch.device(DEV)))
    assert rc == -1 and b"token strides" in lib.m2_last_error()      # M2_ERR_SHAPE
    p.x_stride_l = d["X"].stride(1)
    assert lib.m2_ssd_fwd(p, _lib.stream_ptr(torch.device(DEV))) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b,l,h,p,n,g", CASES)
def test_ssd_backward(dtype, b, l, h, p, n, g):
    from mamba2.mamba2_kernel import mamba2_kernel
    d = make_ssd_inputs(b, l, h, p, n, g, seed=l + 1, dtype=dtype)
    r = _f64(d)
    ref = ssd_grads_ref(r["dt"], r["A"], r["X"], r["B"], r["C"], r["D"], r["dy"], chunk=64)
    dd = _dev(d)
    leaves = {k: dd[k].clone().requires_grad_(True) for k in ("dt", "A", "X", "B", "C", "D")}
    y = mamba2_kernel(leaves["dt"], leaves["A"], leaves["X"], leaves["B"], leaves["C"], leaves["D"])
    y.backward(dd["dy"])
    tol, metric = _tol(dtype)
    for name, key in (("dX", "X"), ("ddt", "dt"), ("dA", "A"), ("dB", "B"), ("dC", "C"), ("dD", "D")):
        e = metric(leaves[key].grad, ref[name])
        assert e < tol, f"{name}: {e}"
    assert leaves["X"].grad.dtype == dtype and leaves["dt"].grad.dtype == dtype and leaves["A"].grad.dtype == torch.float32


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_backward_states(dtype):
    # gradient through the final state and into the initial state
    from mamba2.mamba2_kernel import mamba2_kernel
    b, l, h, p, n, g = 2, 300, 4, 64, 64, 2
    d = make_ssd_inputs(b, l, h, p, n, g, seed=12, dtype=dtype)
    gen = torch.Generator().manual_seed(4)
    S0 = 0.1 * torch.randn(b, h, p, n, generator=gen)
    dS = torch.randn(b, h, p, n, generator=gen)
    r = _f64(d)
    ref = ssd_grads_ref(r["dt"], r["A"], r["X"], r["B"], r["C"], r["D"], r["dy"], initial_state=S0.double(),
                        d_final_state=dS.double(), chunk=128)
    dd = _dev(d)
    leaves = {k: dd[k].clone().requires_grad_(True) for k in ("dt", "A", "X", "B", "C", "D")}
    S0d = S0.to(DEV).requires_grad_(True)
    y, S = mamba2_kernel(leaves["dt"], leaves["A"], leaves["X"], leaves["B"], leaves["C"], leaves["D"], initial_state=S0d,
                         return_final_state=True)
    torch.autograd.backward([y, S], [dd["dy"], dS.to(DEV)])
    tol, metric = _tol(dtype)
    for name, key in (("dX", "X"), ("ddt", "dt"), ("dA", "A"), ("dB", "B"), ("dC", "C"), ("dD", "D")):
        e = metric(leaves[key].grad, ref[name])
        assert e < tol, f"{name}: {e}"
    assert metric(S0d.grad, ref["dinitial_state"]) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ssd_backward_kept_chunk_states_equal_recompute(dtype):
    # the backward handed the forward's chunk states must give exactly what the recomputing backward gives
    from mamba2.mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward
    b, l, h, p, n, g = 2, 300, 4, 64, 128, 2
    d = _dev(make_ssd_inputs(b, l, h, p, n, g, seed=21, dtype=dtype))
    S0 = 0.1 * torch.randn(b, h, p, n, generator=torch.Generator().manual_seed(5)).to(DEV)
    states = alloc_chunk_states(d["dt"], d["A"], d["X"], d["B"], d["C"])
    assert states.dtype == torch.uint8 and states.numel() >= b * 3 * h * p * n * d["X"].element_size()
    y1, _ = ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], S0, chunk_states=states)
    y0, _ = ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], S0)
    assert torch.equal(y0, y1)
    first = states[:b * 3 * h * p * n * d["X"].element_size()].view(dtype).view(b, 3, h, p, n)
    assert torch.equal(first[:, 0].float(), S0.to(dtype).float())      # the state entering chunk 0 is the initial state
    g0 = ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], d["dy"], S0, want_dinitial=True)
    g1 = ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], d["dy"], S0, want_dinitial=True, chunk_states=states)
    for a_, b_ in zip(g0, g1):
        assert torch.equal(a_, b_)
    with pytest.raises(ValueError, match="chunk_states"):
        ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], d["dy"], chunk_states=states[:-256].contiguous())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b,l,h,p,n,g", [(2, 384, 4, 64, 128, 2), (1, 200, 2, 128, 64, 1), (1, 77, 8, 64, 64, 1)])
def test_ssd_softplus_folded_into_scan(dtype, b, l, h, p, n, g):
    """dt_bias given: dt is the raw projection, the step size softplus(dt + dt_bias) is formed inside the scan, the
    backward returns the gradient of the raw dt and d_dt_bias (fused_kernel.py:33-73, 273, 338)."""
    from mamba2.mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward
    from oracle.mixer import softplus_ref
    tol, err = _tol(dtype)
    d = make_ssd_inputs(b, l, h, p, n, g, seed=l + 7, dtype=dtype)
    gen = torch.Generator().manual_seed(l)
    # raw dt as the last h columns of a wider buffer; values on both sides of the softplus threshold
    raw = (torch.randn(b, l, 24 + h, generator=gen) * 1.5).to(dtype)
    if dtype == torch.float32:
        raw[0, : l // 8, 24] = 12.0          # beyond the threshold (in bf16 such steps, 100 x the usual size, only test the error metric)
    bias = torch.empty(h).uniform_(-4.0, -1.0, generator=gen)
    r = _f64(d)
    dt_raw = raw[..., 24:].double().requires_grad_(True)
    bias_d = bias.double().requires_grad_(True)
    lv = {k: r[k].clone().requires_grad_(True) for k in ("A", "X", "B", "C", "D")}
    y_ref, _ = ssd_chunked_ref(softplus_ref(dt_raw + bias_d), lv["A"], lv["X"], lv["B"], lv["C"], lv["D"], chunk=64)
    y_ref.backward(r["dy"])
    g_ = _dev(d)
    rawg = raw.to(DEV)
    dtv = rawg[..., 24:]
    st = alloc_chunk_states(dtv, g_["A"], g_["X"], g_["B"], g_["C"])
    y, _ = ssd_forward(dtv, g_["A"], g_["X"], g_["B"], g_["C"], g_["D"], chunk_states=st, dt_bias=bias.to(DEV))
    assert err(y.cpu(), y_ref.detach()) < tol
    gbuf = torch.full((b, l, 24 + h), 5.0, dtype=dtype, device=DEV)
    for states in (st, None):        # with the forward's tables, and recomputing them (softplus applied again there)
        ddt, dA, dX, dB, dC, dD, _, dbias = ssd_backward(dtv, g_["A"], g_["X"], g_["B"], g_["C"], g_["D"], g_["dy"], chunk_states=states,
                                                          dt_bias=bias.to(DEV), out_ddt=gbuf[..., 24:])
        assert ddt.data_ptr() == gbuf[..., 24:].data_ptr()
        if dtype == torch.float32:
            assert err(ddt.cpu(), dt_raw.grad) < tol
        else:
            # stored in bf16, and heavy-tailed here (the tokens with step sizes beyond the threshold): a bf16 value just
            # above a power of two is off by up to 2^-8 of itself from storage alone, which roundings=2 discounts
            assert rel_rms_err(ddt.cpu(), dt_raw.grad) < tol
        # a signed sum over all b * l tokens of ddt terms that are each within the tolerance: a few times the element bound
        assert err(dbias.cpu(), bias_d.grad) < (5e-4 if dtype == torch.float32 else tol)
        assert err(dX.cpu(), lv["X"].grad) < tol
        # dA, like d_dt_bias, is a signed sum over all tokens (here with step sizes from 1e-2 up to 11, beyond the threshold)
        assert err(dA.cpu(), lv["A"].grad) < (5e-4 if dtype == torch.float32 else tol)
        assert torch.equal(gbuf[..., :24], torch.full((b, l, 24), 5.0, dtype=dtype, device=DEV))
