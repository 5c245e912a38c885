"""GPU: MFMA tile self-test, conv1d and decode-step parity against the CPU oracle (through the C ABI)."""
import math

import pytest
import torch

from conftest import rel_err, rel_rms_err
from oracle.conv import conv1d_grads_ref, conv1d_ref, make_conv_inputs
from oracle.decode import decode_step_ref, make_decode_inputs
from oracle.ssd import ssd_recurrent_ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tol(dtype):
    return (1e-4, rel_err) if dtype == torch.float32 else (2e-2, rel_rms_err)


# ----------------------------------------------------------------------------- MFMA layout
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_mfma_tile_selftest(lib, dtype):
    from mamba2 import _lib
    M, N, K = 256, 128, 96
    g = torch.Generator().manual_seed(0)
    A = torch.randn(M, K, generator=g).to(dtype).to(DEV)
    Bt = torch.randn(N, K, generator=g).to(dtype).to(DEV)
    Cm = torch.empty(M, N, dtype=torch.float32, device=DEV)
    _lib.check(lib.m2_mfma_selftest(_lib.ptr(A), _lib.ptr(Bt), _lib.ptr(Cm), M, N, K, _lib.dtype_code(dtype),
                                    _lib.stream_ptr()), "selftest")
    torch.cuda.synchronize()
    ref = A.double().cpu() @ Bt.double().cpu().T
    assert rel_err(Cm.cpu(), ref) < (1e-5 if dtype == torch.float32 else 1e-5)   # exact products, fp32 accumulation


# ----------------------------------------------------------------------------- memory probes
def test_stream_copy_and_tile_walk_are_exact(lib):
    """The measurement probes move bytes and nothing else: the copy is the identity, the tile walk a re-tiling."""
    from mamba2 import _lib
    batch, rows, row_bytes = 2, 384, 1024
    g = torch.Generator().manual_seed(5)
    src = torch.randint(0, 256, (batch, rows, row_bytes), generator=g, dtype=torch.uint8).to(DEV)
    dst = torch.zeros_like(src)
    _lib.check(lib.m2_stream_copy(_lib.ptr(src), _lib.ptr(dst), src.numel(), _lib.stream_ptr()), "copy")
    assert torch.equal(dst, src)
    for piece in (64, 128, 256, 512):
        units = row_bytes // piece
        want = src.view(batch, rows // 128, 128, units, piece).permute(0, 1, 3, 2, 4).contiguous().view(-1)
        for in_order in (1, 0):
            dst.zero_()
            _lib.check(lib.m2_tile_walk(_lib.ptr(src), _lib.ptr(dst), batch, rows, row_bytes, piece, in_order, _lib.stream_ptr()), "walk")
            assert torch.equal(dst.view(-1), want), (piece, in_order)
    assert lib.m2_tile_walk(_lib.ptr(src), _lib.ptr(dst), batch, rows, row_bytes, 96, 1, _lib.stream_ptr()) != 0      # refused, not run


# ----------------------------------------------------------------------------- conv1d
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b,l,C", [(2, 256, 512), (3, 100, 264), (1, 5, 8), (2, 33, 7), (1, 1, 64), (1, 2, 16), (1, 3, 16)])
@pytest.mark.parametrize("act", ["silu", None])
def test_conv_channels_last_fwd_bwd(dtype, b, l, C, act):
    from mamba2.conv1d_grouped import conv1d_backward, conv1d_forward
    d = make_conv_inputs(b, l, C, seed=l + C, dtype=dtype)
    y_ref, dx_ref, dw_ref, db_ref = conv1d_grads_ref(d["x"].double(), d["w"].double(), d["bias"].double(), d["dy"].double(), act)
    x, w, bias, dy = (d[k].to(DEV) for k in ("x", "w", "bias", "dy"))
    y = conv1d_forward(x, w, bias, act, channels_last=True)
    dx, dw, db = conv1d_backward(x, w, bias, dy, act, channels_last=True)
    tol, metric = _tol(dtype)
    assert metric(y, y_ref) < tol
    assert metric(dx, dx_ref) < tol
    assert metric(dw, dw_ref) < tol
    assert metric(db, db_ref) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_module_channel_major_autograd(dtype):
    # the reference's own parity recipe (conv1d_grouped.py:343-367): ConvNKI vs nn.Conv1d + silu, layout (B, D, L)
    from mamba2.conv1d_grouped import ConvNKI
    B, D, L, k = 2, 96, 200, 4
    d = make_conv_inputs(B, L, D, seed=3, dtype=dtype)
    x_bdl = d["x"].transpose(1, 2).contiguous()
    dy_bdl = d["dy"].transpose(1, 2).contiguous()
    y_ref, dx_ref, dw_ref, db_ref = conv1d_grads_ref(x_bdl.double(), d["w"].double(), d["bias"].double(), dy_bdl.double(),
                                                     "silu", channels_last=False)
    m = ConvNKI(D, D, k, groups=D, padding=k - 1, activation="silu").to(DEV, dtype)
    with torch.no_grad():
        m.weight.copy_(d["w"].to(DEV))
        m.bias.copy_(d["bias"].to(DEV))
    xin = x_bdl.to(DEV).requires_grad_(True)
    y = m(xin)
    y.backward(dy_bdl.to(DEV))
    tol, metric = _tol(dtype)
    assert metric(y, y_ref) < tol
    assert metric(xin.grad, dx_ref) < tol
    assert metric(m.weight.grad, dw_ref) < tol
    assert metric(m.bias.grad, db_ref) < tol


def test_conv_strided_views_and_no_bias():
    # x is a slice of a wider packed buffer (as xBC inside zxBCdt); outputs go to a strided destination too
    from mamba2.conv1d_grouped import conv1d_backward, conv1d_forward
    b, l, C, off, width = 2, 130, 64, 32, 160
    g = torch.Generator().manual_seed(5)
    big = torch.randn(b, l, width, generator=g).to(torch.bfloat16)
    w = (torch.rand(C, 1, 4, generator=g) - 0.5).to(torch.bfloat16)
    dy = torch.randn(b, l, C, generator=g).to(torch.bfloat16)
    xs = big[:, :, off:off + C]
    y_ref, dx_ref, dw_ref, _ = conv1d_grads_ref(xs.double(), w.double(), None, dy.double(), "silu")
    bigd = big.to(DEV)
    outbig = torch.zeros(b, l, width, dtype=torch.bfloat16, device=DEV)
    y = conv1d_forward(bigd[:, :, off:off + C], w.to(DEV), None, "silu", channels_last=True)
    dx, dw, db = conv1d_backward(bigd[:, :, off:off + C], w.to(DEV), None, dy.to(DEV), "silu", channels_last=True,
                                 out_dx=outbig[:, :, off:off + C])
    assert db is None
    assert rel_rms_err(y, y_ref) < 2e-2 and rel_rms_err(outbig[:, :, off:off + C], dx_ref) < 2e-2 and rel_rms_err(dw, dw_ref) < 2e-2
    assert outbig[:, :, :off].abs().max() == 0 and outbig[:, :, off + C:].abs().max() == 0


def test_conv_empty_and_errors():
    from mamba2.conv1d_grouped import conv1d_forward, nki_conv1d
    w = torch.zeros(8, 1, 4, device=DEV)
    y = conv1d_forward(torch.zeros(0, 16, 8, device=DEV), w, None, "silu", channels_last=True)
    assert y.shape == (0, 16, 8)
    y = conv1d_forward(torch.zeros(2, 0, 8, device=DEV), w, None, "silu", channels_last=True)
    assert y.shape == (2, 0, 8)
    with pytest.raises(ValueError):
        nki_conv1d(torch.zeros(1, 8, 16, device=DEV), w, None, "tanh")
    with pytest.raises(ValueError):
        conv1d_forward(torch.zeros(1, 16, 8, device=DEV), torch.zeros(8, 1, 9, device=DEV), None, None, channels_last=True)
    with pytest.raises(RuntimeError):
        conv1d_forward(torch.zeros(1, 16, 8), torch.zeros(8, 1, 4), None, None, channels_last=True)   # CPU tensors: no fallback


# ----------------------------------------------------------------------------- decode step
def _run_decode(d, g, W=None):
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    dd = {k: v.clone().to(DEV) for k, v in d.items()}
    y, cs, S = mamba2_kernel_inference(dd["xBC"], dd["conv_state"], dd["conv_weight"], dd["conv_bias"], dd["S"], dd["dt"],
                                       dd["A"], dd["D"], n_groups=g)
    assert cs.data_ptr() == dd["conv_state"].data_ptr() and S.data_ptr() == dd["S"].data_ptr()   # in place
    return y, cs, S


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b,h,p,n,g,W", [(2, 4, 8, 16, 1, 4), (3, 3, 6, 16, 1, 4), (1, 2, 4, 16, 1, 3), (2, 8, 64, 128, 2, 3),
                                         (2, 4, 16, 10, 2, 3), (4, 16, 64, 64, 8, 4)])
def test_decode_matches_oracle(dtype, b, h, p, n, g, W):
    d = make_decode_inputs(b, h, p, n, g, W=W, seed=b * 100 + h, act_dtype=dtype)
    dd = {k: v.double() for k, v in d.items()}
    y_ref, cs_ref, S_ref = decode_step_ref(dd["xBC"], dd["conv_state"], dd["conv_weight"], dd["conv_bias"], dd["S"], dd["dt"],
                                           dd["A"], dd["D"], n_groups=g)
    y, cs, S = _run_decode(d, g)
    tol, metric = _tol(dtype)
    assert metric(y, y_ref) < tol
    assert rel_err(S, S_ref) < 1e-5             # state is fp32 in both modes
    assert torch.equal(cs.cpu().double(), cs_ref)   # pure data movement: bit exact


def test_decode_zero_in_zero_out():
    # tests/mamba2_kernel_test_no_tp.py:62-105
    b, h, p, n, g = 1, 2, 4, 16, 1
    d = make_decode_inputs(b, h, p, n, g, W=4, seed=0)
    d = {k: torch.zeros_like(v) for k, v in d.items()}
    d["A"] = torch.full((h,), -1e-6)
    d["D"] = torch.full((h,), 1e-6)
    y, cs, S = _run_decode(d, g)
    assert y.abs().max() == 0 and cs.abs().max() == 0 and S.abs().max() == 0
    assert y.shape == (b, 1, h * p) and cs.shape == (b, h * p + 2 * g * n, 4) and S.shape == (b, h, p, n)


def test_decode_batch_row_consistency():
    # tests/mamba2_kernel_test_no_tp.py:108-148
    b, h, p, n, g = 3, 3, 6, 16, 1
    d = make_decode_inputs(1, h, p, n, g, W=4, seed=1)
    rep = lambda t: t.repeat(b, *([1] * (t.dim() - 1))) if t.dim() > 1 else t
    d = {k: (rep(v) if k in ("xBC", "conv_state", "S", "dt") else v) for k, v in d.items()}
    y, cs, S = _run_decode(d, g)
    for i in range(1, b):
        assert torch.equal(y[0], y[i]) and torch.equal(cs[0], cs[i]) and torch.equal(S[0], S[i])


def test_decode_steps_equal_conv_plus_recurrence():
    # the intent of tests/mamba2_kernel_test_no_tp.py:203-268: token-by-token decode == sequence path
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    b, h, p, n, g, l, W = 2, 4, 64, 64, 2, 40, 3
    d = make_decode_inputs(b, h, p, n, g, W=W, seed=4)
    gen = torch.Generator().manual_seed(8)
    Cx = h * p + 2 * g * n
    seq = torch.randn(b, l, Cx, generator=gen)
    dts = torch.exp(torch.empty(b, l, h).uniform_(math.log(1e-3), math.log(1e-1), generator=gen))
    conv_state = torch.zeros(b, Cx, W, device=DEV)
    S = torch.zeros(b, h, p, n, device=DEV)
    w, bias, A, D = (d[k].to(DEV) for k in ("conv_weight", "conv_bias", "A", "D"))
    ys = []
    for t in range(l):
        y, conv_state, S = mamba2_kernel_inference(seq[:, t:t + 1].to(DEV), conv_state, w, bias, S, dts[:, t:t + 1].to(DEV), A, D,
                                                   n_groups=g)
        ys.append(y.cpu())
    act = conv1d_ref(seq.double(), d["conv_weight"].double()[:, None, :], d["conv_bias"].double(), "silu")
    x, Bm, Cm = torch.split(act, [h * p, g * n, g * n], dim=-1)
    y_ref, S_ref = ssd_recurrent_ref(dts.double(), d["A"].double(), x.reshape(b, l, h, p), Bm.reshape(b, l, g, n),
                                     Cm.reshape(b, l, g, n), d["D"].double())
    assert rel_err(torch.cat(ys, 1), y_ref.reshape(b, l, -1)) < 1e-4
    assert rel_err(S, S_ref) < 1e-4
    assert torch.equal(conv_state.cpu(), seq[:, -W:].transpose(1, 2))
