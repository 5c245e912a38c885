"""GPU parity of the mixer glue kernels (m2_softplus_bias_*, m2_rmsnorm_gated_*) against the fp64 oracle
(oracle/mixer.py: softplus_ref, rmsnorm_gated_ref; backward = autograd through the oracle).

Shapes: the group widths of the reference's configurations (2.7B: 5120 channels in one group; 7B: 8192 in 8 groups of
1024; 370M-like 2048), ragged widths (not a multiple of 64 vectors), row counts that do not fill the last block, column
slices of a packed [z | xBC | dt] buffer, no gate.  Tolerances: fp32 1e-4 relative to RMS; bf16 2e-2 x RMS.
"""
import pytest
import torch

from conftest import rel_rms_err
from oracle.mixer import rmsnorm_gated_ref, softplus_ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("b,l,h", [(2, 100, 4), (4, 2048, 80), (1, 1, 128), (3, 77, 24)])
def test_softplus_bias_fwd_bwd(dtype, b, l, h):
    from mamba2 import glue
    # dt as the last h columns of a wider buffer (the packed projection output), values on both sides of the threshold
    width = 40 + h
    buf = _rand((b, l, width), dtype, 1, scale=6.0)
    bias = _rand((h,), torch.float32, 2)
    dt = buf.to(DEV)[..., 40:]
    out = glue.softplus_bias_hip(dt, bias.to(DEV))
    ref = softplus_ref(buf[..., 40:].double() + bias.double())
    assert out.shape == (b, l, h) and out.dtype == dtype and out.is_contiguous()
    assert rel_rms_err(out.cpu(), ref) < TOL[dtype]
    # backward into a column slice of a gradient buffer
    d_out = _rand((b, l, h), dtype, 3)
    gbuf = torch.full((b, l, width), 7.0, dtype=dtype, device=DEV)
    d_in, d_bias = glue.softplus_bias_bwd_hip(dt, bias.to(DEV), d_out.to(DEV), out_d_in=gbuf[..., 40:])
    v = (buf[..., 40:].double() + bias.double()).requires_grad_(True)
    softplus_ref(v).backward(d_out.double())
    # the kernel takes the derivative above the threshold as exactly 1 (sigmoid(10) = 1 - 4.5e-5)
    assert rel_rms_err(d_in.cpu(), v.grad) < TOL[dtype] + 1e-4
    assert rel_rms_err(d_bias.cpu(), v.grad.sum(dim=(0, 1))) < (1e-4 if dtype == torch.float32 else 2e-3)
    assert torch.equal(gbuf[..., :40], torch.full((b, l, 40), 7.0, dtype=dtype, device=DEV))      # neighbours untouched
    assert d_bias.dtype == torch.float32


NORM_SHAPES = [
    # rows (b, l), channels, groups
    ((2, 96), 5120, 1),        # 2.7B: one group of 5120 (four waves per row, 2.5 vectors per lane)
    ((1, 130), 8192, 8),       # 7B: eight groups of 1024 (one wave per row and group)
    ((2, 37), 2048, 1),        # one wave, four vectors per lane
    ((1, 50), 256, 2),         # groups of 128: 16 vectors, most lanes idle
    ((3, 5), 4160, 1),         # 520 vectors: ragged over 256 threads
    ((1, 3), 8192, 1),         # the widest supported group
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,d,g", NORM_SHAPES)
@pytest.mark.parametrize("gated", [True, False])
def test_rmsnorm_gated_fwd_bwd(dtype, rows, d, g, gated):
    from mamba2 import glue
    eps = 1e-5
    x = _rand((*rows, d), dtype, 11)
    z = _rand((*rows, d), dtype, 12) if gated else None
    w = 1.0 + 0.2 * _rand((d,), torch.float32, 13)
    dout = _rand((*rows, d), dtype, 14)
    xg, wg, dg = x.to(DEV), w.to(DEV), dout.to(DEV)
    zg = z.to(DEV) if gated else None
    xd = x.double().requires_grad_(True)
    zd = z.double().requires_grad_(True) if gated else None
    wd = w.double().requires_grad_(True)
    ref = rmsnorm_gated_ref(xd, zd, wd, g, eps)
    ref.backward(dout.double())
    # fp32 output: nothing is rounded on the way out, so the bound is the fp32 one whatever the input type
    out32 = glue.rmsnorm_gated_hip(xg, zg, wg, g, eps, out_dtype=torch.float32)
    assert out32.dtype == torch.float32 and out32.shape == x.shape
    assert rel_rms_err(out32.cpu(), ref.detach()) < 1e-4
    # output in the input type: the same values, rounded once
    out = glue.rmsnorm_gated_hip(xg, zg, wg, g, eps, out_dtype=dtype)
    assert out.dtype == dtype and torch.equal(out, out32.to(dtype))
    dx, dw, dz = glue.rmsnorm_gated_bwd_hip(xg, zg, wg, dg, g, eps)
    # dx, dz are stored in the input type.  h = x silu(z) is heavy-tailed (elements beyond 10 RMS), and a bf16 value just
    # above a power of two is off by up to 2^-8 of itself from storage alone: roundings=2 discounts that worst case
    # instead of the 2^-9 best case, the arithmetic (fp32 throughout) must stay inside the tolerance
    assert rel_rms_err(dx.cpu(), xd.grad) < TOL[dtype]
    if gated:
        assert rel_rms_err(dz.cpu(), zd.grad) < TOL[dtype]
    else:
        assert dz is None
    # dw is an fp32 sum over the rows of products of the (bf16) inputs: the inputs are exact, the sum is not rounded to bf16
    assert rel_rms_err(dw.cpu(), wd.grad) < 1e-4 if dtype == torch.float32 else rel_rms_err(dw.cpu(), wd.grad) < 2e-3
    assert dw.dtype == torch.float32


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width_pad", [0, 4])     # 4: rows of the packed buffer are not 16-byte aligned
def test_rmsnorm_gated_on_packed_views(dtype, width_pad):
    """z and dz as the first d columns of a packed (b, l, d + extra) buffer, as the fused mixer core passes them."""
    from mamba2 import glue
    b, l, d, g, eps = 2, 64, 512, 2, 1e-5
    extra = 136 + width_pad
    packed = _rand((b, l, d + extra), dtype, 21).to(DEV)
    z = packed[..., :d]
    x = _rand((b, l, d), dtype, 22).to(DEV)
    w = (1.0 + 0.1 * _rand((d,), torch.float32, 23)).to(DEV)
    dout = _rand((b, l, d), dtype, 24).to(DEV)
    out = glue.rmsnorm_gated_hip(x, z, w, g, eps, out_dtype=dtype)
    out_c = glue.rmsnorm_gated_hip(x, z.contiguous(), w, g, eps, out_dtype=dtype)
    assert torch.equal(out, out_c)
    gpacked = torch.full((b, l, d + extra), 3.0, dtype=dtype, device=DEV)
    dx, dw, dz = glue.rmsnorm_gated_bwd_hip(x, z, w, dout, g, eps, out_dz=gpacked[..., :d])
    dx_c, dw_c, dz_c = glue.rmsnorm_gated_bwd_hip(x, z.contiguous(), w, dout, g, eps)
    assert torch.equal(dx, dx_c) and torch.equal(dw, dw_c) and torch.equal(gpacked[..., :d], dz_c)
    assert torch.equal(gpacked[..., d:], torch.full((b, l, extra), 3.0, dtype=dtype, device=DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,d", [(128, 2560), (3, 4096), (1, 8192), (130, 100), (5, 1028)])
def test_add_rmsnorm_in_place_residual(dtype, rows, d):
    """residual += delta; out = w * residual * rsqrt(mean(residual^2) + eps): against the fp64 oracle norm of the fp64 sum."""
    from mamba2 import glue
    eps = 1e-5
    res = _rand((rows, d), torch.float32, 31, scale=3.0)
    delta = _rand((rows, d), dtype, 32)
    w = 1.0 + 0.2 * _rand((d,), torch.float32, 33)
    rg = res.to(DEV)
    out = glue.add_rmsnorm_(rg, delta.to(DEV), w.to(DEV), eps, dtype)
    s = res.double() + delta.double()
    ref = rmsnorm_gated_ref(s, None, w.double(), 1, eps)
    assert out.dtype == dtype and out.shape == (rows, d)
    assert rel_rms_err(rg.cpu(), s) < 1e-6                     # the residual stream stays fp32
    assert rel_rms_err(out.cpu(), ref) < TOL[dtype]
    # nothing to add: the residual is left alone
    before = rg.clone()
    out2 = glue.add_rmsnorm_(rg, None, w.to(DEV), eps, dtype)
    assert torch.equal(rg, before) and torch.equal(out2, out)
    with pytest.raises(ValueError):
        glue.add_rmsnorm_(torch.zeros(2, 8200, device=DEV), None, torch.ones(8200, device=DEV), eps, dtype)


def test_glue_empty_and_errors():
    from mamba2 import glue
    x = torch.empty(0, 4, 512, dtype=torch.bfloat16, device=DEV)
    w = torch.ones(512, device=DEV)
    assert glue.rmsnorm_gated_hip(x, x, w, 1, 1e-5).shape == (0, 4, 512)
    dx, dw, dz = glue.rmsnorm_gated_bwd_hip(x, x, w, x, 1, 1e-5)
    assert dx.shape == x.shape and torch.equal(dw, torch.zeros(512, device=DEV))
    dt = torch.empty(0, 3, 8, dtype=torch.bfloat16, device=DEV)
    d_in, d_bias = glue.softplus_bias_bwd_hip(dt, torch.zeros(8, device=DEV), dt)
    assert torch.equal(d_bias, torch.zeros(8, device=DEV))
    with pytest.raises(ValueError):      # group wider than the kernels hold in registers
        glue.rmsnorm_gated_hip(torch.zeros(2, 16384, dtype=torch.bfloat16, device=DEV), None, torch.ones(16384, device=DEV), 1, 1e-5)
    with pytest.raises(ValueError):      # channels per group not a multiple of the vector width
        glue.rmsnorm_gated_hip(torch.zeros(2, 36, dtype=torch.bfloat16, device=DEV), None, torch.ones(36, device=DEV), 3, 1e-5)
    with pytest.raises(RuntimeError):    # no CPU path
        glue.rmsnorm_gated_hip(torch.zeros(2, 64), None, torch.ones(64), 1, 1e-5)
