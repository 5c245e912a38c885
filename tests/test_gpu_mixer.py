"""GPU: fused mixer core (zxBCdt -> norm_out) and the Mamba2Mixer module against the CPU oracle."""
import pytest
import torch

from conftest import raw_rms_err, rel_err, rel_rms_err
from oracle.mixer import fused_core_ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _fused_inputs(b, l, h, p, n, g, dtype, seed=0):
    gen = torch.Generator().manual_seed(seed)
    d_inner = h * p
    width = 2 * d_inner + 2 * g * n + h
    t = {
        "zxBCdt": torch.randn(b, l, width, generator=gen).to(dtype),
        "A": -torch.exp(torch.empty(h).uniform_(0.0, 2.77, generator=gen)),
        "D": torch.ones(h) + 0.1 * torch.randn(h, generator=gen),
        "conv_w": (torch.rand(d_inner + 2 * g * n, 1, 4, generator=gen) - 0.5).to(dtype),
        "conv_b": (torch.rand(d_inner + 2 * g * n, generator=gen) - 0.5).to(dtype),
        "dt_bias": torch.empty(h).uniform_(-5.0, -2.0, generator=gen),      # softplus -> dt in ~[7e-3, 0.13]
        "norm_w": 1.0 + 0.1 * torch.randn(d_inner, generator=gen),
        "dout": torch.randn(b, l, d_inner, generator=gen).to(dtype),
    }
    # scale the B and C columns like the scan configuration (N(0,1)/sqrt(n)) so the state terms stay O(1)
    t["zxBCdt"][..., 2 * d_inner:2 * d_inner + 2 * g * n] /= n ** 0.5
    return t


class _RoundBF16(torch.autograd.Function):
    """Value and gradient both pass through a bfloat16 store (round to nearest even)."""

    @staticmethod
    def forward(ctx, x):
        return x.bfloat16().to(x.dtype)

    @staticmethod
    def backward(ctx, g):
        return g.bfloat16().to(g.dtype)


def _oracle(t, g, n, d_inner, p, handover=None):
    leaves = {k: t[k].double().clone().requires_grad_(True) for k in ("zxBCdt", "A", "D", "conv_w", "conv_b", "dt_bias", "norm_w")}
    zin = leaves["zxBCdt"] if handover is None else handover(leaves["zxBCdt"])   # identity on values, rounds the gradient
    out = fused_core_ref(zin, leaves["A"], leaves["D"], leaves["conv_w"], leaves["conv_b"], leaves["dt_bias"],
                         leaves["norm_w"], g, n, d_inner, p, handover=handover)
    out.backward(t["dout"].double())
    return out.detach(), {k: v.grad for k, v in leaves.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("caching", [False, True])
@pytest.mark.parametrize("b,l,h,p,n,g", [(2, 256, 4, 64, 64, 2), (1, 200, 2, 64, 128, 1)])
def test_fused_kernel_fwd_bwd(dtype, caching, b, l, h, p, n, g):
    from mamba2.fused_kernel import mamba2_fused_kernel, mamba2_fused_kernel_with_caching
    fn = mamba2_fused_kernel_with_caching if caching else mamba2_fused_kernel
    d_inner = h * p
    t = _fused_inputs(b, l, h, p, n, g, dtype, seed=l + h)
    ref_out, ref_g = _oracle(t, g, n, d_inner, p)
    lv = {k: t[k].to(DEV).clone().requires_grad_(True) for k in ("zxBCdt", "A", "D", "conv_w", "conv_b", "dt_bias", "norm_w")}
    out = fn(lv["zxBCdt"], lv["A"], lv["D"], lv["conv_w"], lv["conv_b"], lv["dt_bias"], lv["norm_w"], g, n, d_inner, p)
    out.backward(t["dout"].to(DEV))
    assert out.dtype == dtype and out.shape == (b, l, d_inner)
    parts = [d_inner, d_inner, g * n, g * n, h]       # the packed gradient holds quantities of different scale
    names = ("dz", "dx", "dB", "dC", "ddt")

    def quantities(out_, grads):
        q = {"norm_out": out_}
        q.update(dict(zip(names, torch.split(grads["zxBCdt"], parts, dim=-1))))
        q.update({"d" + k: grads[k] for k in ("A", "D", "conv_w", "conv_b", "dt_bias", "norm_w")})
        return q

    got = quantities(out, {k: v.grad for k, v in lv.items()})
    ref = quantities(ref_out, ref_g)
    if dtype == torch.float32:
        for k in got:
            assert rel_err(got[k], ref[k]) < 1e-4, k
        return
    # bf16.  Each kernel alone is held to 2e-2 x RMS by its own test.  The chain hands bf16 tensors from stage to
    # stage (conv output, scan output, norm output; the gradients cross the same points in reverse), and rounding
    # those hand-overs alone -- all arithmetic exact -- already costs 4e-2..1e-1 x RMS in the max norm on these
    # heavy-tailed tensors.  That floor is measured here: the same fp64 oracle with a bf16 round at each hand-over
    # gives the error no implementation with the reference's storage types can avoid.  The bar: raw error <= 2e-2 x RMS
    # + that floor (+ the storage floor of the result itself), and <= 1e-2 in relative L2 error, which outliers do
    # not dominate.
    floor_out, floor_g = _oracle(t, g, n, d_inner, p, handover=_RoundBF16.apply)
    floor = quantities(floor_out, floor_g)
    for k in got:
        e_floor = raw_rms_err(floor[k], ref[k])
        e = rel_rms_err(got[k], ref[k], name=k, extra_floor=e_floor)
        assert e < 2e-2, f"{k}: {e} above the hand-over floor {e_floor}"
        l2 = ((got[k].double().cpu() - ref[k]).norm() / ref[k].norm()).item()
        assert l2 < 1e-2, f"{k}: relative L2 error {l2}"


def _mixer(dtype, g=2, layer_idx=0):
    from mamba2.configuration_mamba2 import Mamba2Config
    from mamba2.mamba2_mixer import Mamba2Mixer
    cfg = Mamba2Config(num_heads=4, head_dim=64, hidden_size=128, state_size=64, n_groups=g, num_hidden_layers=2, expand=2)
    torch.manual_seed(0)
    m = Mamba2Mixer(cfg, layer_idx).to(DEV)
    with torch.no_grad():
        m.in_proj.weight.normal_(0, 0.05)
        m.out_proj.weight.normal_(0, 0.05)
        m.A_log.copy_(torch.log(torch.linspace(1.0, 8.0, cfg.num_heads)))
    return cfg, m.to(dtype) if dtype != torch.float32 else m


def test_mixer_parameter_names_and_shapes():
    cfg, m = _mixer(torch.float32)
    names = dict(m.named_parameters())
    d_inner, conv_dim = 256, 256 + 2 * 2 * 64
    assert names["conv1d.weight"].shape == (conv_dim, 1, 4) and names["conv1d.bias"].shape == (conv_dim,)
    assert names["in_proj.weight"].shape == (d_inner + conv_dim + 4, 128) and names["out_proj.weight"].shape == (128, d_inner)
    assert names["dt_bias"].shape == (4,) and names["A_log"].shape == (4,) and names["D"].shape == (4,)
    assert names["norm.weight"].shape == (d_inner,)


@pytest.mark.parametrize("recompute", [False, True])
def test_mixer_forward_backward_matches_oracle(recompute):
    cfg, m = _mixer(torch.float32)
    m.recompute_core = recompute            # False (default): the core's activations are kept; True: the reference's recompute
    x = torch.randn(2, 256, 128, generator=torch.Generator().manual_seed(1))
    xd = x.to(DEV).requires_grad_(True)
    y = m(xd)
    dy = torch.randn(2, 256, 128, generator=torch.Generator().manual_seed(2))
    y.backward(dy.to(DEV))
    # oracle: same weights in fp64 on the CPU
    W = {k: v.detach().double().cpu().requires_grad_(True) for k, v in m.named_parameters()}
    xr = x.double().requires_grad_(True)
    z = xr @ W["in_proj.weight"].T
    core = fused_core_ref(z, -torch.exp(W["A_log"]), W["D"], W["conv1d.weight"], W["conv1d.bias"], W["dt_bias"], W["norm.weight"],
                          cfg.n_groups, cfg.state_size, 256, cfg.head_dim)
    yr = core @ W["out_proj.weight"].T
    yr.backward(dy.double())
    assert rel_err(y, yr.detach()) < 2e-4
    assert rel_err(xd.grad, xr.grad) < 5e-4
    for k, p in m.named_parameters():
        assert rel_err(p.grad, W[k].grad) < 1e-3, k


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixer_step_equals_forward(dtype):
    # chunked sequence path == token-by-token recurrent path, at layer level (mamba2_inference_no_tp.py:97-133)
    from mamba2.mamba2_mixer import Mamba2Cache
    cfg, m = _mixer(dtype)
    b, l = 2, 160
    x = torch.randn(b, l, 128, generator=torch.Generator().manual_seed(3)).to(dtype).to(DEV)
    with torch.no_grad():
        y_seq = m(x)
        cache = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=3)
        ys = [m.step(x[:, t:t + 1], cache) for t in range(l)]
    y_step = torch.cat(ys, dim=1)
    if dtype == torch.float32:
        assert rel_err(y_step, y_seq) < 2e-4
    else:
        assert rel_rms_err(y_step, y_seq.float()) < 3e-2
