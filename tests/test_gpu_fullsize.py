"""GPU: size-independent properties at the full benchmark shapes (the fp64 oracle is too slow there).

* sequence split: scanning the whole sequence == scanning its two halves with the final state of the first handed to
  the second as initial state (forward), for the 2.7B (c1) and 7B-layer (c3) SSD shapes;
* linearity of the backward in dy, and dD == sum(dy * x) (mamba2_kernel.py:471), at the c1 and c3 shapes;
* conv: shifting the input by one token shifts the output by one token (causality + time invariance), c2 shape;
* decode: 4 token steps from the prefill's final state == the chunked scan over the 4 extra tokens, c4 width;
* the whole mixer layer at the 7B-layer (c3) and 2.7B shapes: finite, batch rows independent;
* two model layers at the 2.7B width: token-by-token path, prefill hand-off and captured step against the sequence forward.
"""
import pytest
import torch

from conftest import rel_rms_err
from oracle.ssd import make_ssd_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("b,l,h,p,n,g", [(4, 2048, 80, 64, 128, 1), (2, 4096, 128, 64, 128, 8)])
def test_ssd_sequence_split_bf16(b, l, h, p, n, g):
    from mamba2.mamba2_kernel import ssd_forward
    d = make_ssd_inputs(b, l, h, p, n, g, seed=3, dtype=torch.bfloat16, device=DEV)
    y, S = ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], want_final_state=True)
    m = l // 2 + 128 * 3 + 40          # not a chunk multiple
    a = {k: d[k][:, :m] for k in ("dt", "X", "B", "C")}
    z = {k: d[k][:, m:] for k in ("dt", "X", "B", "C")}
    y1, S1 = ssd_forward(a["dt"], d["A"], a["X"], a["B"], a["C"], d["D"], want_final_state=True)
    y2, S2 = ssd_forward(z["dt"], d["A"], z["X"], z["B"], z["C"], d["D"], initial_state=S1, want_final_state=True)
    assert torch.isfinite(y.float()).all()
    # both sides are bf16 computations, each within 2e-2 x RMS of the exact result (the parity bar): triangle inequality
    assert rel_rms_err(torch.cat([y1, y2], dim=1), y.float()) < 4e-2
    # the states are fp32 sums of MFMA products whose operands (dt * decay * x, B) were rounded to bf16, and the chunk
    # boundaries of the two scans differ, so the rounded operands differ: same bound
    assert rel_rms_err(S2, S) < 4e-2
    assert (S2 - S).norm() / S.norm() < 5e-3


@pytest.mark.parametrize("b,l,h,p,n,g", [(4, 2048, 80, 64, 128, 1), (2, 4096, 128, 64, 128, 8)])
def test_ssd_backward_linearity(b, l, h, p, n, g):
    from mamba2.mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward
    d = make_ssd_inputs(b, l, h, p, n, g, seed=5, dtype=torch.bfloat16, device=DEV)
    st = alloc_chunk_states(d["dt"], d["A"], d["X"], d["B"], d["C"])
    ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], chunk_states=st)
    gen = torch.Generator(device=DEV).manual_seed(1)
    dy1 = torch.randn(b, l, h, p, device=DEV, generator=gen).to(torch.bfloat16)
    dy2 = torch.randn(b, l, h, p, device=DEV, generator=gen).to(torch.bfloat16)
    dys = (dy1.float() + dy2.float())
    dy12 = dys.to(torch.bfloat16)
    g1 = ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], dy1, chunk_states=st)
    g2 = ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], dy2, chunk_states=st)
    g12 = ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], dy12, chunk_states=st)
    for name, a_, b_, c_ in zip(("ddt", "dA", "dX", "dB", "dC", "dD"), g1, g2, g12):
        assert torch.isfinite(c_.float()).all(), name
        # three bf16 computations, each within 2e-2 x RMS of its exact gradient: triangle inequality on the maximum,
        # and a tight bound on the relative L2 difference, which a wrong term or sign would break
        assert rel_rms_err(c_.float(), a_.float() + b_.float()) < 6e-2, name
        assert (c_.float() - a_.float() - b_.float()).norm() / c_.float().norm() < 1e-2, name
    # dD_h = sum over batch, tokens and channels of dy * x  (mamba2_kernel.py:471)
    dD_direct = (dy12.float() * d["X"].float()).sum(dim=(0, 1, 3))
    assert rel_rms_err(g12[5], dD_direct) < 1e-3


def test_conv_shift_equivariance_c2():
    from mamba2.conv1d_grouped import conv1d_forward
    from oracle.conv import make_conv_inputs
    d = make_conv_inputs(4, 2048, 5376, 4, seed=2, dtype=torch.bfloat16, device=DEV)
    y = conv1d_forward(d["x"], d["w"], d["bias"], "silu", channels_last=True)
    xs = torch.zeros_like(d["x"])
    xs[:, 1:] = d["x"][:, :-1]
    ys = conv1d_forward(xs, d["w"], d["bias"], "silu", channels_last=True)
    assert torch.equal(ys[:, 1:], y[:, :-1])
    # a zero token in front sees only the bias
    assert torch.equal(ys[:, 0], torch.nn.functional.silu(d["bias"].float()).to(torch.bfloat16).expand(4, -1))


def test_decode_continues_prefill_c4_width():
    # prefill l tokens with the chunked scan, then 4 decode steps == chunked scan over l + 4 tokens (last 4 outputs, final state)
    from mamba2.mamba2_kernel import ssd_forward
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    b, l, h, p, n, g = 8, 256, 80, 64, 128, 1
    extra = 4
    d = make_ssd_inputs(b, l + extra, h, p, n, g, seed=7, dtype=torch.bfloat16, device=DEV)
    y_all, S_all = ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], want_final_state=True)
    _, S = ssd_forward(d["dt"][:, :l], d["A"], d["X"][:, :l], d["B"][:, :l], d["C"][:, :l], d["D"], want_final_state=True)
    # the decode step convolves and activates its input; an identity conv (weight 1 on the current token, no bias, no
    # activation) hands x, B, C of the extra tokens to the state update unchanged
    C = h * p + 2 * g * n
    w = torch.zeros(C, 4, dtype=torch.bfloat16, device=DEV)
    w[:, 3] = 1
    conv_state = torch.zeros(b, C, 3, dtype=torch.bfloat16, device=DEV)
    ys = []
    for t in range(l, l + extra):
        xBC = torch.cat([d["X"][:, t].reshape(b, -1), d["B"][:, t].reshape(b, -1), d["C"][:, t].reshape(b, -1)], dim=-1).unsqueeze(1)
        y, conv_state, S = mamba2_kernel_inference(xBC.contiguous(), conv_state, w, None, S, d["dt"][:, t:t + 1].contiguous(), d["A"], d["D"],
                                                   n_groups=g, activation=None)
        ys.append(y)
    y_dec = torch.cat(ys, dim=1).view(b, extra, h, p)
    # the decode step works in fp32 on the bf16 inputs; the chunked scan rounds its MFMA operands to bf16
    assert rel_rms_err(y_dec, y_all[:, l:].float()) < 2e-2
    assert rel_rms_err(S, S_all) < 4e-2
    assert (S - S_all).norm() / S_all.norm() < 5e-3


@pytest.mark.parametrize("hidden,heads,groups,b,l", [(4096, 128, 8, 2, 4096), (2560, 80, 1, 4, 2048)])
def test_mixer_layer_full_shape_batch_rows_independent(hidden, heads, groups, b, l):
    """The whole mixer layer (in_proj -> fused core -> out_proj) at the 7B-layer and 2.7B shapes, forward + backward:
    finite, and every batch row computed alone gives what it gives inside the batch (outputs and input gradients; the
    rows only meet in the parameter gradients)."""
    from mamba2.configuration_mamba2 import Mamba2Config
    from mamba2.mamba2_mixer import Mamba2Mixer
    cfg = Mamba2Config(num_heads=heads, head_dim=64, hidden_size=hidden, state_size=128, n_groups=groups, num_hidden_layers=1)
    torch.manual_seed(0)
    with torch.device(DEV):
        mix = Mamba2Mixer(cfg, 0).to(torch.bfloat16)
    gen = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn(b, l, hidden, device=DEV, generator=gen).to(torch.bfloat16).requires_grad_(True)
    dy = torch.randn(b, l, hidden, device=DEV, generator=gen).to(torch.bfloat16)
    y = mix(x)
    y.backward(dy)
    assert torch.isfinite(y.float()).all() and torch.isfinite(x.grad.float()).all()
    for name, p_ in mix.named_parameters():
        assert p_.grad is not None and torch.isfinite(p_.grad.float()).all(), name
    x1 = x.detach()[b - 1:].clone().requires_grad_(True)
    y1 = mix(x1)
    y1.backward(dy[b - 1:])
    # the projections may pick different GEMM tiles for the one-row batch, so this compares two bf16 computations, each
    # within 2e-2 x RMS of the exact result: triangle inequality, and a tight relative-L2 bound
    for a_, b_ in ((y1, y.detach()[b - 1:]), (x1.grad, x.grad[b - 1:])):
        assert rel_rms_err(a_.float(), b_.float()) < 4e-2
        assert ((a_.float() - b_.float()).norm() / b_.float().norm()).item() < 5e-3


def test_model_step_full_width_two_layers():
    """Two layers at the 2.7B width (d_model 2560, 80 heads, one group, n 128), bf16: the token-by-token path, the prefill
    hand-off and the captured step against the sequence forward, on the kernels' fast paths for this head count."""
    from mamba2.configuration_mamba2 import Mamba2Config
    from mamba2.mamba2_mixer import Mamba2Cache
    from mamba2.modeling_mamba2 import GraphedStep, Mamba2ForCausalLM
    cfg = Mamba2Config(num_heads=80, head_dim=64, hidden_size=2560, state_size=128, n_groups=1, num_hidden_layers=2, vocab_size=1024,
                       initializer_range=0.5)
    torch.manual_seed(0)
    with torch.device(DEV):
        m = Mamba2ForCausalLM(cfg).to(torch.bfloat16).eval()
    b, l1, l2 = 4, 200, 8
    ids = torch.randint(0, cfg.vocab_size, (b, l1 + l2), device=DEV, generator=torch.Generator(device=DEV).manual_seed(2))

    def close(got, ref):
        g_, r_ = got.double(), ref.double()
        return ((g_ - r_).norm() / r_.norm()).item() < 2e-2 and rel_rms_err(got.float(), ref.float()) < 0.2

    with torch.no_grad():
        full = m(input_ids=ids).logits
        cache = Mamba2Cache(cfg, b, dtype=torch.bfloat16, device=DEV, conv_width=3)
        pre = m(input_ids=ids[:, :l1], cache_params=cache, use_cache=True).logits
        assert close(pre, full[:, :l1])
        snap = [t.clone() for t in cache.conv_states + cache.ssm_states]
        steps = torch.cat([m.step(ids[:, l1 + t:l1 + t + 1], cache) for t in range(l2)], dim=1)
        assert close(steps, full[:, l1:])
        for t, k in zip(cache.conv_states + cache.ssm_states, snap):
            t.copy_(k)
        graphed = GraphedStep(m, cache, b)
        replayed = torch.cat([graphed(ids[:, l1 + t:l1 + t + 1]).clone() for t in range(l2)], dim=1)
    assert torch.equal(replayed, steps)
