"""GPU: the entry points can be captured into a HIP graph and replayed (they allocate nothing, clear nothing with
memset nodes and never synchronise): SSD forward + backward, the fused mixer core, and a run of decode steps.

Each graph is replayed several times with new input contents, with eager work and synchronisations between the
replays, and every replay is compared with the eager result for the same inputs (bit-exact: the kernels are
deterministic).
"""
import pytest
import torch

from oracle.ssd import make_ssd_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _capture(fn, warmup=2):
    """Run fn eagerly on a side stream (so lazily created workspaces exist), then capture it."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(warmup):
            fn()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn()
    return g, out


def test_ssd_fwd_bwd_graph_replay():
    from mamba2.mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward
    b, l, h, p, n, g = 2, 300, 8, 64, 128, 2
    d = make_ssd_inputs(b, l, h, p, n, g, seed=0, dtype=torch.bfloat16, device=DEV)
    st = alloc_chunk_states(d["dt"], d["A"], d["X"], d["B"], d["C"])
    keys = ("dt", "X", "B", "C", "dy")

    def step():
        y, S = ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], chunk_states=st, want_final_state=True)
        grads = ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], d["dy"], chunk_states=st)
        return (y, S) + tuple(t for t in grads if t is not None)

    graph, outs = _capture(step)
    for seed in (1, 2, 3):
        new = make_ssd_inputs(b, l, h, p, n, g, seed=seed, dtype=torch.bfloat16, device=DEV)
        for k in keys:
            d[k].copy_(new[k])
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        # eager work on the same stream between the replays, and the eager result for the same inputs
        ref = [t.clone() for t in step()]
        torch.cuda.synchronize()
        for i, (a, e) in enumerate(zip(got, ref)):
            assert torch.equal(a, e), (seed, i)


def test_fused_core_graph_replay():
    from mamba2.fused_kernel import _backward_parts, _forward_parts
    b, l, h, p, n, g = 2, 256, 8, 64, 64, 2
    d_inner = h * p
    width = 2 * d_inner + 2 * g * n + h          # 1288: rows of the packed buffer are 16-byte aligned
    gen = torch.Generator(device=DEV).manual_seed(0)
    zx = torch.randn(b, l, width, device=DEV, generator=gen).to(torch.bfloat16)
    A = -torch.exp(torch.empty(h, device=DEV).uniform_(0.0, 2.0, generator=gen))
    D = torch.ones(h, device=DEV)
    cw = (torch.rand(d_inner + 2 * g * n, 1, 4, device=DEV, generator=gen) - 0.5).to(torch.bfloat16)
    cb = (torch.rand(d_inner + 2 * g * n, device=DEV, generator=gen) - 0.5).to(torch.bfloat16)
    dtb = torch.empty(h, device=DEV).uniform_(-5.0, -2.0, generator=gen)
    nw = torch.ones(d_inner, device=DEV)
    dout = torch.randn(b, l, d_inner, device=DEV, generator=gen).to(torch.bfloat16)
    dims = (g, n, d_inner, p)

    def step():
        with torch.no_grad():
            norm_out, conv_out, scan_out, states = _forward_parts(zx, A, D, cw, cb, dtb, nw, *dims, keep_states=True)
            grads = _backward_parts(dout, zx, A, D, cw, cb, dtb, nw, conv_out, scan_out, states, *dims)
        return (norm_out,) + tuple(grads)

    graph, outs = _capture(step)
    for seed in (1, 2, 3):
        g2 = torch.Generator(device=DEV).manual_seed(seed)
        zx.copy_(torch.randn(b, l, width, device=DEV, generator=g2).to(torch.bfloat16))
        dout.copy_(torch.randn(b, l, d_inner, device=DEV, generator=g2).to(torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        ref = [t.clone() for t in step()]
        torch.cuda.synchronize()
        for i, (a, e) in enumerate(zip(got, ref)):
            assert torch.equal(a, e), (seed, i)


def test_decode_steps_graph_replay():
    """One captured decode step replayed token after token: the in-place conv and SSM states advance exactly as in eager mode."""
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    from oracle.decode import make_decode_inputs
    b, h, p, n, g = 3, 8, 64, 128, 2
    q = {k: v.to(DEV) for k, v in make_decode_inputs(b, h, p, n, g, W=3, seed=0, act_dtype=torch.bfloat16).items()}
    conv_g, S_g = q["conv_state"].clone(), q["S"].clone()
    conv_e, S_e = q["conv_state"].clone(), q["S"].clone()
    xBC, dt = q["xBC"].clone(), q["dt"].clone()

    def step_graph():
        y, _, _ = mamba2_kernel_inference(xBC, conv_g, q["conv_weight"], q["conv_bias"], S_g, dt, q["A"], q["D"], n_groups=g)
        return y

    # warm-up steps run on copies so that the captured states start where the eager ones do
    keep = (conv_g.clone(), S_g.clone())
    graph, y_out = _capture(step_graph)
    conv_g.copy_(keep[0]); S_g.copy_(keep[1])
    gen = torch.Generator(device=DEV).manual_seed(5)
    for t in range(4):
        xBC.copy_(torch.randn(xBC.shape, device=DEV, generator=gen).to(xBC.dtype))
        dt.copy_((0.05 + 0.1 * torch.rand(dt.shape, device=DEV, generator=gen)).to(dt.dtype))
        graph.replay()
        torch.cuda.synchronize()
        y_e, _, _ = mamba2_kernel_inference(xBC, conv_e, q["conv_weight"], q["conv_bias"], S_e, dt, q["A"], q["D"], n_groups=g)
        torch.cuda.synchronize()
        assert torch.equal(y_out, y_e), t
        assert torch.equal(conv_g, conv_e) and torch.equal(S_g, S_e), t
