#!/usr/bin/env python3
"""Benchmark of the MI355X Mamba-2 mixer hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|ssd|conv|glue|core|layer|decode|model|copy|pattern] [--no-cpu] [--no-gemm-tuning]

One "step" is one pass of the hot path over one batch of synthetic input, inputs resident in HBM:
  ssd    : SSD chunked scan fwd+bwd, bf16, 2.7B shape (b4, l2048, h80, p64, n128, g1, chunk 128)   <- headline
  conv   : depthwise conv1d k=4 + SiLU fwd+bwd, bf16 (b4, l2048, C5376)
  layer  : one whole Mamba2Mixer layer fwd+bwd at the 7B shape (b2, l4096, d_model 4096, h128, g8)
  decode : one decode token-step over 64 stacked layers of the 2.7B shape, batch 128
Prints ONE JSON line (rank 0).  The headline metric is SSD fwd+bwd tokens/s; `roofline` prices the
SSD step against the dense bf16 MFMA peak using the ALGORITHMIC FLOPs (G shared per group, no
recompute counted); conv and decode are reported under `other` against the HBM peak with their
algorithmic bytes.  `cpu_baseline` is the pure-PyTorch oracle timed on this box's host cores.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "state-space-models-neuron_amd"))

MFMA_BF16_PEAK_TFLOPS = 2500.0     # MI355X dense bf16
HBM_PEAK_GBS = 8000.0              # MI355X HBM3E
# HBM bytes per step as PROFILED (two rocprofv3 --pmc runs of this file, FETCH_SIZE then WRITE_SIZE, each scaled by what
# the same counter reads for the 1 GiB copy kernel in the same run; summaries under profiles/).  They are constants of
# the kernels as last profiled, not measurements of this run: `traffic_source` in the JSON says so.
SSD_TRAFFIC_BYTES = 1.460e9
CONV_TRAFFIC_BYTES = 489.3e6
DECODE_TRAFFIC_BYTES = 64 * 689.2e6
GLUE_TRAFFIC_BYTES = 710.5e6
TRAFFIC_SOURCE = "profiled constant: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this workload, scaled by the 1 GiB copy kernel; not measured in this run"

SSD_CFG = dict(b=4, l=2048, h=80, p=64, n=128, g=1)
CONV_CFG = dict(b=4, l=2048, C=5376, k=4)
DEC_CFG = dict(b=128, h=80, p=64, n=128, g=1, k=4, W=3, layers=64)
Q = 128


def ssd_flops_fwd(b, l, h, p, n, g):
    c = math.ceil(l / Q)
    return b * c * (h * (2 * Q * Q * p + 4 * Q * n * p) + g * 2 * Q * Q * n)


def parity_entry(got, ref):
    """Acceptance figures of one tensor against the oracle (oracle.parity.bf16_figures): raw max|err| / RMS(ref) against
    the bf16 bar of 2e-2; for a tensor STORED in bf16 whose raw figure is over the bar, `adjusted` = raw less the storage
    floor max|bf16(ref) - ref| / RMS(ref) (the exact result rounded once to bf16); an fp32 result is held to the raw
    bar.  Also the relative L2 error, held to 1e-2."""
    from oracle.parity import bf16_figures
    f = bf16_figures(got, ref)
    return {"raw": round(f["raw"], 5), "adjusted": round(f["adjusted"], 5), "bf16_floor": round(f["tensor_floor"], 5),
            "kind": "stored bf16" if f["stored_bf16"] else "fp32 result", "rel_l2": round(f["rel_l2"], 6),
            "ok": bool(f["value"] < 2e-2 and f["rel_l2"] < 1e-2)}


def require_parity(name, table):
    bad = {k: v for k, v in table.items() if not v["ok"]}
    if bad:
        raise RuntimeError(f"{name}: outputs differ from the oracle, nothing timed: {bad}")


def event_time_ms(fn, steps, warmup):
    """Per-step durations from HIP events recorded on the stream the kernels are launched on."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for s, e in evs:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    per = [s.elapsed_time(e) for s, e in evs]
    return wall, per


def check_ssd(cfg, ref=None):
    """The HIP forward + backward against the oracle on the same seeded bf16 inputs, before anything is timed.  `ref`:
    oracle results already computed for cfg by the CPU-baseline leg (fp32 arithmetic on the same inputs)."""
    import torch
    from mamba2.mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward
    from oracle.ssd import make_ssd_inputs, ssd_grads_ref
    d = make_ssd_inputs(cfg["b"], cfg["l"], cfg["h"], cfg["p"], cfg["n"], cfg["g"], seed=0, dtype=torch.bfloat16)
    if ref is None:
        ref = ssd_grads_ref(*(d[k].double() for k in ("dt", "A", "X", "B", "C", "D", "dy")), chunk=Q)
    g = {k: v.to("cuda:0") for k, v in d.items()}
    st = alloc_chunk_states(g["dt"], g["A"], g["X"], g["B"], g["C"])
    y, S = ssd_forward(g["dt"], g["A"], g["X"], g["B"], g["C"], g["D"], want_final_state=True, chunk_states=st)
    ddt, dA, dX, dB, dC, dD, _ = ssd_backward(g["dt"], g["A"], g["X"], g["B"], g["C"], g["D"], g["dy"], chunk_states=st)
    got = {"y": y, "dX": dX, "ddt": ddt, "dB": dB, "dC": dC, "dA": dA, "dD": dD}
    got["final_state"] = S
    table = {k: parity_entry(v, ref[k]) for k, v in got.items()}
    require_parity("ssd", table)
    return table


def bench_ssd(steps, warmup, ref=None, check_cfg=None):
    import torch
    from mamba2.mamba2_kernel import SAVE_CHUNK_STATES, alloc_chunk_states, ssd_backward, ssd_forward
    from oracle.ssd import make_ssd_inputs
    cfg = SSD_CFG
    parity = check_ssd(check_cfg or cfg, ref)
    d = make_ssd_inputs(cfg["b"], cfg["l"], cfg["h"], cfg["p"], cfg["n"], cfg["g"], seed=0, dtype=torch.bfloat16, device="cuda:0")
    # what Mamba2Kernel.forward/backward do: the forward keeps the chunk states and operand tiles for the backward (102 MB here)
    states = alloc_chunk_states(d["dt"], d["A"], d["X"], d["B"], d["C"]) if SAVE_CHUNK_STATES else None

    def step():
        ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], want_final_state=True, chunk_states=states)
        ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], d["dy"], chunk_states=states)

    wall_ms, per = event_time_ms(step, steps, warmup)
    per.sort()
    ms = sum(per) / len(per)
    tokens = cfg["b"] * cfg["l"]
    flops = 3 * ssd_flops_fwd(**cfg)
    io_bytes = 2 * (5 * cfg["b"] * cfg["l"] * cfg["h"] * cfg["p"] + 4 * cfg["b"] * cfg["l"] * cfg["g"] * cfg["n"] + 2 * cfg["b"] * cfg["l"] * cfg["h"])
    return dict(ms_per_step=wall_ms, ms_event_avg=ms, ms_event_min=per[0], ms_event_median=per[len(per) // 2],
                tokens_per_s=tokens / (wall_ms * 1e-3), flops=flops, io_bytes=io_bytes, tflops=flops / (ms * 1e-3) / 1e12, tokens=tokens,
                parity=parity, parity_shape="b{b} l{l} h{h} p{p} n{n} g{g}".format(**(check_cfg or cfg)))


def bench_conv(steps, warmup):
    import torch
    from mamba2.conv1d_grouped import conv1d_backward, conv1d_forward
    from oracle.conv import make_conv_inputs
    cfg = CONV_CFG
    nsets = 4          # rotate input sets so the 256 MB MALL does not serve the reads
    sets = [make_conv_inputs(cfg["b"], cfg["l"], cfg["C"], cfg["k"], seed=s, dtype=torch.bfloat16, device="cuda:0") for s in range(nsets)]
    outs = [torch.empty_like(sets[0]["x"]) for _ in range(2)]
    state = {"i": 0}
    # the full workload against the oracle (F.conv1d + SiLU + autograd, fp64) before timing
    from oracle.conv import conv1d_grads_ref
    c0 = {k: v.cpu().double() for k, v in sets[0].items()}
    y_ref, dx_ref, dw_ref, db_ref = conv1d_grads_ref(c0["x"], c0["w"], c0["bias"], c0["dy"], "silu")
    y0 = conv1d_forward(sets[0]["x"], sets[0]["w"], sets[0]["bias"], "silu", channels_last=True)
    dx0, dw0, db0 = conv1d_backward(sets[0]["x"], sets[0]["w"], sets[0]["bias"], sets[0]["dy"], "silu", channels_last=True)
    parity = {"y": parity_entry(y0, y_ref), "dx": parity_entry(dx0, dx_ref), "dw": parity_entry(dw0, dw_ref), "db": parity_entry(db0, db_ref)}
    require_parity("conv1d", parity)
    del c0, y_ref, dx_ref, y0, dx0

    def step():
        d = sets[state["i"] % nsets]
        state["i"] += 1
        conv1d_forward(d["x"], d["w"], d["bias"], "silu", channels_last=True, out=outs[0])
        conv1d_backward(d["x"], d["w"], d["bias"], d["dy"], "silu", channels_last=True, out_dx=outs[1])

    wall_ms, per = event_time_ms(step, steps, warmup)
    ms = sum(per) / len(per)
    elems = cfg["b"] * cfg["l"] * cfg["C"]
    bytes_ = elems * 2 * 5          # fwd: read x, write y; bwd: read x, dy, write dx
    tokens = cfg["b"] * cfg["l"]
    return dict(metric="conv1d+SiLU fwd+bwd tokens/s", value=tokens / (ms * 1e-3), unit="tokens/s", ms_per_step=ms, dtype="bf16",
                config={"workload": "depthwise conv1d k=4 + SiLU fwd+bwd, b4 l2048 C5376, channels-last"}, parity=parity,
                roofline={"bound": "hbm", "achieved": bytes_ / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": bytes_ / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": CONV_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                          "algorithmic_bytes_per_step": bytes_, "kernels": "conv_fwd_cl_kernel + conv_bwd_cl_kernel + conv_reduce_partials_kernel"})


def bench_glue(steps, warmup):
    """Mixer glue at the 2.7B layer shape: gated RMSNorm over d_inner = 5120 (one group) and softplus(dt + bias) over 80
    heads, forward + backward, with z / dz / dt / ddt as column slices of packed (b, l, 10576) buffers as in the layer."""
    import torch
    from mamba2 import glue
    b, l, d, h, g = SSD_CFG["b"], SSD_CFG["l"], SSD_CFG["h"] * SSD_CFG["p"], SSD_CFG["h"], SSD_CFG["g"]
    width = 2 * d + 2 * g * SSD_CFG["n"] + h
    gen = torch.Generator(device="cuda:0").manual_seed(0)
    nsets = 3          # rotate input sets so the 256 MB MALL does not serve the reads
    sets = []
    for _ in range(nsets):
        packed = torch.randn(b, l, width, device="cuda:0", generator=gen).to(torch.bfloat16)
        sets.append(dict(packed=packed, x=torch.randn(b, l, d, device="cuda:0", generator=gen).to(torch.bfloat16),
                         dout=torch.randn(b, l, d, device="cuda:0", generator=gen).to(torch.bfloat16),
                         ddt=torch.randn(b, l, h, device="cuda:0", generator=gen).to(torch.bfloat16)))
    w = torch.ones(d, device="cuda:0")
    bias = torch.zeros(h, device="cuda:0")
    dpacked = torch.empty(b, l, width, dtype=torch.bfloat16, device="cuda:0")
    state = {"i": 0}

    def step():
        s_ = sets[state["i"] % nsets]
        state["i"] += 1
        z, dt = s_["packed"][..., :d], s_["packed"][..., width - h:]
        glue.softplus_bias_hip(dt, bias)
        glue.rmsnorm_gated_hip(s_["x"], z, w, g, 1e-5, out_dtype=torch.bfloat16)
        glue.rmsnorm_gated_bwd_hip(s_["x"], z, w, s_["dout"], g, 1e-5, out_dz=dpacked[..., :d])
        glue.softplus_bias_bwd_hip(dt, bias, s_["ddt"], out_d_in=dpacked[..., width - h:])

    wall_ms, per = event_time_ms(step, steps, warmup)
    ms = sum(per) / len(per)
    bytes_ = b * l * d * 2 * 8 + b * l * h * 2 * 5      # norm: x, z, out | x, z, d_out, dx, dz; softplus: dt, out | dt, d_out, d_in
    tokens = b * l
    return dict(metric="mixer glue (gated RMSNorm + softplus) fwd+bwd tokens/s", value=tokens / (ms * 1e-3), unit="tokens/s", ms_per_step=ms,
                dtype="bf16 I/O, f32 arithmetic",
                config={"workload": "gated RMSNorm d5120 g1 + softplus(dt + bias) h80, fwd+bwd, b4 l2048, packed-buffer column slices"},
                roofline={"bound": "hbm", "achieved": bytes_ / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": bytes_ / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": GLUE_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                          "algorithmic_bytes_per_step": bytes_,
                          "kernels": "rmsnorm_gated_kernel fwd + bwd, column_sum_kernel, softplus_fwd_kernel, softplus_bwd_kernel"})


def bench_core(steps, warmup):
    """The fused mixer core zxBCdt -> norm_out (conv + SiLU, softplus, SSD scan, gated norm) forward + backward at the
    2.7B layer shape, through the reference's autograd-function signature (the caching variant: nothing is recomputed)."""
    import torch
    from mamba2.fused_kernel import mamba2_fused_kernel_with_caching
    cfg = SSD_CFG
    b, l, h, p, n, g = cfg["b"], cfg["l"], cfg["h"], cfg["p"], cfg["n"], cfg["g"]
    d = h * p
    width = 2 * d + 2 * g * n + h
    gen = torch.Generator(device="cuda:0").manual_seed(0)
    zx = torch.randn(b, l, width, device="cuda:0", generator=gen)
    zx[..., 2 * d:2 * d + 2 * g * n] /= n ** 0.5
    zx = zx.to(torch.bfloat16).requires_grad_(True)
    A = (-torch.exp(torch.empty(h, device="cuda:0").uniform_(0.0, 2.77, generator=gen))).requires_grad_(True)
    D = torch.ones(h, device="cuda:0", requires_grad=True)
    cw = (torch.rand(d + 2 * g * n, 1, 4, device="cuda:0", generator=gen) - 0.5).to(torch.bfloat16).requires_grad_(True)
    cb = (torch.rand(d + 2 * g * n, device="cuda:0", generator=gen) - 0.5).to(torch.bfloat16).requires_grad_(True)
    dtb = torch.empty(h, device="cuda:0").uniform_(-5.0, -2.0, generator=gen).requires_grad_(True)
    nw = torch.ones(d, device="cuda:0", requires_grad=True)
    dout = torch.randn(b, l, d, device="cuda:0", generator=gen).to(torch.bfloat16)
    leaves = (zx, A, D, cw, cb, dtb, nw)

    def step():
        for t in leaves:
            t.grad = None
        out = mamba2_fused_kernel_with_caching(zx, A, D, cw, cb, dtb, nw, g, n, d, p)
        # the core computes and returns d_zxBCdt as always; autograd is only told not to copy it into zx.grad (in the layer
        # zxBCdt is the projection's output and its gradient goes straight into that GEMM's backward, no copy either)
        out.backward(dout, inputs=leaves[1:])

    wall_ms, per = event_time_ms(step, steps, warmup)
    ms = sum(per) / len(per)
    tokens = b * l
    return dict(metric="fused mixer core fwd+bwd tokens/s", value=tokens / (wall_ms * 1e-3), unit="tokens/s", ms_per_step=wall_ms,
                event_ms_avg=ms, dtype="bf16",
                config={"workload": "mamba2_fused_kernel_with_caching fwd+bwd, zxBCdt (4, 2048, 10576): conv k4 + SiLU, softplus, SSD h80 p64 n128 g1, gated RMSNorm"})


LAYER_C3 = dict(b=2, l=4096, d_model=4096, h=128, p=64, n=128, g=8)


def check_core_c3_width(cfg, b=1, l=512):
    """The fused mixer core at the 7B layer's width (d_inner 8192, 128 heads, 8 groups) against oracle.mixer.fused_core_ref
    (fp64) on seeded bf16 inputs, forward and backward, on a short batch (b1 l512: the width is what the kernels' slicing
    depends on; the whole shape runs in tests/test_gpu_fullsize_oracle.py).  The chain hands bf16 tensors from stage to
    stage, so next to the raw figure stands the floor of those hand-overs: the same oracle with a bf16 round at each."""
    import torch
    from mamba2.fused_kernel import mamba2_fused_kernel
    from oracle.mixer import fused_core_ref
    h, p, n, g = cfg["h"], cfg["p"], cfg["n"], cfg["g"]
    d = h * p
    width = 2 * d + 2 * g * n + h
    gen = torch.Generator().manual_seed(3)
    zx = torch.randn(b, l, width, generator=gen)
    zx[..., 2 * d:2 * d + 2 * g * n] /= n ** 0.5
    t = {"zxBCdt": zx.to(torch.bfloat16), "A": -torch.exp(torch.empty(h).uniform_(0.0, 2.77, generator=gen)), "D": torch.ones(h),
         "conv_w": (torch.rand(d + 2 * g * n, 1, 4, generator=gen) - 0.5).to(torch.bfloat16),
         "conv_b": (torch.rand(d + 2 * g * n, generator=gen) - 0.5).to(torch.bfloat16),
         "dt_bias": torch.empty(h).uniform_(-5.0, -2.0, generator=gen), "norm_w": torch.ones(d)}
    dout = torch.randn(b, l, d, generator=gen).to(torch.bfloat16)
    names = ("zxBCdt", "A", "D", "conv_w", "conv_b", "dt_bias", "norm_w")

    class RoundBF16(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            return x.bfloat16().to(x.dtype)

        @staticmethod
        def backward(ctx, gr):
            return gr.bfloat16().to(gr.dtype)

    def oracle(handover):
        lv = {k: t[k].double().clone().requires_grad_(True) for k in names}
        zin = lv["zxBCdt"] if handover is None else handover(lv["zxBCdt"])
        out = fused_core_ref(zin, lv["A"], lv["D"], lv["conv_w"], lv["conv_b"], lv["dt_bias"], lv["norm_w"], g, n, d, p, handover=handover)
        out.backward(dout.double())
        return out.detach(), lv["zxBCdt"].grad

    ref_out, ref_dz = oracle(None)
    flo_out, flo_dz = oracle(RoundBF16.apply)
    lv = {k: t[k].to("cuda:0").clone().requires_grad_(True) for k in names}
    out = mamba2_fused_kernel(*(lv[k] for k in names), g, n, d, p)
    out.backward(dout.to("cuda:0"))
    table = {}
    for k, got, ref, flo in (("norm_out", out.detach(), ref_out, flo_out), ("d_zxBCdt", lv["zxBCdt"].grad, ref_dz, flo_dz)):
        e = parity_entry(got, ref)
        hand = parity_entry(flo.to(torch.bfloat16), ref)["raw"]
        e["hand_over_floor"] = hand
        e["ok"] = bool(e["adjusted"] < 2e-2 + hand and e["rel_l2"] < 1e-2)
        table[k] = e
    require_parity("mixer core at the 7B width", table)
    return table


def bench_layer_c3(steps, warmup):
    """BASELINE configuration 3: one whole Mamba2Mixer layer at the 7B shape, forward + backward through autograd (in_proj,
    conv1d + SiLU, SSD scan, grouped gated RMSNorm, out_proj), bf16, weights ~ N(0, 0.02), hidden ~ N(0, 1).  The headline
    figure keeps the core's activations for the backward (this build's default); the form that recomputes them in the
    backward, as the reference's mixer does (mamba2/fused_kernel.py:352-367), is timed next to it.  Also the SSD scan alone
    at this shape (the part the MFMA roofline prices)."""
    import torch
    from mamba2.configuration_mamba2 import Mamba2Config
    from mamba2.mamba2_kernel import alloc_chunk_states, ssd_backward, ssd_forward
    from mamba2.mamba2_mixer import Mamba2Mixer
    from oracle.ssd import make_ssd_inputs
    cfg = LAYER_C3
    b, l, dm, h, p, n, g = (cfg[k] for k in ("b", "l", "d_model", "h", "p", "n", "g"))
    parity = check_core_c3_width(cfg)
    mc = Mamba2Config(num_heads=h, head_dim=p, hidden_size=dm, state_size=n, n_groups=g, num_hidden_layers=1, expand=2)
    torch.manual_seed(0)
    with torch.device("cuda:0"):
        m = Mamba2Mixer(mc, 0)
    with torch.no_grad():
        for w in (m.in_proj.weight, m.out_proj.weight):
            w.normal_(0.0, 0.02)
    m = m.to(torch.bfloat16)
    gen = torch.Generator(device="cuda:0").manual_seed(0)
    hidden = torch.randn(b, l, dm, device="cuda:0", generator=gen).to(torch.bfloat16).requires_grad_(True)
    dout = torch.randn(b, l, dm, device="cuda:0", generator=gen).to(torch.bfloat16)

    def layer_step():
        hidden.grad = None
        for q in m.parameters():
            q.grad = None
        m(hidden).backward(dout)

    wall_ms, per = event_time_ms(layer_step, steps, warmup)
    ms = sum(per) / len(per)
    m.recompute_core = True
    _, per_r = event_time_ms(layer_step, steps, warmup)
    ms_recompute = sum(per_r) / len(per_r)
    m.recompute_core = False
    # the scan alone at this shape, forward + backward with the forward's chunk states kept
    d = make_ssd_inputs(b, l, h, p, n, g, seed=0, dtype=torch.bfloat16, device="cuda:0")
    states = alloc_chunk_states(d["dt"], d["A"], d["X"], d["B"], d["C"])

    def ssd_step():
        ssd_forward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], chunk_states=states)
        ssd_backward(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], d["dy"], chunk_states=states)

    _, per_s = event_time_ms(ssd_step, steps, warmup)
    ms_ssd = sum(per_s) / len(per_s)
    ssd_flops = 3 * ssd_flops_fwd(b, l, h, p, n, g)
    d_inner = h * p
    gemm_flops = 3 * 2 * b * l * dm * (2 * d_inner + 2 * g * n + h) + 3 * 2 * b * l * d_inner * dm
    tokens = b * l
    return dict(metric="Mamba2Mixer layer fwd+bwd tokens/s (7B shape)", value=tokens / (ms * 1e-3), unit="tokens/s", ms_per_step=ms,
                wall_ms_per_step=wall_ms, ms_per_step_recompute_core=ms_recompute, dtype="bf16",
                config={"workload": "Mamba2Mixer fwd+bwd, b2 l4096 d_model4096 d_inner8192 h128 p64 n128 g8 chunk128: in_proj, conv1d+SiLU, SSD, grouped gated RMSNorm, out_proj; core activations kept for the backward"},
                parity={"against": "oracle.mixer.fused_core_ref (fp64), fused core at this width, b1 l512, checked before timing", "tensors": parity},
                projections={"gemm_flops_per_step": gemm_flops, "library": "hipBLASLt behind nn.Linear (outside the hot path)"},
                ssd_part={"ms_per_step": ms_ssd, "algorithmic_flops_per_step": ssd_flops,
                          "roofline": {"bound": "mfma", "achieved": ssd_flops / (ms_ssd * 1e-3) / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS,
                                       "unit": "TFLOP/s", "frac": ssd_flops / (ms_ssd * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, "traffic": None}},
                layer_tflops=(gemm_flops + ssd_flops) / (ms * 1e-3) / 1e12)


def bench_decode(steps, warmup):
    import torch
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    from oracle.decode import make_decode_inputs
    cfg = DEC_CFG
    L = cfg["layers"]
    d = make_decode_inputs(cfg["b"], cfg["h"], cfg["p"], cfg["n"], cfg["g"], cfg["k"], cfg["W"], seed=0, act_dtype=torch.bfloat16, device="cuda:0")
    gen = torch.Generator(device="cuda:0").manual_seed(1)
    # distinct state buffers per layer (21.5 GB of fp32 SSM state): nothing is served from cache
    S = [0.1 * torch.randn(cfg["b"], cfg["h"], cfg["p"], cfg["n"], device="cuda:0", generator=gen) for _ in range(L)]
    conv = [torch.randn(cfg["b"], d["xBC"].shape[-1], cfg["W"], device="cuda:0", generator=gen).to(torch.bfloat16) for _ in range(L)]
    # one layer against the oracle (fp64 on the host) before timing: y, the updated SSM state and the shifted conv state
    from oracle.decode import decode_step_ref
    S0, c0 = S[0].clone(), conv[0].clone()
    y_ref, cs_ref, S_ref = decode_step_ref(*(t.cpu().double() for t in (d["xBC"], c0, d["conv_weight"], d["conv_bias"], S0, d["dt"], d["A"], d["D"])),
                                           n_groups=cfg["g"])
    y0, c1, S1 = mamba2_kernel_inference(d["xBC"], c0, d["conv_weight"], d["conv_bias"], S0, d["dt"], d["A"], d["D"], n_groups=cfg["g"])
    parity = {"y": parity_entry(y0, y_ref), "S": parity_entry(S1, S_ref)}
    parity["S"]["ok"] = bool(parity["S"]["raw"] < 1e-4)
    parity["conv_state_bit_exact"] = {"ok": bool(torch.equal(c1.cpu().double(), cs_ref))}
    require_parity("decode", parity)
    del S0, c0, y_ref, cs_ref, S_ref, S1

    def step():
        for i in range(L):
            mamba2_kernel_inference(d["xBC"], conv[i], d["conv_weight"], d["conv_bias"], S[i], d["dt"], d["A"], d["D"], n_groups=cfg["g"])

    wall_ms, per = event_time_ms(step, steps, warmup)
    ms = sum(per) / len(per)
    Cx = d["xBC"].shape[-1]
    per_layer = 2 * S[0].numel() * 4 + 2 * conv[0].numel() * 2 + cfg["b"] * Cx * 2 + cfg["b"] * cfg["h"] * 2 + cfg["b"] * cfg["h"] * cfg["p"] * 2
    bytes_ = per_layer * L
    return dict(metric="decode token-step latency (64 layers, batch 128)", value=ms * 1e3, unit="us/step", higher_is_better=False,
                us_per_sequence_token=ms * 1e3 / cfg["b"], ms_per_step=ms, wall_ms_per_step=wall_ms, dtype="f32 state / bf16 activations",
                config={"workload": "decode step, 64 layers x (b128, h80, p64, n128, C5376, W3), states in place"}, parity=parity,
                roofline={"bound": "hbm", "achieved": bytes_ / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": bytes_ / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": DECODE_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                          "algorithmic_bytes_per_step": bytes_, "kernels": "decode_conv_kernel + decode_ssm_kernel, 64 launches each"})


def bench_model_step(steps, warmup, tune_gemms=True):
    """One decode step of the whole 2.7B-shaped model (embedding, 64 x [RMSNorm, in_proj, decode kernels, gated norm,
    out_proj, residual], final norm, LM head) at batch 128: eager launches and the same step replayed from one HIP graph."""
    import torch
    from mamba2.configuration_mamba2 import Mamba2Config
    from mamba2.mamba2_mixer import Mamba2Cache
    from mamba2.modeling_mamba2 import GraphedStep, Mamba2ForCausalLM
    cfg = Mamba2Config(num_heads=80, head_dim=64, hidden_size=2560, state_size=128, n_groups=1, num_hidden_layers=64, expand=2,
                       vocab_size=50288, residual_in_fp32=True)
    b = DEC_CFG["b"]
    torch.manual_seed(0)
    with torch.device("cuda:0"):
        model = Mamba2ForCausalLM(cfg).to(torch.bfloat16).eval()
    n_params = sum(p.numel() for p in model.parameters())
    cache = Mamba2Cache(cfg, b, dtype=torch.bfloat16, device="cuda:0", conv_width=DEC_CFG["W"])
    gen = torch.Generator(device="cuda:0").manual_seed(0)
    for t in cache.ssm_states:
        t.normal_(0.0, 0.1, generator=gen)
    ids = torch.randint(0, cfg.vocab_size, (b, 1), device="cuda:0", generator=gen)

    def eager():
        with torch.no_grad():
            model.step(ids, cache)

    wall_e, per_e = event_time_ms(eager, steps, warmup)
    try:
        graphed = GraphedStep(model, cache, b, tune_gemms=tune_gemms)      # the serving form: the libraries' best solutions for the three GEMM shapes
    except Exception as e:      # noqa: BLE001  (a torch build without TunableOp: the default solutions, and the line says so)
        if not tune_gemms:
            raise
        print(f"bench: GEMM tuning unavailable ({type(e).__name__}: {e}); capturing the default solutions", file=sys.stderr)
        tune_gemms = False
        graphed = GraphedStep(model, cache, b)
    wall_g, per_g = event_time_ms(lambda: graphed(ids), steps, warmup)
    ms_e, ms_g = sum(per_e) / len(per_e), sum(per_g) / len(per_g)
    # bytes a step has to move: every layer's states read and written, every weight but the embedding table read once
    state_bytes = sum(2 * t.numel() * t.element_size() for t in cache.ssm_states + cache.conv_states)
    weight_bytes = (n_params - model.backbone.embeddings.weight.numel()) * 2
    bytes_ = state_bytes + weight_bytes
    return dict(metric="whole-model decode step latency (2.7B shape, 64 layers, batch 128), HIP graph", value=ms_g * 1e3, unit="us/step",
                higher_is_better=False, ms_per_step=ms_g, ms_per_step_eager=ms_e, wall_ms_per_step=wall_g, wall_ms_per_step_eager=wall_e,
                tokens_per_s=b / (ms_g * 1e-3), parameters=n_params, dtype="bf16 weights and activations / f32 state and residual",
                config={"workload": "Mamba2ForCausalLM.step, d_model 2560, 64 layers, h80 p64 n128 g1, vocab 50288, b128, conv state W3"},
                roofline={"bound": "hbm", "achieved": bytes_ / (ms_g * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": bytes_ / (ms_g * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_step": bytes_,
                          "kernels": "one graph replay: projections (" + ("rocBLAS / hipBLASLt solutions chosen by torch TunableOp during the graph's warm-up; the eager figure uses the libraries' defaults" if tune_gemms else "the BLAS libraries' default solutions") + ") + decode_conv/decode_ssm/rmsnorm_gated kernels + torch elementwise"})


def bench_copy(steps, warmup):
    """Plain 16-byte-per-lane copy kernel over 1 GiB (read 1 GiB + write 1 GiB per launch): the HBM rate a trivial
    streaming kernel reaches on this box, and the dispatch of known size the HBM-traffic counters are scaled by."""
    import torch
    from mamba2 import _lib
    lib = _lib.load()
    nbytes = 1 << 30
    bufs = [(torch.empty(nbytes, dtype=torch.uint8, device="cuda:0").fill_(i), torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")) for i in range(2)]
    state = {"i": 0}

    def step():
        src, dst = bufs[state["i"] % 2]
        state["i"] += 1
        rc = lib.m2_stream_copy(src.data_ptr(), dst.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(lib.m2_last_error().decode())

    _, per = event_time_ms(step, steps, warmup)
    ms = sum(per) / len(per)
    moved = 2 * nbytes
    return dict(metric="plain copy kernel HBM rate", value=moved / (ms * 1e-3) / 1e9, unit="GB/s", ms_per_step=ms, dtype="u8",
                config={"workload": "stream_copy_kernel, 1 GiB read + 1 GiB write per launch"},
                roofline={"bound": "hbm", "achieved": moved / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_step": moved,
                          "kernels": "stream_copy_kernel"})


def bench_access_pattern(steps, warmup):
    """What the memory system gives a kernel with the SSD kernels' streams and no arithmetic: x of the c1 shape (b4 l2048,
    80 heads of 128 bytes per token row) read as per-head tiles of 128 rows and written back as contiguous tiles, against
    a plain copy of the same 84 MB.  A 1 GiB read in front of every timed launch leaves the caches holding none of it."""
    import torch
    from mamba2 import _lib
    lib = _lib.load()
    batch, rows, row_bytes = SSD_CFG["b"], SSD_CFG["l"], SSD_CFG["h"] * SSD_CFG["p"] * 2
    g = torch.Generator().manual_seed(0)
    src = torch.randint(0, 256, (batch * rows * row_bytes,), generator=g, dtype=torch.uint8).to("cuda:0")
    dst = torch.empty_like(src)
    sweep = torch.ones(1 << 28, dtype=torch.int32, device="cuda:0")
    stream = lambda: torch.cuda.current_stream().cuda_stream

    def timed(launch):
        for _ in range(max(2, warmup // 2)):
            launch()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(max(5, steps // 2))]
        for s, e in evs:
            sweep.sum()
            s.record()
            rc = launch()
            e.record()
            if rc != 0:
                raise RuntimeError(lib.m2_last_error().decode())
        torch.cuda.synchronize()
        t = sorted(s.elapsed_time(e) for s, e in evs)
        return t[len(t) // 2]

    moved = 2 * src.numel()
    rows_out = []
    cases = [("plain copy (stream_copy_kernel)", lambda: lib.m2_stream_copy(src.data_ptr(), dst.data_ptr(), src.numel(), stream()))]
    for piece, in_order, what in ((64, 1, "half-head tiles in chunk order, one workgroup per (batch, half head): the state passes' streams"),
                                  (128, 1, "whole-head tiles in chunk order, one workgroup per (batch, head)"),
                                  (128, 0, "whole-head tiles, one workgroup per tile: the chunk-parallel kernels' streams"),
                                  (256, 0, "two-head tiles, one workgroup per tile"),
                                  (512, 0, "four-head tiles, one workgroup per tile")):
        cases.append((f"{what} ({piece}-byte row pieces, {row_bytes} bytes apart)",
                      (lambda p, o: lambda: lib.m2_tile_walk(src.data_ptr(), dst.data_ptr(), batch, rows, row_bytes, p, o, stream()))(piece, in_order)))
    for name, launch in cases:
        ms = timed(launch)
        rows_out.append({"pattern": name, "us": ms * 1e3, "GB/s": moved / (ms * 1e-3) / 1e9})
    copy, head = rows_out[0], rows_out[3]
    return dict(metric="HBM rate of a no-arithmetic kernel with the SSD kernels' access pattern", value=head["GB/s"], unit="GB/s",
                ms_per_step=head["us"] * 1e-3, dtype="u8",
                config={"workload": f"tile_walk_kernel over x of the c1 shape ({src.numel() / 1e6:.0f} MB read + written), caches cleaned before each launch"},
                patterns=rows_out,
                roofline={"bound": "hbm", "achieved": head["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["GB/s"] / HBM_PEAK_GBS,
                          "traffic": None, "algorithmic_bytes_per_step": moved, "kernels": "tile_walk_kernel<8, false>",
                          "plain_copy_same_size_GBs": copy["GB/s"]})


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _cpu_cores():
    """Threads the CPU legs use: the box's CPU share (OMP_NUM_THREADS there), else every core the host reports."""
    import torch
    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    torch.set_num_threads(cores)
    return cores


def _cpu_info(cores):
    return {"cores": cores, "host_cpu_count": os.cpu_count(), "cpu_model": cpu_model()}


def cpu_baseline_ssd():
    """The pure-PyTorch chunked oracle (fp32 arithmetic, autograd) on the host cores: the full headline configuration,
    on the same seeded bf16-rounded inputs the GPU path gets.  Returns (baseline record, the oracle's results)."""
    import torch
    from oracle.ssd import make_ssd_inputs, ssd_grads_ref
    cores = _cpu_cores()
    cfg = SSD_CFG
    d = make_ssd_inputs(cfg["b"], cfg["l"], cfg["h"], cfg["p"], cfg["n"], cfg["g"], seed=0, dtype=torch.bfloat16)
    d = {k: v.float() for k, v in d.items()}
    times = []
    for i in range(4):
        t0 = time.perf_counter()
        ref = ssd_grads_ref(d["dt"], d["A"], d["X"], d["B"], d["C"], d["D"], d["dy"], chunk=Q)
        times.append(time.perf_counter() - t0)
    t = sorted(times[1:])[1]
    rec = {"value": cfg["b"] * cfg["l"] / t, "unit": "tokens/s", "kind": "port",
           "sample": "full workload (b4 l2048 h80 p64 n128), fp32, chunked-matmul oracle with autograd, 1 warm-up + median of 3",
           "seconds_per_step": t}
    rec.update(_cpu_info(cores))
    return rec, ref


def cpu_baseline_conv():
    """F.conv1d + SiLU with autograd (the conv oracle) on the host cores: the full conv workload, fp32."""
    import torch
    from oracle.conv import conv1d_grads_ref, make_conv_inputs
    cores = _cpu_cores()
    cfg = CONV_CFG
    d = make_conv_inputs(cfg["b"], cfg["l"], cfg["C"], cfg["k"], seed=0, dtype=torch.float32)
    times = []
    for _ in range(4):
        t0 = time.perf_counter()
        conv1d_grads_ref(d["x"], d["w"], d["bias"], d["dy"], "silu")
        times.append(time.perf_counter() - t0)
    t = sorted(times[1:])[1]
    rec = {"value": cfg["b"] * cfg["l"] / t, "unit": "tokens/s", "kind": "port", "seconds_per_step": t,
           "sample": "full workload (b4 l2048 C5376 k4), fp32, F.conv1d + SiLU with autograd, 1 warm-up + median of 3"}
    rec.update(_cpu_info(cores))
    return rec


def cpu_baseline_decode():
    """The decode oracle on the host cores: 2 of the 64 layers at batch 128 (fp32), scaled by 32 to a whole step."""
    import torch
    from oracle.decode import decode_step_ref, make_decode_inputs
    cores = _cpu_cores()
    cfg = DEC_CFG
    layers = 2
    q = [make_decode_inputs(cfg["b"], cfg["h"], cfg["p"], cfg["n"], cfg["g"], cfg["k"], cfg["W"], seed=s) for s in range(layers)]
    times = []
    for _ in range(4):
        t0 = time.perf_counter()
        for d in q:
            decode_step_ref(d["xBC"], d["conv_state"], d["conv_weight"], d["conv_bias"], d["S"], d["dt"], d["A"], d["D"], n_groups=cfg["g"])
        times.append(time.perf_counter() - t0)
    t = sorted(times[1:])[1] * cfg["layers"] / layers
    rec = {"value": t * 1e6, "unit": "us/step", "kind": "port", "seconds_per_step": t,
           "sample": "2 of the 64 layers (b128 h80 p64 n128, fp32, out-of-place oracle step), time scaled x32, 1 warm-up + median of 3"}
    rec.update(_cpu_info(cores))
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all", choices=["all", "ssd", "conv", "glue", "core", "layer", "decode", "model", "copy", "pattern"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-gemm-tuning", action="store_true",
                    help="model workload: capture the step with the BLAS libraries' default solutions (for kernel traces: the tuning runs would fill them)")
    ap.add_argument("--exclude", default="", help="comma-separated workloads to leave out of --workload all (for per-kernel profiles)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the hot path has no collective); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from mamba2 import _lib
    _lib.load()          # fails loudly when the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    out = {}
    other = {}
    skip = set(x for x in a.exclude.split(",") if x)

    def wanted(name):
        return a.workload == name or (a.workload == "all" and name not in skip)

    if wanted("ssd"):
        # the CPU leg runs first: its results (the oracle on the same inputs) are what the HIP outputs are checked against
        # before anything is timed; without it the check runs on a quarter of the batch and sequence
        cpu_rec, ref, check_cfg = None, None, None
        if a.no_cpu:
            check_cfg = dict(SSD_CFG, b=1, l=512)
        else:
            cpu_rec, ref = cpu_baseline_ssd()
        r = bench_ssd(a.steps, a.warmup, ref, check_cfg)
        del ref
        out.update({
            "metric": "SSD fwd+bwd tokens/s", "value": r["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1,
            "steps": a.steps, "warmup": a.warmup, "ms_per_step": r["ms_per_step"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "Mamba-2 2.7B-shaped SSD chunked scan fwd+bwd: b4 l2048 h80 p64 n128 g1 chunk128, bf16 I/O, fp32 state"},
            "roofline": {"bound": "mfma", "achieved": r["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": r["tflops"] / MFMA_BF16_PEAK_TFLOPS, "traffic": SSD_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                         "algorithmic_flops_per_step": r["flops"], "event_ms_avg": r["ms_event_avg"],
                         "event_ms_min": r["ms_event_min"],
                         "kernels": "all launches of m2_ssd_fwd + m2_ssd_bwd (one step), HIP events on the launch stream"},
            # the same step against the memory roofline: algorithmic I/O = x (forward), y, x (backward), dy, dx, B, C, dB, dC, dt, ddt
            "roofline_hbm": {"bound": "hbm", "achieved": r["io_bytes"] / (r["ms_event_avg"] * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": r["io_bytes"] / (r["ms_event_avg"] * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": SSD_TRAFFIC_BYTES,
                             "traffic_rate": SSD_TRAFFIC_BYTES / (r["ms_event_avg"] * 1e-3) / 1e9, "algorithmic_bytes_per_step": r["io_bytes"]},
            "parity": {"against": "oracle.ssd.ssd_grads_ref on the same seeded inputs, " + r["parity_shape"] + ", checked before timing",
                       "tensors": r["parity"]},
        })
        if cpu_rec is not None:
            out["cpu_baseline"] = cpu_rec
    def secondary(key, fn, *args):
        # with --workload all a failure in a secondary workload is reported in its place and does not take the headline
        # line with it; asked for by name, it fails loudly
        try:
            other[key] = fn(*args)
        except Exception as e:      # noqa: BLE001
            if a.workload != "all":
                raise
            other[key] = {"error": f"{type(e).__name__}: {e}"}

    if wanted("conv"):
        secondary("conv1d", bench_conv, a.steps, a.warmup)
    if wanted("glue"):
        secondary("mixer_glue", bench_glue, a.steps, a.warmup)
    if wanted("core"):
        secondary("mixer_core", bench_core, a.steps, a.warmup)
    if wanted("layer"):
        secondary("mixer_layer_c3", bench_layer_c3, max(5, a.steps // 2), max(2, a.warmup // 2))
    if wanted("decode"):
        secondary("decode", bench_decode, max(3, a.steps // 4), max(1, a.warmup // 2))
    if wanted("model"):
        secondary("decode_model", bench_model_step, max(3, a.steps // 4), max(1, a.warmup // 2), not a.no_gemm_tuning)
    if wanted("copy"):
        secondary("stream_copy", bench_copy, a.steps, a.warmup)
    if wanted("pattern"):
        secondary("access_pattern", bench_access_pattern, a.steps, a.warmup)
    if a.workload not in ("all", "ssd"):
        key = {"conv": "conv1d", "glue": "mixer_glue", "core": "mixer_core", "layer": "mixer_layer_c3", "decode": "decode", "model": "decode_model", "copy": "stream_copy", "pattern": "access_pattern"}[a.workload]
        out.update(other.pop(key))
        out.update({"n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "scaling": "weak", "vs_baseline": None, "data": "synthetic"})
        out.setdefault("higher_is_better", True)
    if other:
        out["other"] = other
    # the conv and decode oracles timed on the same host, next to their GPU lines
    if not a.no_cpu:
        for key, fn in (("conv1d", cpu_baseline_conv), ("decode", cpu_baseline_decode)):
            tgt = out.get("other", {}).get(key) if key in out.get("other", {}) else (out if out.get("metric", "").startswith(key[:4]) else None)
            if isinstance(tgt, dict) and "error" not in tgt:
                try:
                    tgt["cpu_baseline"] = fn()
                except Exception as e:      # noqa: BLE001
                    tgt["cpu_baseline"] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
