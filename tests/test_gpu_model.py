"""GPU: the model shell (blocks, backbone, LM head) and the prefill -> decode hand-off.

What pins what:
* whole-model logits and gradients against an fp64 CPU restatement assembled from the oracle's pieces
  (oracle/mixer.py: fused_core_ref, rmsnorm_gated_ref) with the same weights;
* the reference's own inference check (mamba2_inference_no_tp.py:97-133): logits of ``model(input_ids)`` equal the
  logits of ``model.step`` fed one token at a time;
* the hand-off: forward over a prefix with a cache, then steps (or a second forward) over the rest, equals one forward
  over everything; the cache after a prefill equals the cache after stepping through the same tokens, and the conv state
  is literally the last W rows of the xBC columns;
* the captured decode step replays bit-exactly what the eager step computes.
"""
import pytest
import torch

from conftest import rel_err, rel_rms_err
from oracle.mixer import fused_core_ref, rmsnorm_gated_ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _model(dtype, layers=2, g=2, vocab=97, residual_in_fp32=True, tie=False):
    from mamba2.configuration_mamba2 import Mamba2Config
    from mamba2.modeling_mamba2 import Mamba2ForCausalLM
    cfg = Mamba2Config(num_heads=4, head_dim=64, hidden_size=128, state_size=64, n_groups=g, num_hidden_layers=layers, expand=2,
                       vocab_size=vocab, residual_in_fp32=residual_in_fp32, tie_word_embeddings=tie, initializer_range=0.5)
    torch.manual_seed(0)
    m = Mamba2ForCausalLM(cfg)
    with torch.no_grad():
        for blk in m.backbone.layers:
            blk.mixer.in_proj.weight.normal_(0, 0.08)
            blk.mixer.out_proj.weight.normal_(0, 0.08)
            blk.mixer.A_log.copy_(torch.log(torch.linspace(1.0, 8.0, cfg.num_heads)))
            blk.norm.weight.copy_(1.0 + 0.1 * torch.randn(cfg.hidden_size))
        m.lm_head.weight.normal_(0, 0.1)
    m = m.to(DEV)
    return cfg, (m.to(dtype) if dtype != torch.float32 else m).eval()


def _oracle_logits(m, cfg, ids):
    """fp64 CPU restatement of Mamba2ForCausalLM.forward with m's weights; returns (logits, dict of weight leaves)."""
    W = {k: v.detach().double().cpu().requires_grad_(True) for k, v in m.named_parameters()}
    d_inner = cfg.expand * cfg.hidden_size
    x = W["backbone.embeddings.weight"][ids]
    for i in range(cfg.num_hidden_layers):
        p = f"backbone.layers.{i}."
        hn = rmsnorm_gated_ref(x, None, W[p + "norm.weight"], 1, cfg.layer_norm_epsilon)
        z = hn @ W[p + "mixer.in_proj.weight"].T
        core = fused_core_ref(z, -torch.exp(W[p + "mixer.A_log"]), W[p + "mixer.D"], W[p + "mixer.conv1d.weight"],
                              W[p + "mixer.conv1d.bias"], W[p + "mixer.dt_bias"], W[p + "mixer.norm.weight"],
                              cfg.n_groups, cfg.state_size, d_inner, cfg.head_dim)
        x = x + core @ W[p + "mixer.out_proj.weight"].T
    hn = rmsnorm_gated_ref(x, None, W["backbone.norm_f.weight"], 1, cfg.layer_norm_epsilon)
    head = W["lm_head.weight"] if "lm_head.weight" in W else W["backbone.embeddings.weight"]
    return hn @ head.T, W


def _close(got, ref, dtype):
    """fp32: the fp32 bar (with head-room for the depth of the model).  bf16: activations are rounded to bf16 at every
    layer boundary, at different places in the sequence and the token-by-token paths, so the bar is statistical (relative
    L2) plus a loose bound on the worst element; the logic is pinned by the fp32 case of the same test."""
    if dtype == torch.float32:
        return rel_err(got, ref) < 5e-4
    g, r = got.double().cpu(), ref.double().cpu()
    return ((g - r).norm() / r.norm()).item() < 2e-2 and rel_rms_err(got.float(), ref) < 0.2


def test_model_parameter_names():
    cfg, m = _model(torch.float32)
    names = set(k for k, _ in m.named_parameters())
    for k in ("backbone.embeddings.weight", "backbone.layers.0.norm.weight", "backbone.layers.1.mixer.in_proj.weight",
              "backbone.layers.0.mixer.conv1d.weight", "backbone.layers.0.mixer.norm.weight", "backbone.norm_f.weight", "lm_head.weight"):
        assert k in names, k
    # a state-spaces style key for the table is accepted on load
    sd = {k.replace("embeddings.", "embedding."): v for k, v in m.state_dict().items()}
    m.load_state_dict(sd)
    _, tied = _model(torch.float32, tie=True)
    assert tied.lm_head.weight is tied.backbone.embeddings.weight


def test_model_logits_loss_and_grads_match_oracle():
    cfg, m = _model(torch.float32)
    m.train()
    ids = torch.randint(0, cfg.vocab_size, (2, 200), generator=torch.Generator().manual_seed(1))
    out = m(input_ids=ids.to(DEV), labels=ids.to(DEV))
    out.loss.backward()
    ref_logits, W = _oracle_logits(m, cfg, ids)
    ref_loss = torch.nn.functional.cross_entropy(ref_logits[:, :-1].reshape(-1, cfg.vocab_size), ids[:, 1:].reshape(-1))
    ref_loss.backward()
    assert out.logits.dtype == torch.float32 and out.logits.shape == (2, 200, cfg.vocab_size)
    assert rel_err(out.logits, ref_logits.detach()) < 5e-4
    assert abs(out.loss.item() - ref_loss.item()) < 1e-4 * max(1.0, abs(ref_loss.item()))
    for k, p in m.named_parameters():
        assert p.grad is not None, k
        assert rel_err(p.grad, W[k].grad) < 2e-3, k


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_step_logits_equal_forward_logits(dtype):
    from mamba2.mamba2_mixer import Mamba2Cache
    cfg, m = _model(dtype)
    b, l = 2, 140
    ids = torch.randint(0, cfg.vocab_size, (b, l), generator=torch.Generator().manual_seed(2)).to(DEV)
    with torch.no_grad():
        full = m(input_ids=ids).logits
        cache = Mamba2Cache(cfg, b, dtype=dtype, device=DEV)
        steps = torch.cat([m.step(ids[:, t:t + 1], cache) for t in range(l)], dim=1)
    ref_logits, _ = _oracle_logits(m, cfg, ids.cpu())
    assert _close(steps, full, dtype)
    assert _close(full, ref_logits.detach(), dtype)
    assert _close(steps, ref_logits.detach(), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("residual_in_fp32", [True, False])
def test_model_step_equals_block_by_block_steps(dtype, residual_in_fp32):
    """Mamba2Model.step (residual add fused with the next norm when the residual stream is fp32) against the blocks'
    own step methods chained by hand (modeling_mamba2.py:337-350)."""
    from mamba2.mamba2_mixer import Mamba2Cache
    cfg, m = _model(dtype, layers=3, residual_in_fp32=residual_in_fp32)
    b = 5
    ids = torch.randint(0, cfg.vocab_size, (b, 6), generator=torch.Generator().manual_seed(7)).to(DEV)
    c1 = Mamba2Cache(cfg, b, dtype=dtype, device=DEV)
    c2 = Mamba2Cache(cfg, b, dtype=dtype, device=DEV)
    with torch.no_grad():
        for t in range(6):
            got = m.backbone.step(ids[:, t:t + 1], c1)
            x = m.backbone.embeddings(ids[:, t:t + 1])
            for blk in m.backbone.layers:
                x = blk.step(x, cache_params=c2)
            ref = m.backbone.norm_f(x)
            if dtype == torch.float32:
                assert rel_err(got, ref) < 1e-5, t
            else:
                assert rel_rms_err(got, ref.float()) < 2e-2, t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [3, 4])
@pytest.mark.parametrize("l1,l2", [(130, 40), (2, 131), (256, 1)])
def test_prefill_hands_over_to_step_and_to_prefill(dtype, W, l1, l2):
    """forward(prefix, cache) then step x l2, or then forward(rest, cache), equals forward(everything)."""
    from mamba2.mamba2_mixer import Mamba2Cache
    cfg, m = _model(dtype)
    b = 2
    ids = torch.randint(0, cfg.vocab_size, (b, l1 + l2), generator=torch.Generator().manual_seed(3)).to(DEV)
    tol = lambda a, e: _close(a, e, dtype)
    with torch.no_grad():
        full = m(input_ids=ids).logits
        # prefix by prefill, rest by steps
        cache = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=W)
        pre = m(input_ids=ids[:, :l1], cache_params=cache, use_cache=True)
        assert pre.cache_params is cache and cache.seqlen_offset == l1
        assert tol(pre.logits, full[:, :l1])
        n_step = min(l2, 24)
        steps = torch.cat([m.step(ids[:, l1 + t:l1 + t + 1], cache) for t in range(n_step)], dim=1)
        assert tol(steps, full[:, l1:l1 + n_step])
        # prefix by prefill, rest by a second prefill that continues from the cache
        cache2 = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=W)
        m(input_ids=ids[:, :l1], cache_params=cache2, use_cache=True)
        rest = m(input_ids=ids[:, l1:], cache_params=cache2, use_cache=True)
        assert cache2.seqlen_offset == l1 + l2
        assert tol(rest.logits, full[:, l1:])
        # the cache after prefilling everything in two pieces == the cache after prefilling it in one
        cache3 = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=W)
        m(input_ids=ids, cache_params=cache3, use_cache=True)
        for i in range(cfg.num_hidden_layers):
            assert _close(cache2.ssm_states[i], cache3.ssm_states[i], dtype)
            assert _close(cache2.conv_states[i], cache3.conv_states[i], dtype)


@pytest.mark.parametrize("W", [3, 4])
def test_prefill_cache_contents(W):
    """After a prefill the conv state is the last W rows of the xBC columns and the SSM state that of the recurrence
    (compared with stepping through the same tokens from an empty cache)."""
    from mamba2.mamba2_mixer import Mamba2Cache
    from test_gpu_mixer import _mixer
    cfg, mix = _mixer(torch.float32)
    b, l = 2, 150
    x = torch.randn(b, l, 128, generator=torch.Generator().manual_seed(4)).to(DEV)
    d_inner = 256
    conv_dim = d_inner + 2 * cfg.n_groups * cfg.state_size
    with torch.no_grad():
        c_pre = Mamba2Cache(cfg, b, dtype=torch.float32, device=DEV, conv_width=W)
        y_pre = mix(x, cache_params=c_pre)
        c_step = Mamba2Cache(cfg, b, dtype=torch.float32, device=DEV, conv_width=W)
        y_step = torch.cat([mix.step(x[:, t:t + 1], c_step) for t in range(l)], dim=1)
        xBC = mix.in_proj(x)[..., d_inner:d_inner + conv_dim]
        y_plain = mix(x)
    assert torch.equal(y_pre, y_plain)             # the cache changes nothing in the outputs of a first prefill
    assert rel_err(y_step, y_pre) < 2e-4
    assert torch.equal(c_pre.conv_states[0], xBC[:, l - W:].transpose(1, 2))
    assert rel_err(c_step.conv_states[0], c_pre.conv_states[0]) < 1e-5       # (the one-row projections may round differently)
    assert rel_err(c_step.ssm_states[0], c_pre.ssm_states[0]) < 2e-4
    assert torch.equal(c_pre.ssm_states[1], torch.zeros_like(c_pre.ssm_states[1]))      # other layers' entries untouched
    # a sequence shorter than the conv state: zeros stay in front
    with torch.no_grad():
        c_short = Mamba2Cache(cfg, b, dtype=torch.float32, device=DEV, conv_width=W)
        mix(x[:, :2], cache_params=c_short)
    assert torch.equal(c_short.conv_states[0][..., :W - 2], torch.zeros(b, conv_dim, W - 2, device=DEV))
    assert rel_err(c_short.conv_states[0][..., W - 2:], xBC[:, :2].transpose(1, 2)) < 1e-5
    with pytest.raises(AssertionError):            # the prefill is an inference path
        mix(x, cache_params=c_short)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_graphed_step_replays_equal_eager_steps(dtype):
    from mamba2.mamba2_mixer import Mamba2Cache
    from mamba2.modeling_mamba2 import GraphedStep
    cfg, m = _model(dtype, layers=3)
    b = 3
    ids = torch.randint(0, cfg.vocab_size, (b, 40), generator=torch.Generator().manual_seed(5)).to(DEV)
    cache_g = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=3)
    cache_e = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=3)
    with torch.no_grad():
        # both caches start from the same prefilled prefix
        m(input_ids=ids[:, :17], cache_params=cache_g, use_cache=True)
        m(input_ids=ids[:, :17], cache_params=cache_e, use_cache=True)
    step = GraphedStep(m, cache_g, b)
    for i in range(cfg.num_hidden_layers):          # capture and warm-up left the states where they were
        assert torch.equal(cache_g.ssm_states[i], cache_e.ssm_states[i]) and torch.equal(cache_g.conv_states[i], cache_e.conv_states[i])
    for t in range(17, 40):
        got = step(ids[:, t:t + 1]).clone()
        torch.cuda.synchronize()
        with torch.no_grad():
            ref = m.step(ids[:, t:t + 1], cache_e)           # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, ref), t
    for i in range(cfg.num_hidden_layers):
        assert torch.equal(cache_g.ssm_states[i], cache_e.ssm_states[i]) and torch.equal(cache_g.conv_states[i], cache_e.conv_states[i])
    # the same graph serves a new sequence after the cache is refilled
    cache_g.reset(); cache_e.reset()
    with torch.no_grad():
        m(input_ids=ids[:, 5:9], cache_params=cache_g, use_cache=True)
        m(input_ids=ids[:, 5:9], cache_params=cache_e, use_cache=True)
        assert torch.equal(step(ids[:, 9:10]), m.step(ids[:, 9:10], cache_e))


def test_graphed_step_with_tuned_gemms_agrees_with_eager():
    """tune_gemms: the captured projections may be other library solutions than the eager ones; replays agree with the eager
    step to bf16 accuracy, the process-wide TunableOp switches are back where they were, and nothing keeps tuning."""
    import torch.cuda.tunable as tunable
    from mamba2.mamba2_mixer import Mamba2Cache
    from mamba2.modeling_mamba2 import GraphedStep
    dtype = torch.bfloat16
    cfg, m = _model(dtype, layers=2)
    b = 4
    ids = torch.randint(0, cfg.vocab_size, (b, 30), generator=torch.Generator().manual_seed(9)).to(DEV)
    cache_g = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=3)
    cache_e = Mamba2Cache(cfg, b, dtype=dtype, device=DEV, conv_width=3)
    with torch.no_grad():
        m(input_ids=ids[:, :9], cache_params=cache_g, use_cache=True)
        m(input_ids=ids[:, :9], cache_params=cache_e, use_cache=True)
    before = (tunable.is_enabled(), tunable.tuning_is_enabled())
    step = GraphedStep(m, cache_g, b, tune_gemms=True)
    assert (tunable.is_enabled(), tunable.tuning_is_enabled()) == before
    for i in range(cfg.num_hidden_layers):          # capture, tuning runs and warm-up left the states where they were
        assert torch.equal(cache_g.ssm_states[i], cache_e.ssm_states[i]) and torch.equal(cache_g.conv_states[i], cache_e.conv_states[i])
    for t in range(9, 30):
        got = step(ids[:, t:t + 1]).clone()
        torch.cuda.synchronize()
        with torch.no_grad():
            ref = m.step(ids[:, t:t + 1], cache_e)
        torch.cuda.synchronize()
        g_, r_ = got.double(), ref.double()
        assert ((g_ - r_).norm() / r_.norm()).item() < 2e-2, t          # two bf16 evaluations of the same step
    for i in range(cfg.num_hidden_layers):
        assert rel_err(cache_g.ssm_states[i], cache_e.ssm_states[i]) < 2e-2


def test_decode_step_softplus_inside_matches_softplus_outside():
    """m2_decode_step with dt_bias (raw dt) against the same step fed softplus(dt + dt_bias) computed by the oracle."""
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    from oracle.decode import make_decode_inputs
    from oracle.mixer import softplus_ref
    b, h, p, n, g = 4, 8, 64, 128, 2
    q = {k: v.to(DEV) for k, v in make_decode_inputs(b, h, p, n, g, W=3, seed=1).items()}
    gen = torch.Generator().manual_seed(6)
    raw = (torch.randn(b, 1, h, generator=gen) * 6.0).to(DEV)            # both sides of the threshold
    bias = torch.randn(h, generator=gen).to(DEV)
    dt = softplus_ref(raw.double() + bias.double()).float()
    S1, S2 = q["S"].clone(), q["S"].clone()
    c1, c2 = q["conv_state"].clone(), q["conv_state"].clone()
    y1, _, _ = mamba2_kernel_inference(q["xBC"], c1, q["conv_weight"], q["conv_bias"], S1, raw, q["A"], q["D"], n_groups=g, dt_bias=bias)
    y2, _, _ = mamba2_kernel_inference(q["xBC"], c2, q["conv_weight"], q["conv_bias"], S2, dt, q["A"], q["D"], n_groups=g)
    assert rel_err(y1, y2) < 1e-5 and rel_err(S1, S2) < 1e-5 and torch.equal(c1, c2)


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_generate_matches_recomputing_the_prefix(use_graph):
    """Prefill + (captured) steps pick the same tokens as running the whole sequence again for every new token."""
    from mamba2.modeling_mamba2 import greedy_generate
    cfg, m = _model(torch.float32, layers=2)
    prompt = torch.randint(0, cfg.vocab_size, (3, 37), generator=torch.Generator().manual_seed(8)).to(DEV)
    got = greedy_generate(m, prompt, 12, use_graph=use_graph, conv_width=3)
    seq = prompt
    with torch.no_grad():
        for _ in range(12):
            logits = m(input_ids=seq).logits[:, -1]
            top2 = logits.topk(2, dim=-1).values
            assert ((top2[:, 0] - top2[:, 1]) > 1e-3).all(), "near tie: the comparison of token ids would not be meaningful"
            seq = torch.cat([seq, logits.argmax(-1, keepdim=True)], dim=1)
    assert got.shape == (3, 49) and torch.equal(got, seq)
