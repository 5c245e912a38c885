"""GPU: the reference's own two integration checks, at their shapes.

* tests/mamba2_kernel_test_no_tp.py:203-268 -- 2048 decode steps against conv1d + the chunked scan over the same 2048 tokens:
  batch 3, the Mamba370M layer (d_model 1024 -> d_inner 2048, head_dim 128 -> 16 heads, d_state 128), n_groups 8, conv
  state of width 4 (= the kernel width), fp32, SiLU on all of [x | B | C].  The reference's final assert compares against
  the last step only, on inputs scaled so that every output is ~0; the intent is adopted instead: the WHOLE sequence, the
  final SSM state and the final conv state are compared, on the benchmark's input recipe, and both device paths are also
  held against the fp64 oracle.
* tests/xla_mamba2_ssm_checkpoint_forward.py:33-47 -- load a converted checkpoint directory, left-pad the ids to the chunk
  size, one forward, logits shape; here the directory is a synthetic one in the state-spaces layout (and the Codestral
  layout with split projections, and a tied head), and the logits are compared with the oracle on the same tensors.
"""
import json
import math

import pytest
import torch

from conftest import rel_err
from oracle.conv import conv1d_ref
from oracle.mixer import fused_core_ref, rmsnorm_gated_ref
from oracle.ssd import ssd_recurrent_ref

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]
DEV = "cuda:0"


def test_2048_decode_steps_equal_conv_plus_scan_mamba370m():
    from mamba2.conv1d_grouped import conv1d_forward
    from mamba2.mamba2_kernel import mamba2_kernel
    from mamba2.mamba2_kernel_inference import mamba2_kernel_inference
    b, l, g, k = 3, 2048, 8, 4
    d_inner, p, n = 2048, 128, 128
    h = d_inner // p
    Cx = d_inner + 2 * g * n
    gen = torch.Generator().manual_seed(0)
    xBC = torch.randn(b, l, Cx, generator=gen)
    xBC[..., d_inner:] /= math.sqrt(n)
    w = torch.rand(Cx, k, generator=gen) - 0.5
    bias = torch.rand(Cx, generator=gen) - 0.5
    dt = torch.exp(torch.empty(b, l, h).uniform_(math.log(1e-3), math.log(1e-1), generator=gen))
    A = -torch.exp(torch.empty(h).uniform_(0.0, math.log(16.0), generator=gen))
    D = torch.ones(h)
    xd, wd, bd, dtd, Ad, Dd = (t.to(DEV) for t in (xBC, w, bias, dt, A, D))

    # token by token: conv state (b, Cx, 4) and SSM state start at zero and are updated in place
    conv_state = torch.zeros(b, Cx, k, device=DEV)
    S = torch.zeros(b, h, p, n, device=DEV)
    ys = []
    for t in range(l):
        y, conv_state, S = mamba2_kernel_inference(xd[:, t:t + 1], conv_state, wd, bd, S, dtd[:, t:t + 1], Ad, Dd, n_groups=g)
        ys.append(y)
    y_steps = torch.cat(ys, dim=1)

    # the sequence path: conv1d + SiLU over all of [x | B | C], then the chunked scan on views of the packed conv output
    conv_out = conv1d_forward(xd, wd[:, None, :], bd, "silu", channels_last=True)
    X = conv_out[..., :d_inner].unflatten(-1, (h, p))
    Bm = conv_out[..., d_inner:d_inner + g * n].unflatten(-1, (g, n))
    Cm = conv_out[..., d_inner + g * n:].unflatten(-1, (g, n))
    y_seq, S_seq = mamba2_kernel(dtd, Ad, X, Bm, Cm, Dd, return_final_state=True)
    y_seq = y_seq.reshape(b, l, d_inner)

    assert torch.isfinite(y_steps).all() and torch.isfinite(y_seq).all()
    assert rel_err(y_steps, y_seq) < 1e-4
    assert rel_err(S, S_seq) < 1e-4
    # the conv state holds the last 4 inputs, oldest first
    assert torch.equal(conv_state, xd[:, l - k:].transpose(1, 2))

    # both against the fp64 oracle: conv, then the token recurrence
    co = torch.nn.functional.silu(conv1d_ref(xBC.double(), w.double()[:, None, :], bias.double(), None, channels_last=True))
    y_ref, S_ref = ssd_recurrent_ref(dt.double(), A.double(), co[..., :d_inner].unflatten(-1, (h, p)),
                                     co[..., d_inner:d_inner + g * n].unflatten(-1, (g, n)), co[..., d_inner + g * n:].unflatten(-1, (g, n)),
                                     D.double())
    y_ref = y_ref.reshape(b, l, d_inner)
    assert rel_err(y_steps.cpu(), y_ref) < 1e-4 and rel_err(y_seq.cpu(), y_ref) < 1e-4
    assert rel_err(S.cpu(), S_ref) < 1e-4 and rel_err(S_seq.cpu(), S_ref) < 1e-4


def _source_model(seed, tie):
    from mamba2.configuration_mamba2 import Mamba2Config
    from mamba2.modeling_mamba2 import Mamba2ForCausalLM
    cfg = Mamba2Config(num_heads=4, head_dim=64, hidden_size=128, state_size=64, n_groups=2, num_hidden_layers=2, expand=2,
                       vocab_size=96, tie_word_embeddings=tie, initializer_range=0.5)
    torch.manual_seed(seed)
    m = Mamba2ForCausalLM(cfg)
    with torch.no_grad():
        for blk in m.backbone.layers:
            blk.mixer.in_proj.weight.normal_(0, 0.08)
            blk.mixer.out_proj.weight.normal_(0, 0.08)
            blk.norm.weight.copy_(1.0 + 0.1 * torch.randn(cfg.hidden_size))
    return cfg, m


def _oracle_logits(sd, cfg, ids):
    W = {k: v.detach().double().cpu() for k, v in sd.items()}
    d_inner = cfg.expand * cfg.hidden_size
    x = W["backbone.embeddings.weight"][ids]
    for i in range(cfg.num_hidden_layers):
        q = f"backbone.layers.{i}."
        hn = rmsnorm_gated_ref(x, None, W[q + "norm.weight"], 1, cfg.layer_norm_epsilon)
        core = fused_core_ref(hn @ W[q + "mixer.in_proj.weight"].T, -torch.exp(W[q + "mixer.A_log"]), W[q + "mixer.D"],
                              W[q + "mixer.conv1d.weight"], W[q + "mixer.conv1d.bias"], W[q + "mixer.dt_bias"],
                              W[q + "mixer.norm.weight"], cfg.n_groups, cfg.state_size, d_inner, cfg.head_dim)
        x = x + core @ W[q + "mixer.out_proj.weight"].T
    hn = rmsnorm_gated_ref(x, None, W["backbone.norm_f.weight"], 1, cfg.layer_norm_epsilon)
    return hn @ W.get("lm_head.weight", W["backbone.embeddings.weight"]).T


@pytest.mark.parametrize("layout", ["state_spaces", "codestral_split", "state_spaces_tied"])
def test_checkpoint_directory_to_device_logits(tmp_path, layout):
    from mamba2.checkpoint import load_pretrained, split_projection_matrix
    tie = layout.endswith("tied")
    cfg, src = _source_model(3, tie)
    sd = src.state_dict()
    renamed = {k.replace("embeddings.", "embedding."): v for k, v in sd.items() if not (tie and k.startswith("lm_head"))}
    if layout.startswith("state_spaces"):
        torch.save(renamed, tmp_path / "pytorch_model.bin")
        json.dump({"d_model": 128, "n_layer": 2, "vocab_size": 90, "pad_vocab_size_multiple": 16, "tie_embeddings": tie,
                   "ssm_cfg": {"ngroups": 2}}, open(tmp_path / "config.json", "w"))
        model = load_pretrained(str(tmp_path), "mamba_ssm", dtype=torch.float32, device=DEV, state_size=64, num_heads=4)
    else:
        from safetensors.torch import save_file
        sp = split_projection_matrix(renamed, cfg)
        assert not any(k.endswith("in_proj.weight") for k in sp)
        save_file({"model." + k: v.contiguous() for k, v in sp.items()}, str(tmp_path / "consolidated.safetensors"))
        json.dump({"dim": 128, "n_layers": 2, "n_groups": 2, "vocab_size": 96, "tie_embeddings": False}, open(tmp_path / "params.json", "w"))
        model = load_pretrained(str(tmp_path), "codestral", dtype=torch.float32, device=DEV, state_size=64, num_heads=4)
    model.eval()
    assert next(model.parameters()).is_cuda
    if tie:
        assert model.lm_head.weight is model.backbone.embeddings.weight
    # the reference's forward check: left-pad to a multiple of the chunk size with the pad token, one forward
    ids = torch.randint(1, 90, (1, 37), generator=torch.Generator().manual_seed(4))
    pad_len = model.config.chunk_size - (ids.shape[1] % model.config.chunk_size)
    ids = torch.nn.functional.pad(ids, (pad_len, 0), value=model.config.pad_token_id)
    assert ids.shape[1] % model.config.chunk_size == 0
    with torch.no_grad():
        logits = model(input_ids=ids.to(DEV)).logits
    assert logits.shape == (1, ids.shape[1], 96)
    ref = _oracle_logits(sd, cfg, ids)
    assert rel_err(logits, ref) < 5e-4
