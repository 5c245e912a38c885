"""CPU: weight-format bookkeeping (mamba2/checkpoint.py) on small synthetic checkpoints written in the source formats
the reference converts (convert_mamba2_ssm_checkpoint.py, merge_tp_checkpoints.py).  No kernels run here."""
import json
import os

import pytest
import torch


def _cfg(**kw):
    from mamba2.configuration_mamba2 import Mamba2Config
    base = dict(num_heads=4, head_dim=64, hidden_size=128, state_size=32, n_groups=2, num_hidden_layers=2, expand=2, vocab_size=64)
    base.update(kw)
    return Mamba2Config(**base)


def _random_model(cfg, seed=0):
    from mamba2.modeling_mamba2 import Mamba2ForCausalLM
    torch.manual_seed(seed)
    m = Mamba2ForCausalLM(cfg)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn_like(p))
    return m


def test_config_conversion_pads_vocab_and_derives_heads():
    from mamba2.checkpoint import convert_ssm_config
    c = convert_ssm_config({"d_model": 2560, "n_layer": 64, "vocab_size": 50277, "pad_vocab_size_multiple": 16, "tie_embeddings": True,
                            "ssm_cfg": {"layer": "Mamba2"}}, "mamba_ssm")
    assert (c.hidden_size, c.num_hidden_layers, c.num_heads, c.n_groups, c.vocab_size) == (2560, 64, 80, 1, 50288)
    assert c.tie_word_embeddings and c.pad_token_id == 0
    c = convert_ssm_config({"dim": 4096, "n_layers": 64, "n_groups": 8, "vocab_size": 32768, "tie_embeddings": False}, "codestral")
    assert (c.hidden_size, c.num_heads, c.n_groups, c.vocab_size, c.pad_token_id, c.eos_token_id) == (4096, 128, 8, 32768, 1, 2)


def test_split_and_merge_projection_round_trip():
    from mamba2.checkpoint import merge_projection_matrix, split_projection_matrix
    cfg = _cfg()
    sd = _random_model(cfg).state_dict()
    sp = split_projection_matrix(sd, cfg)
    k = "backbone.layers.1.mixer."
    assert k + "in_proj.weight" not in sp
    assert sp[k + "in_proj_z.weight"].shape == (256, 128) and sp[k + "in_proj_xBC.weight"].shape == (256 + 128, 128)
    assert sp[k + "in_proj_dt.weight"].shape == (4, 128)
    assert torch.equal(sp[k + "in_proj_xBC.weight"], sd[k + "in_proj.weight"][256:256 + 384])
    back = merge_projection_matrix(sp)
    assert back.keys() == sd.keys() and all(torch.equal(back[n], sd[n]) for n in sd)


@pytest.mark.parametrize("tp", [1, 2])
def test_tp_shard_then_merge_is_identity(tp):
    from mamba2.checkpoint import merge_tp_state_dicts, shard_state_dict
    cfg = _cfg()
    sd = _random_model(cfg, seed=1).state_dict()
    shards = [shard_state_dict(sd, r, tp, cfg) for r in range(tp)]
    k = "backbone.layers.0.mixer."
    if tp == 2:
        s1 = shards[1]
        assert s1[k + "out_proj.weight"].shape == (128, 128) and torch.equal(s1[k + "out_proj.weight"], sd[k + "out_proj.weight"][:, 128:])
        # rank 1 of in_proj: second half of z, of x, group 1 of B, group 1 of C, heads 2-3 of dt
        w = sd[k + "in_proj.weight"]
        want = torch.cat([w[128:256], w[256 + 128:512], w[512 + 32:512 + 64], w[576 + 32:576 + 64], w[640 + 2:640 + 4]])
        assert torch.equal(s1[k + "in_proj.weight"], want)
        cw = sd[k + "conv1d.weight"]
        assert torch.equal(s1[k + "conv1d.weight"], torch.cat([cw[128:256], cw[256 + 32:256 + 64], cw[320 + 32:320 + 64]]))
        assert torch.equal(s1[k + "A_log"], sd[k + "A_log"][2:]) and torch.equal(s1[k + "norm.weight"], sd[k + "norm.weight"][128:])
        assert torch.equal(s1["backbone.layers.0.norm.weight"], sd["backbone.layers.0.norm.weight"])      # replicated
        # the embedding table and the LM head are cut along the vocabulary (mamba2_inference_no_tp.py:159-162)
        v = sd["backbone.embeddings.weight"].shape[0]
        assert torch.equal(s1["backbone.embeddings.weight"], sd["backbone.embeddings.weight"][v // 2:])
        assert torch.equal(s1["lm_head.weight"], sd["lm_head.weight"][v // 2:])
    merged = merge_tp_state_dicts(shards, cfg)
    assert merged.keys() == sd.keys() and all(torch.equal(merged[n], sd[n]) for n in sd)
    with pytest.raises(ValueError):
        shard_state_dict(sd, 0, 3, cfg)


def test_merge_shards_built_the_trainers_way():
    """Shards cut the way the reference's loader cuts them (mamba2_inference_no_tp.py:142-165, written out here
    independently of shard_state_dict: one group per rank, n_groups == tp as the trainer forces, train.py:44) merge back
    into the full state dict, vocabulary-split table and head included (merge_tp_checkpoints.py:6-72)."""
    from mamba2.checkpoint import merge_tp_state_dicts, shard_state_dict
    cfg = _cfg(vocab_size=48)
    sd = _random_model(cfg, seed=5).state_dict()
    tp = cfg.n_groups
    d_inner, gn, h = cfg.num_heads * cfg.head_dim, cfg.n_groups * cfg.state_size, cfg.num_heads

    def cut(v, sections, r):
        return torch.cat([torch.split(part, part.shape[0] // tp, dim=0)[r] for part in torch.split(v, sections, dim=0)], dim=0)

    shards = []
    for r in range(tp):
        sh = {}
        for k, v in sd.items():
            if k.endswith("out_proj.weight"):
                sh[k] = torch.split(v, v.shape[1] // tp, dim=1)[r]
            elif "conv1d" in k:
                sh[k] = cut(v, [d_inner, gn, gn], r)
            elif k.endswith("in_proj.weight"):
                sh[k] = cut(v, [d_inner, d_inner, gn, gn, h], r)
            elif "norm" in k and "mixer" not in k:
                sh[k] = v
            else:
                sh[k] = torch.split(v, v.shape[0] // tp, dim=0)[r]
        shards.append(sh)
    assert shards[0]["backbone.embeddings.weight"].shape[0] == 48 // tp and shards[1]["lm_head.weight"].shape[0] == 48 // tp
    merged = merge_tp_state_dicts(shards, cfg)
    assert merged.keys() == sd.keys() and all(torch.equal(merged[n], sd[n]) for n in sd)
    for r in range(tp):
        mine = shard_state_dict(sd, r, tp, cfg)
        assert all(torch.equal(mine[n], shards[r][n]) for n in sd), r


def test_load_state_spaces_and_codestral_directories(tmp_path):
    from mamba2.checkpoint import load_pretrained, split_projection_matrix
    cfg = _cfg(vocab_size=48)
    src = _random_model(cfg, seed=2)
    sd = src.state_dict()
    # state-spaces layout: "embedding" table, torch-saved tensors, config.json with d_model / n_layer / ssm_cfg.ngroups
    d1 = tmp_path / "ssm"; d1.mkdir()
    torch.save({k.replace("embeddings.", "embedding."): v for k, v in sd.items()}, d1 / "pytorch_model.bin")
    json.dump({"d_model": 128, "n_layer": 2, "vocab_size": 45, "pad_vocab_size_multiple": 16, "tie_embeddings": False,
               "ssm_cfg": {"ngroups": 2}}, open(d1 / "config.json", "w"))
    m1 = load_pretrained(str(d1), "mamba_ssm", dtype=torch.float32, device="cpu", state_size=32, num_heads=4)
    assert all(torch.equal(v, sd[k]) for k, v in m1.state_dict().items())
    # Codestral layout: safetensors with a "model." prefix, params.json with dim / n_layers / n_groups; split projections
    from safetensors.torch import save_file
    d2 = tmp_path / "codestral"; d2.mkdir()
    sp = split_projection_matrix({k.replace("embeddings.", "embedding."): v for k, v in sd.items()}, cfg)
    save_file({"model." + k: v.contiguous() for k, v in sp.items()}, str(d2 / "consolidated.safetensors"))
    json.dump({"dim": 128, "n_layers": 2, "n_groups": 2, "vocab_size": 48, "tie_embeddings": False}, open(d2 / "params.json", "w"))
    m2 = load_pretrained(str(d2), "codestral", dtype=torch.float32, device="cpu", state_size=32, num_heads=4)
    assert all(torch.equal(v, sd[k]) for k, v in m2.state_dict().items())
    # tied embeddings: the head is the table
    d3 = tmp_path / "tied"; d3.mkdir()
    tied = {k.replace("embeddings.", "embedding."): v for k, v in sd.items() if not k.startswith("lm_head")}
    torch.save(tied, d3 / "pytorch_model.bin")
    json.dump({"d_model": 128, "n_layer": 2, "vocab_size": 48, "pad_vocab_size_multiple": 8, "tie_embeddings": True,
               "ssm_cfg": {"ngroups": 2}}, open(d3 / "config.json", "w"))
    m3 = load_pretrained(str(d3), "mamba_ssm", dtype=torch.float32, device="cpu", state_size=32, num_heads=4)
    assert m3.lm_head.weight is m3.backbone.embeddings.weight
    assert torch.equal(m3.lm_head.weight, sd["backbone.embeddings.weight"])
