"""Weight formats around the model shell: state-spaces (``mamba_ssm``) and Codestral checkpoints into
``Mamba2ForCausalLM`` (``convert_mamba2_ssm_checkpoint.py:33-170``), the split-projection layout
(``:119-141``), and tensor-parallel shards of the reference's trainer merged into / cut from one state dict
(``merge_tp_checkpoints.py:6-72``, ``mamba2_inference_no_tp.py:142-165``).

Everything here is host-side tensor bookkeeping on CPU tensors.  Files are read with loaders that execute nothing
from the file: ``torch.load(..., weights_only=True)`` and safetensors.

Layouts (rows of a weight = output features):
  in_proj.weight   rows [z (d_inner) | x (d_inner) | B (g*n) | C (g*n) | dt (h)]     ``mamba2_mixer.py:156,265``
  conv1d.weight/.bias  rows [x | B | C]
  out_proj.weight  columns d_inner
A tensor-parallel rank holds, of every section, its contiguous 1/tp slice (heads, groups and channels are dealt out in
order, ``mamba2_mixer.py:192-206``); block norms, ``norm_f``, ``A_log``/``D``/``dt_bias``/``mixer.norm`` follow the same rule
(the block norms are replicated, the per-head and per-channel vectors are sliced).
"""
import json
import os
from typing import Dict, List

import torch

from .configuration_mamba2 import Mamba2Config

# names of the fields in the source config files (convert_mamba2_ssm_checkpoint.py:96-119)
MODEL_TYPES = {
    "codestral": {"hidden_size": "dim", "num_hidden_layers": "n_layers", "n_groups": "n_groups", "bos_token_id": 0, "pad_token_id": 1,
                  "eos_token_id": 2, "config_name": "params.json", "ckpt_name": "consolidated.safetensors"},
    "mamba_ssm": {"hidden_size": "d_model", "num_hidden_layers": "n_layer", "n_groups": "ngroups", "bos_token_id": 0, "pad_token_id": 0,
                  "eos_token_id": 0, "config_name": "config.json", "ckpt_name": "pytorch_model.bin"},
}


def convert_ssm_config(config_ssm: Dict, model_type: str = "mamba_ssm", **overrides) -> Mamba2Config:
    """Source config dict -> ``Mamba2Config``: heads from the width, groups (default 1, also read from the nested
    ``ssm_cfg`` of state-spaces configs), vocabulary padded to the stated multiple."""
    names = MODEL_TYPES[model_type]
    cfg = Mamba2Config(**overrides)
    cfg.hidden_size = config_ssm[names["hidden_size"]]
    cfg.num_heads = (cfg.hidden_size * cfg.expand) // cfg.head_dim
    cfg.num_hidden_layers = config_ssm[names["num_hidden_layers"]]
    nested = config_ssm.get("ssm_cfg") or {}
    cfg.n_groups = config_ssm.get(names["n_groups"], nested.get(names["n_groups"], 1))
    cfg.tie_word_embeddings = bool(config_ssm.get("tie_embeddings", False))
    cfg.bos_token_id, cfg.pad_token_id, cfg.eos_token_id = names["bos_token_id"], names["pad_token_id"], names["eos_token_id"]
    cfg.residual_in_fp32 = bool(config_ssm.get("residual_in_fp32", cfg.residual_in_fp32))
    vocab = config_ssm["vocab_size"]
    mult = config_ssm.get("pad_vocab_size_multiple", 1)
    if vocab % mult:
        vocab += mult - vocab % mult
    cfg.vocab_size = vocab
    cfg.time_step_rank = -(-cfg.hidden_size // 16)
    return cfg


def load_source_state_dict(checkpoint_dir: str, model_type: str = "mamba_ssm") -> Dict[str, torch.Tensor]:
    names = MODEL_TYPES[model_type]
    path = os.path.join(checkpoint_dir, names["ckpt_name"])
    if path.endswith(".safetensors"):
        from safetensors import safe_open
        out = {}
        with safe_open(path, framework="pt") as f:
            for k in f.keys():
                out[k[len("model."):] if k.startswith("model.") else k] = f.get_tensor(k).clone()
        return out
    return torch.load(path, map_location="cpu", weights_only=True)


def _mixer_dims(cfg):
    d_inner = int(cfg.expand * cfg.hidden_size)
    gn = cfg.n_groups * cfg.state_size
    return d_inner, gn, cfg.num_heads


def split_projection_matrix(state_dict, cfg):
    """in_proj.weight -> in_proj_z / in_proj_xBC / in_proj_dt (the reference's ``--split_proj`` layout)."""
    d_inner, gn, h = _mixer_dims(cfg)
    out = {}
    for k, v in state_dict.items():
        if not k.endswith("in_proj.weight"):
            out[k] = v
            continue
        base = k[:-len(".in_proj.weight")]
        w_z, w_xBC, w_dt = torch.split(v, [d_inner, d_inner + 2 * gn, h], dim=0)
        out[base + ".in_proj_z.weight"], out[base + ".in_proj_xBC.weight"], out[base + ".in_proj_dt.weight"] = (
            w_z.clone(), w_xBC.clone(), w_dt.clone())
    return out


def merge_projection_matrix(state_dict):
    """The inverse: in_proj_z / in_proj_xBC / in_proj_dt -> in_proj.weight (rows [z | xBC | dt])."""
    out = {k: v for k, v in state_dict.items() if ".in_proj_" not in k}
    for k in state_dict:
        if k.endswith(".in_proj_z.weight"):
            base = k[:-len(".in_proj_z.weight")]
            out[base + ".in_proj.weight"] = torch.cat([state_dict[base + ".in_proj_z.weight"], state_dict[base + ".in_proj_xBC.weight"],
                                                       state_dict[base + ".in_proj_dt.weight"]], dim=0)
    return out


def _sections(key, cfg):
    """Row sections of a sharded tensor, or None when it is sliced whole along dim 0."""
    d_inner, gn, h = _mixer_dims(cfg)
    if "conv1d" in key or key.endswith("in_proj_xBC.weight"):
        return [d_inner, gn, gn]
    if key.endswith("in_proj.weight"):
        return [d_inner, d_inner, gn, gn, h]
    return None


def _is_replicated(key):
    """Block norms and the final norm are the only tensors every rank holds whole (``merge_tp_checkpoints.py:66-67``,
    ``mamba2_inference_no_tp.py:157-158``); the embedding table and the LM head are sharded along the vocabulary like any
    other column-parallel tensor (``ParallelEmbedding`` / ``ColumnParallelLinear``; the loaders' else-branches)."""
    return "norm" in key and "mixer" not in key


def shard_state_dict(state_dict, rank: int, tp: int, cfg) -> Dict[str, torch.Tensor]:
    """The slice of a full state dict that tensor-parallel rank ``rank`` of ``tp`` holds (``mamba2_inference_no_tp.py:142-165``).
    Block norms are kept whole; the embedding table and the LM head are cut along the vocabulary."""
    if cfg.n_groups % tp or cfg.num_heads % tp:
        raise ValueError(f"n_groups {cfg.n_groups} and num_heads {cfg.num_heads} must be divisible by tp {tp}")
    for k, v in state_dict.items():
        if ("embedding" in k or k.startswith("lm_head")) and v.shape[0] % tp:
            raise ValueError(f"{k}: vocabulary {v.shape[0]} is not divisible by tp {tp}")
    out = {}
    for k, v in state_dict.items():
        if _is_replicated(k):
            out[k] = v
        elif k.endswith("out_proj.weight"):
            out[k] = torch.chunk(v, tp, dim=1)[rank].clone()
        else:
            sec = _sections(k, cfg)
            parts = torch.split(v, sec, dim=0) if sec else [v]
            out[k] = torch.cat([torch.chunk(p, tp, dim=0)[rank] for p in parts], dim=0).clone()
    return out


def merge_tp_state_dicts(shards: List[Dict[str, torch.Tensor]], cfg) -> Dict[str, torch.Tensor]:
    """Tensor-parallel shards (rank order) -> one state dict (``merge_tp_checkpoints.py:6-72``, for any number of groups per rank)."""
    tp = len(shards)
    out = {}
    for k, v in shards[0].items():
        if _is_replicated(k):
            out[k] = v
        elif k.endswith("out_proj.weight"):
            out[k] = torch.cat([s[k] for s in shards], dim=1)
        else:
            sec = _sections(k, cfg)
            if sec is None:
                out[k] = torch.cat([s[k] for s in shards], dim=0)
            else:
                per_rank = [torch.split(s[k], [n // tp for n in sec], dim=0) for s in shards]
                out[k] = torch.cat([torch.cat([pr[i] for pr in per_rank], dim=0) for i in range(len(sec))], dim=0)
    return out


def load_pretrained(checkpoint_dir: str, model_type: str = "mamba_ssm", dtype=torch.bfloat16, device="cuda", **config_overrides):
    """Directory with the source config + weights -> ``Mamba2ForCausalLM`` with those weights (split projections merged,
    the ``embedding`` table renamed by the model's load hook)."""
    from .modeling_mamba2 import Mamba2ForCausalLM
    with open(os.path.join(checkpoint_dir, MODEL_TYPES[model_type]["config_name"]), "r", encoding="utf-8") as f:
        cfg = convert_ssm_config(json.load(f), model_type, **config_overrides)
    sd = merge_projection_matrix(load_source_state_dict(checkpoint_dir, model_type))
    model = Mamba2ForCausalLM(cfg)
    if cfg.tie_word_embeddings and "lm_head.weight" not in sd:
        emb = [k for k in sd if k.endswith("embedding.weight") or k.endswith("embeddings.weight")]
        sd["lm_head.weight"] = sd[emb[0]]
    model.load_state_dict(sd)
    return model.to(device=device, dtype=dtype)
