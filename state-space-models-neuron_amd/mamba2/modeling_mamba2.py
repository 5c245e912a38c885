"""The model shell around the mixer with the reference's module interface (``mamba2/modeling_mamba2.py``):
``Mamba2RMSNorm`` (``:86-103``), ``Mamba2Block`` (``:106-140``), ``Mamba2Model`` (``:220-350``) and
``Mamba2ForCausalLM`` (``:359-531``), each with ``forward`` (whole sequences) and ``step`` (one token against a
``Mamba2Cache``), on one MI355X: the parallel embedding and linears of the reference are ``nn.Embedding`` and
``nn.Linear`` (tp = 1), parameter names are the reference's (``backbone.embeddings``, ``backbone.layers.N.norm``,
``backbone.layers.N.mixer.*``, ``backbone.norm_f``, ``lm_head``), and the lazy-graph cuts (``xm.mark_step``) have no
counterpart.  ``forward`` with ``cache_params`` and ``use_cache=True`` is the prefill that hands over to ``step``.

``GraphedStep`` captures ``Mamba2ForCausalLM.step`` for a fixed batch size into one HIP graph: a decode step of a
64-layer model is several hundred short launches, which replay as one submission (the reference's step loop,
``mamba2_inference_no_tp.py:108-127``, cuts one lazy graph per layer instead).
"""
import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn

from . import glue
from .configuration_mamba2 import Mamba2Config
from .mamba2_mixer import Mamba2Cache, Mamba2Mixer


class Mamba2RMSNorm(nn.Module):
    """weight * x * rsqrt(mean(x^2) + eps), computed in fp32, returned in the input's dtype (``modeling_mamba2.py:94-103``)."""

    def __init__(self, hidden_size, eps=1e-6, sequence_parallel_enabled=False):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, hidden_states):
        # the gated, grouped norm kernel with no gate and one group is this norm
        return glue.rmsnorm_gated_fn(hidden_states, None, self.weight, 1, self.variance_epsilon, out_dtype=hidden_states.dtype)


class Mamba2Block(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.residual_in_fp32 = config.residual_in_fp32
        self.norm = Mamba2RMSNorm(config.hidden_size, eps=config.layer_norm_epsilon)
        self.mixer = Mamba2Mixer(config, layer_idx=layer_idx)

    def _normed(self, x):
        # the residual stream may be fp32 while the projections hold bf16 weights
        return self.norm(x).to(self.mixer.in_proj.weight.dtype)

    def forward(self, hidden_states, cache_params: Optional[Mamba2Cache] = None, cache_position: Optional[torch.LongTensor] = None,
                attention_mask: Optional[torch.Tensor] = None):
        residual = hidden_states
        if self.residual_in_fp32:
            residual = residual.to(torch.float32)
        hidden_states = self.mixer(self._normed(hidden_states), cache_params=cache_params, cache_position=cache_position,
                                   attention_mask=attention_mask)
        return residual + hidden_states

    def step(self, x, cache_params: Optional[Mamba2Cache] = None):
        residual = x
        if self.residual_in_fp32:
            residual = residual.to(torch.float32)
        return self.mixer.step(self._normed(x), cache_params=cache_params) + residual


@dataclass
class Mamba2Output:
    last_hidden_state: Optional[torch.Tensor] = None
    cache_params: Optional[Mamba2Cache] = None
    hidden_states: Optional[Tuple[torch.Tensor, ...]] = None


@dataclass
class Mamba2CausalLMOutput:
    loss: Optional[torch.Tensor] = None
    logits: Optional[torch.Tensor] = None
    cache_params: Optional[Mamba2Cache] = None
    hidden_states: Optional[Tuple[torch.Tensor, ...]] = None


class Mamba2PreTrainedModel(nn.Module):
    """Weight initialisation of the reference (``modeling_mamba2.py:155-189``)."""
    config_class = Mamba2Config
    base_model_prefix = "backbone"

    def __init__(self, config):
        super().__init__()
        self.config = config

    def _init_weights(self, module):
        if isinstance(module, Mamba2Mixer):
            module.A_log._no_weight_decay = True
            module.D._no_weight_decay = True
        elif isinstance(module, nn.Linear):
            if module.bias is not None and not getattr(module.bias, "_no_reinit", False):
                nn.init.zeros_(module.bias)
        elif isinstance(module, nn.Embedding):
            nn.init.normal_(module.weight, std=self.config.initializer_range)
        if self.config.rescale_prenorm_residual:
            # residual-path projections scaled by 1/sqrt(number of layers)
            for name, p in module.named_parameters(recurse=False):
                if name == "weight" and getattr(module, "_is_out_proj", False):
                    nn.init.kaiming_uniform_(p, a=math.sqrt(5))
                    with torch.no_grad():
                        p /= math.sqrt(self.config.num_hidden_layers)

    def post_init(self):
        for blk in getattr(self, "layers", []):
            blk.mixer.out_proj._is_out_proj = True
        self.apply(self._init_weights)

    @property
    def device(self):
        return next(self.parameters()).device


class Mamba2Model(Mamba2PreTrainedModel):
    def __init__(self, config):
        super().__init__(config)
        self.embeddings = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([Mamba2Block(config, layer_idx=idx) for idx in range(config.num_hidden_layers)])
        self.gradient_checkpointing = False
        self.norm_f = Mamba2RMSNorm(config.hidden_size, eps=config.layer_norm_epsilon)
        self._register_load_state_dict_pre_hook(self.load_hook)
        self.post_init()

    def load_hook(self, state_dict, prefix, *args):
        # state-spaces checkpoints name the table "embedding" (modeling_mamba2.py:236-240)
        for k in list(state_dict):
            if "embedding." in k:
                state_dict[k.replace("embedding.", "embeddings.")] = state_dict.pop(k)

    def get_input_embeddings(self):
        return self.embeddings

    def set_input_embeddings(self, new_embeddings):
        self.embeddings = new_embeddings

    def forward(self, input_ids: Optional[torch.LongTensor] = None, inputs_embeds: Optional[torch.Tensor] = None,
                cache_params: Optional[Mamba2Cache] = None, use_cache: Optional[bool] = None,
                output_hidden_states: Optional[bool] = None, return_dict: Optional[bool] = None,
                cache_position: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None, **kwargs):
        if (input_ids is None) == (inputs_embeds is None):
            raise ValueError("You cannot specify both input_ids and inputs_embeds at the same time, and must specify either one")
        use_cache = bool(use_cache) if use_cache is not None else (cache_params is not None and not self.training)
        return_dict = True if return_dict is None else return_dict
        if inputs_embeds is None:
            inputs_embeds = self.embeddings(input_ids)
        if use_cache and cache_params is None:
            cache_params = Mamba2Cache(self.config, inputs_embeds.size(0), device=inputs_embeds.device, dtype=inputs_embeds.dtype)
        hidden_states = inputs_embeds
        all_hidden_states = () if output_hidden_states else None
        for mixer_block in self.layers:
            hidden_states = mixer_block(hidden_states, cache_params=cache_params if use_cache else None,
                                        cache_position=cache_position, attention_mask=attention_mask)
            if output_hidden_states:
                all_hidden_states = all_hidden_states + (hidden_states,)
        if use_cache:
            cache_params.seqlen_offset += inputs_embeds.shape[1]
        hidden_states = self.norm_f(hidden_states)
        if output_hidden_states:
            all_hidden_states = all_hidden_states + (hidden_states,)
        if not return_dict:
            return tuple(v for v in [hidden_states, cache_params if use_cache else None, all_hidden_states] if v is not None)
        return Mamba2Output(last_hidden_state=hidden_states, cache_params=cache_params if use_cache else None,
                            hidden_states=all_hidden_states)

    def step(self, input_ids, cache_params: Optional[Mamba2Cache] = None):
        """input_ids: int64 (batch, 1), one token per sequence -> hidden states (batch, 1, hidden) after the final norm.
        The caller advances ``cache_params.seqlen_offset`` (a host integer, so that a captured step stays replayable)."""
        x = self.embeddings(input_ids)
        act = self.layers[0].mixer.in_proj.weight.dtype if len(self.layers) else x.dtype
        if not (self.config.residual_in_fp32 and not torch.is_grad_enabled() and x.is_cuda and glue.add_rmsnorm_ok(x.shape[-1], act)):
            for mixer_block in self.layers:
                x = mixer_block.step(x, cache_params=cache_params)
            return self.norm_f(x)
        # fp32 residual stream: each block's residual add and the next norm are one kernel (the same arithmetic as
        # Mamba2Block.step followed by Mamba2RMSNorm: fp32 sum, fp32 norm, one rounding to the activation dtype)
        residual, delta = x.float().contiguous(), None
        for mixer_block in self.layers:
            normed = glue.add_rmsnorm_(residual, delta, mixer_block.norm.weight, mixer_block.norm.variance_epsilon, act)
            delta = mixer_block.mixer.step(normed, cache_params=cache_params)
        return glue.add_rmsnorm_(residual, delta, self.norm_f.weight, self.norm_f.variance_epsilon, act)


class Mamba2ForCausalLM(Mamba2PreTrainedModel):
    _tied_weights_keys = []

    def __init__(self, config):
        super().__init__(config)
        self.backbone = Mamba2Model(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.apply(self._init_weights)
        # the head starts from the same normal law as the table (modeling_mamba2.py:366-377: init_method on the parallel linear)
        nn.init.normal_(self.lm_head.weight, std=config.initializer_range)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.backbone.embeddings.weight

    def get_output_embeddings(self):
        return self.lm_head

    def set_output_embeddings(self, new_embeddings):
        self.lm_head = new_embeddings

    def get_input_embeddings(self):
        return self.backbone.get_input_embeddings()

    def set_input_embeddings(self, new_embeddings):
        return self.backbone.set_input_embeddings(new_embeddings)

    def forward(self, input_ids: Optional[torch.LongTensor] = None, inputs_embeds: Optional[torch.FloatTensor] = None,
                cache_params: Optional[Mamba2Cache] = None, labels: Optional[torch.LongTensor] = None,
                output_hidden_states: Optional[bool] = None, return_dict: Optional[bool] = None, use_cache: Optional[bool] = None,
                cache_position: Optional[torch.Tensor] = None, attention_mask: Optional[torch.Tensor] = None, **kwargs):
        return_dict = True if return_dict is None else return_dict
        out = self.backbone(input_ids, inputs_embeds=inputs_embeds, cache_params=cache_params, use_cache=use_cache,
                            output_hidden_states=output_hidden_states, return_dict=True, cache_position=cache_position,
                            attention_mask=attention_mask)
        logits = self.lm_head(out.last_hidden_state.to(self.lm_head.weight.dtype)).float()
        loss = None
        if labels is not None:
            # next-token loss: position t predicts token t+1  (modeling_mamba2.py:498-507)
            shift_logits = logits[..., :-1, :].contiguous()
            shift_labels = labels[..., 1:].contiguous().to(logits.device)
            loss = F.cross_entropy(shift_logits.view(-1, shift_logits.size(-1)), shift_labels.view(-1))
        if not return_dict:
            output = (logits,) + tuple(v for v in (out.cache_params, out.hidden_states) if v is not None)
            return ((loss,) + output) if loss is not None else output
        return Mamba2CausalLMOutput(loss=loss, logits=logits, cache_params=out.cache_params, hidden_states=out.hidden_states)

    def step(self, idx, cache_params: Optional[Mamba2Cache] = None):
        """idx: int64 (batch, 1) -> logits (batch, 1, vocab) fp32; the layers' states in ``cache_params`` advance by one token."""
        hidden_states = self.backbone.step(idx, cache_params=cache_params)
        return self.lm_head(hidden_states.to(self.lm_head.weight.dtype)).float()


@torch.no_grad()
def greedy_generate(model: "Mamba2ForCausalLM", input_ids, max_new_tokens: int, use_graph: bool = True, conv_width: Optional[int] = None):
    """Greedy continuation of ``input_ids`` (batch, prompt_len) by ``max_new_tokens`` tokens: the prompt goes through the
    sequence kernels once and leaves its states in a fresh cache (prefill), then every new token is one ``step`` --
    replayed from one HIP graph when ``use_graph``.  The loop of ``mamba2_inference_no_tp.py:108-127`` with the prompt
    prefilled instead of stepped through.  Returns (batch, prompt_len + max_new_tokens) token ids."""
    b = input_ids.shape[0]
    dtype = model.backbone.layers[0].mixer.in_proj.weight.dtype
    cache = Mamba2Cache(model.config, b, dtype=dtype, device=input_ids.device, conv_width=conv_width)
    logits = model(input_ids=input_ids, cache_params=cache, use_cache=True).logits[:, -1:]
    step = GraphedStep(model, cache, b) if (use_graph and max_new_tokens > 1) else (lambda idx: model.step(idx, cache))
    out = [input_ids]
    for t in range(max_new_tokens):
        nxt = logits.argmax(dim=-1)
        out.append(nxt)
        if t + 1 < max_new_tokens:
            logits = step(nxt)
            cache.seqlen_offset += 1
    return torch.cat(out, dim=1)


class _TunedGemms:
    """torch.cuda.tunable switched on for a stretch of code and put back afterwards.  Results go to a file in the
    temporary directory unless the caller has chosen one (TunableOp writes its table when the process ends)."""

    def __init__(self):
        import os
        import tempfile
        import torch.cuda.tunable as tunable
        self.t = tunable
        self.was_enabled, self.was_tuning = tunable.is_enabled(), tunable.tuning_is_enabled()
        if not self.was_enabled and not os.environ.get("PYTORCH_TUNABLEOP_FILENAME"):
            tunable.set_filename(os.path.join(tempfile.gettempdir(), f"mamba2_tunableop_{os.getpid()}.csv"))

    def start_tuning(self):
        self.t.enable(True)
        self.t.tuning_enable(True)

    def stop_tuning(self):
        self.t.tuning_enable(False)

    def restore(self):
        self.t.tuning_enable(self.was_tuning)
        self.t.enable(self.was_enabled)


class GraphedStep:
    """``Mamba2ForCausalLM.step`` for one batch size, captured once into a HIP graph and replayed per token.

    The graph reads the token ids from ``self.input_ids`` and the states from ``cache_params`` (updated in place by the
    decode kernel, so each replay continues from the last) and leaves the logits in ``self.logits``; ``__call__`` copies
    the ids in, replays and returns ``self.logits`` (overwritten by the next call).  The model's parameters and the cache
    tensors must stay where they are, and the parameters unchanged, while the object lives (the graph holds their
    addresses, and for a model kept in bfloat16 the fp32 copies of the small per-head and norm parameters made before the
    capture): build a new object after loading other weights.  ``cache_params`` may be reset or refilled by a prefill
    between replays.  The states advanced by the warm-up and capture runs are restored before ``__init__`` returns.

    ``tune_gemms=True`` lets torch's TunableOp time the BLAS libraries' solutions for the step's projection shapes (in_proj,
    out_proj, LM head: 128-row products for which the libraries' default choices are 15-25 % off their best) during the
    warm-up and captures the chosen ones; the process-wide TunableOp switches are put back afterwards, the graph keeps the
    kernels it captured.  The chosen solutions may round differently from the default ones, so replays then agree with the
    eager step to bf16 accuracy, not bit for bit.
    """

    def __init__(self, model: Mamba2ForCausalLM, cache_params: Mamba2Cache, batch_size: int, warmup: int = 2,
                 tune_gemms: bool = False):
        dev = model.device
        if dev.type != "cuda":
            raise RuntimeError("GraphedStep needs the model on a GPU device; there is no CPU path")
        self.model, self.cache = model, cache_params
        self.input_ids = torch.zeros(batch_size, 1, dtype=torch.long, device=dev)
        keep = [t.clone() for t in cache_params.conv_states + cache_params.ssm_states]
        tun = _TunedGemms() if tune_gemms else None
        try:
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.no_grad(), torch.cuda.stream(side):
                if tun:
                    tun.start_tuning()          # the first warm-up step times the libraries' solutions for its three GEMM shapes
                for _ in range(warmup):         # lazily created workspaces and library handles exist before the capture
                    model.step(self.input_ids, cache_params)
                if tun:
                    tun.stop_tuning()           # (no timing runs inside the capture: the chosen solutions are looked up)
            torch.cuda.current_stream(dev).wait_stream(side)
            torch.cuda.synchronize(dev)
            self.graph = torch.cuda.CUDAGraph()
            with torch.no_grad(), torch.cuda.graph(self.graph):
                self.logits = model.step(self.input_ids, cache_params)
        finally:
            if tun:
                tun.restore()
        for t, k in zip(cache_params.conv_states + cache_params.ssm_states, keep):
            t.copy_(k)

    def __call__(self, idx):
        self.input_ids.copy_(idx)
        self.graph.replay()
        return self.logits
