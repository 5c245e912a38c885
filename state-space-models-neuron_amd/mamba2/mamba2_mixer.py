"""``Mamba2Mixer`` with the reference's module interface (``mamba2/mamba2_mixer.py:108-282``) on one MI355X.

Parameter names and shapes are the reference's (and HF / state-spaces'): ``in_proj``, ``conv1d.weight (C,1,k)``,
``conv1d.bias``, ``dt_bias``, ``A_log``, ``D``, ``norm.weight``, ``out_proj``.  The tensor-parallel linears of the
reference become ``nn.Linear`` (tp = 1) and its XLA-device assert is dropped.  ``forward`` = in_proj ->
``mamba2_fused_kernel`` -> out_proj; ``step`` = in_proj -> ``mamba2_kernel_inference`` on the [xBC | dt] columns
(softplus applied inside) -> gated norm -> out_proj: two projections and three kernels of this library per token.

``forward`` with ``cache_params`` (inference only) is the prefill that hands over to ``step``: it leaves the layer's
SSM and conv state in the cache, and continues from them when ``cache_params.seqlen_offset > 0``.  The reference
asserts the cache away there (``mamba2_mixer.py:220``); the cache fields are the ones its ``step`` uses (``:270-276``).
"""
import math
from typing import Optional

import torch
from torch import nn

from .configuration_mamba2 import Mamba2Config
from .conv1d_grouped import ConvNKI
from .fused_kernel import mamba2_fused_kernel, mamba2_fused_kernel_with_caching, mamba2_fused_prefill
from .mamba2_kernel_inference import mamba2_kernel_inference
from . import glue


def softplus(x, threshold=10):
    return torch.where(x < threshold, torch.log1p(torch.exp(torch.clamp(x, max=threshold))), x)


class Mamba2Cache:
    """Minimal decode cache: per-layer ``conv_states[i]`` (b, conv_dim, W) and ``ssm_states[i]`` (b, h, p, n) fp32,
    plus ``seqlen_offset`` (the fields the reference touches, ``mamba2_mixer.py:270-276``, ``modeling_mamba2.py:321``)."""

    def __init__(self, config: Mamba2Config, batch_size: int, dtype=torch.float32, device=None, conv_width: Optional[int] = None):
        d_inner = int(config.expand * config.hidden_size)
        conv_dim = d_inner + 2 * config.n_groups * config.state_size
        W = config.conv_kernel if conv_width is None else conv_width
        self.seqlen_offset = 0
        self.dtype = dtype
        self.conv_states = [torch.zeros(batch_size, conv_dim, W, dtype=dtype, device=device) for _ in range(config.num_hidden_layers)]
        self.ssm_states = [torch.zeros(batch_size, config.num_heads, config.head_dim, config.state_size, dtype=torch.float32, device=device)
                           for _ in range(config.num_hidden_layers)]

    def reset(self):
        for t in self.conv_states + self.ssm_states:
            t.zero_()
        self.seqlen_offset = 0


class MambaRMSNormGated(nn.Module):
    """Gated RMSNorm that normalises independently inside each of ``n_groups`` channel groups
    (``mamba2_mixer.py:41-105``); fp32 output."""

    def __init__(self, d: int, eps: float = 1e-5, device=None, n_groups: int = 1, rmsnorm_within_groups=True,
                 name=None, hidden_size=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(d, device=device))
        self.n_groups = n_groups
        self.rmsnorm_within_groups = rmsnorm_within_groups
        self.name = name
        self.hidden_size = hidden_size

    def forward(self, hidden_states, gate=None, out_dtype=None):
        g = self.n_groups if self.rmsnorm_within_groups else 1
        return glue.rmsnorm_gated_fn(hidden_states, gate, self.weight, g, self.eps, out_dtype=out_dtype)


class Mamba2Mixer(nn.Module):
    def __init__(self, config: Mamba2Config, layer_idx: int):
        super().__init__()
        self.num_heads = config.num_heads
        self.hidden_size = config.hidden_size
        self.ssm_state_size = config.state_size
        self.conv_kernel_size = config.conv_kernel
        self.intermediate_size = int(config.expand * self.hidden_size)
        self.time_step_rank = int(config.time_step_rank)
        self.layer_idx = layer_idx
        self.use_conv_bias = config.use_conv_bias
        self.activation = config.hidden_act
        self.layer_norm_epsilon = config.layer_norm_epsilon
        self.rms_norm = config.rms_norm
        self.rmsnorm_within_groups = config.rmsnorm_within_groups
        self.n_groups = config.n_groups
        self.head_dim = config.head_dim
        self.chunk_size = config.chunk_size
        self.time_step_limit = config.time_step_limit
        self.time_step_min = config.time_step_min
        self.time_step_max = config.time_step_max

        assert self.intermediate_size % self.head_dim == 0
        assert self.intermediate_size // self.head_dim == self.num_heads

        self.conv_dim = self.intermediate_size + 2 * self.n_groups * self.ssm_state_size
        self.conv1d = ConvNKI(
            in_channels=self.conv_dim,
            out_channels=self.conv_dim,
            bias=config.use_conv_bias,
            kernel_size=config.conv_kernel,
            groups=self.conv_dim,
            padding=config.conv_kernel - 1,
        )
        self.in_proj = nn.Linear(self.hidden_size, self.intermediate_size + self.conv_dim + self.num_heads, bias=config.use_bias)

        # dt_bias = softplus^{-1}(dt), dt log-uniform in [time_step_min, time_step_max]  (mamba2_mixer.py:160-168)
        dt = torch.exp(
            torch.rand(config.num_heads) * (math.log(config.time_step_max) - math.log(config.time_step_min))
            + math.log(config.time_step_min)
        ).clamp(min=config.time_step_floor)
        inv_dt = dt + torch.log(-torch.expm1(-dt))
        self.dt_bias = nn.Parameter(inv_dt)
        self.dt_bias._no_reinit = True

        A = torch.arange(1, self.num_heads + 1)
        self.A_log = nn.Parameter(torch.log(A))
        self.A_log._no_weight_decay = True
        self.norm = MambaRMSNormGated(self.intermediate_size, eps=self.layer_norm_epsilon, n_groups=self.n_groups,
                                      rmsnorm_within_groups=self.rmsnorm_within_groups,
                                      name=f"backbone.layers.{layer_idx}.mixer.norm", hidden_size=config.hidden_size)
        self.D = nn.Parameter(torch.ones(self.num_heads))
        self.D._no_weight_decay = True
        self.out_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=config.use_bias)
        self.use_bias = config.use_bias
        # tp = 1: the per-rank sizes of the reference equal the full sizes
        self.intermediate_size_tp = self.intermediate_size
        self.n_groups_tp = self.n_groups
        self.num_heads_tp = self.num_heads
        self.conv_dim_tp = self.conv_dim
        self._fp32_params = None
        self.recompute_core = bool(getattr(config, "recompute_core", False))

    def _inference_params(self):
        """fp32 (A, D, dt_bias) as the decode kernel takes them, rebuilt only when a parameter changed."""
        ps = (self.A_log, self.D, self.dt_bias)
        key = tuple((p.data_ptr(), p._version, p.dtype) for p in ps)
        if self._fp32_params is None or self._fp32_params[0] != key:
            with torch.no_grad():
                self._fp32_params = (key, -torch.exp(self.A_log.float()), self.D.float(), self.dt_bias.float())
        return self._fp32_params[1:]

    def nki_kernels_forward(self, hidden_states, cache_params: Optional[Mamba2Cache] = None,
                            cache_position: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None):
        assert attention_mask is None, "attention mask not supported yet"
        assert self.time_step_limit[0] == 0.0 and self.time_step_limit[1] == float("inf"), "dt limit not supported yet"
        assert self.activation in ["silu", "swish"]
        assert self.rmsnorm_within_groups, "the fused core always normalises within groups (fused_kernel.py:255)"

        if cache_params is not None:
            assert not torch.is_grad_enabled(), "forward with a cache is the inference prefill: call it under torch.no_grad()"
            A, D, dt_bias = self._inference_params()
            zxBCdt = self.in_proj(hidden_states)
            scan_output = mamba2_fused_prefill(zxBCdt, A, D, self.conv1d.weight, self.conv1d.bias, dt_bias, self.norm.weight,
                                               self.n_groups_tp, self.ssm_state_size, self.intermediate_size_tp, self.head_dim,
                                               cache_params.conv_states[self.layer_idx], cache_params.ssm_states[self.layer_idx],
                                               continuing=cache_params.seqlen_offset > 0)
            return self.out_proj(scan_output)
        A = -torch.exp(self.A_log.float())
        zxBCdt = self.in_proj(hidden_states)
        core = mamba2_fused_kernel if self.recompute_core else mamba2_fused_kernel_with_caching
        scan_output = core(zxBCdt, A, self.D, self.conv1d.weight, self.conv1d.bias, self.dt_bias, self.norm.weight,
                           self.n_groups_tp, self.ssm_state_size, self.intermediate_size_tp, self.head_dim)
        return self.out_proj(scan_output)

    def forward(self, hidden_states, cache_params: Optional[Mamba2Cache] = None,
                cache_position: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None):
        return self.nki_kernels_forward(hidden_states, cache_params, cache_position, attention_mask)

    def step(self, hidden_states, cache_params: Optional[Mamba2Cache] = None):
        """hidden_states: (B, 1, D) -> same shape; updates the layer's conv and SSM state."""
        batch, seqlen, dim = hidden_states.shape
        assert seqlen == 1
        zxBCdt = self.in_proj(hidden_states)
        n_groups, d_state, d_inner, d_head = self.n_groups_tp, self.ssm_state_size, self.intermediate_size_tp, self.head_dim
        n_heads = d_inner // d_head
        d_conv = d_inner + 2 * n_groups * d_state
        assert zxBCdt.shape[-1] == d_inner + d_conv + n_heads
        # the kernels read the [z | xBC | dt] columns where the projection left them; softplus(dt + dt_bias) happens inside
        z, xBC, dt = torch.split(zxBCdt, [d_inner, d_conv, n_heads], dim=-1)
        A, D, dt_bias = self._inference_params()
        y, new_conv_state, new_ssm_state = mamba2_kernel_inference(
            xBC, cache_params.conv_states[self.layer_idx], self.conv1d.weight.squeeze(1), self.conv1d.bias,
            cache_params.ssm_states[self.layer_idx], dt, A, D, n_groups=self.n_groups_tp, dt_bias=dt_bias)
        cache_params.conv_states[self.layer_idx] = new_conv_state
        cache_params.ssm_states[self.layer_idx] = new_ssm_state
        y = self.norm(y.view(batch, seqlen, -1), z, out_dtype=hidden_states.dtype)
        return self.out_proj(y)
