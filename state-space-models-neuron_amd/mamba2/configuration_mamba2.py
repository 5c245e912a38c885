"""Configuration object holding the fields ``Mamba2Mixer`` reads (``mamba2/configuration_mamba2.py:114-189``;
defaults as there: 128 heads, head_dim 64, state 128, 8 groups, conv kernel 4, chunk 256, eps 1e-5)."""
import math


class Mamba2Config:
    model_type = "mamba2"

    def __init__(self, num_heads=128, head_dim=64, vocab_size=32768, hidden_size=4096, state_size=128, num_hidden_layers=64,
                 layer_norm_epsilon=1e-5, expand=2, conv_kernel=4, n_groups=8, use_bias=False, use_conv_bias=True,
                 hidden_act="silu", initializer_range=0.1, residual_in_fp32=True, time_step_rank="auto",
                 time_step_min=0.001, time_step_max=0.1, time_step_floor=1e-4, time_step_limit=(0.0, float("inf")),
                 rescale_prenorm_residual=False, use_cache=True, rms_norm=True, rmsnorm_within_groups=True, chunk_size=256,
                 tie_word_embeddings=False, sequence_parallel_enabled=False, dtype=None, recompute_core=False, **kwargs):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.state_size = state_size
        self.num_hidden_layers = num_hidden_layers
        self.layer_norm_epsilon = layer_norm_epsilon
        self.conv_kernel = conv_kernel
        self.expand = expand
        self.use_bias = use_bias
        self.use_conv_bias = use_conv_bias
        self.hidden_act = hidden_act
        self.initializer_range = initializer_range
        self.time_step_rank = math.ceil(hidden_size / 16) if time_step_rank == "auto" else time_step_rank
        self.time_step_min = time_step_min
        self.time_step_max = time_step_max
        self.time_step_floor = time_step_floor
        self.rescale_prenorm_residual = rescale_prenorm_residual
        self.residual_in_fp32 = residual_in_fp32
        self.use_cache = use_cache
        self.n_groups = n_groups
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.rms_norm = rms_norm
        self.rmsnorm_within_groups = rmsnorm_within_groups
        self.chunk_size = chunk_size
        self.time_step_limit = tuple(time_step_limit)
        self.tie_word_embeddings = tie_word_embeddings
        # False: the fused core keeps its conv output, scan output and chunk states for the backward (288 GB of HBM make that
        # cheaper than a second forward); True: only the inputs are kept and the backward recomputes, as the reference's
        # mixer does (mamba2_mixer.py:229)
        self.recompute_core = recompute_core
        self.sequence_parallel_enabled = sequence_parallel_enabled
        self.dtype = dtype
        for k, v in kwargs.items():
            setattr(self, k, v)
