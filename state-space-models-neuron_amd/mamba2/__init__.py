"""MI355X-native Mamba-2 mixer hot path behind the reference's operator API.

Module and symbol names follow awslabs/state-space-models-neuron's ``mamba2`` package:
``mamba2_kernel`` (SSD scan), ``conv1d_grouped`` (depthwise conv1d + SiLU),
``mamba2_kernel_inference`` (decode step), ``fused_kernel`` (mixer core) and
``mamba2_mixer`` (the nn.Module).  All device work goes through libmamba2_hip.so.
"""
