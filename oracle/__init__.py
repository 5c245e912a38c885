"""CPU oracle for the Mamba-2 mixer hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this directory.  It is imported by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` -- always as the checker, never as the thing measured or shipped.

The oracle is a pure-PyTorch restatement (CPU, fp32 or fp64) of the maths of
the reference's device kernels:

* ``oracle.ssd``     -- SSD scan: token recurrence (ground truth) and the
  chunked form that follows ``mamba2/mamba2_kernel.py:15-62,137-169``.
* ``oracle.conv``    -- causal depthwise conv1d (+SiLU), following
  ``mamba2/conv1d_grouped.py:69-81``.
* ``oracle.decode``  -- one-token recurrent step, following
  ``mamba2/mamba2_kernel_inference.py:13-23,80-104``.
* ``oracle.mixer``   -- softplus, gated grouped RMSNorm and the fused mixer
  core pipeline, following ``mamba2/fused_kernel.py:33-47,76-103,252-282`` and
  ``mamba2/mamba2_mixer.py:36-38,88-105``.

How each function is pinned (which independent check would fail on a dropped
term, wrong sign, or transposed operand) is stated in its docstring and
exercised by ``tests/test_oracle_*.py``.  The reference's own torch oracle
(``mamba2_kernel_reference.ssd_minimal_discrete_fused``, imported at
``mamba2/mamba2_kernel.py:573``) is absent from the reference tree, and the
reference stores no golden vectors, so the pins are: the closed-form token
recurrence in fp64, brute-force loops on tiny inputs, special cases that
reduce to textbook routines (causal linear attention, ``F.conv1d``),
``torch.autograd.gradcheck``, and golden vectors written from the pure-torch
Mamba-2 functions of HuggingFace transformers (the library the reference's
fused parity script compares against, ``mamba2/fused_kernel.py:547-555``).
"""
