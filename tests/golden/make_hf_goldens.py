"""Write small golden vectors from HuggingFace transformers' pure-torch Mamba-2 functions.

The reference's fused-layer parity script compares its kernels with
``transformers.models.mamba2.modeling_mamba2`` (``mamba2/fused_kernel.py:547-555``);
the reference itself stores no golden vectors and its own torch SSD oracle file is
absent from its tree (``mamba2/mamba2_kernel.py:573``).  This script evaluates the
torch bodies of HF's ``mamba2_chunk_scan``, ``mamba2_selective_state_update``,
``causal_conv1d_fn`` and ``MambaRMSNormGated`` on seeded fp64/fp32 inputs and stores
inputs + outputs in ``hf_goldens.npz`` next to this file.  Tests only read the .npz;
transformers is not needed to run them.

Run (only needed to regenerate):  python tests/golden/make_hf_goldens.py
"""
import math
import os

import numpy as np
import torch


def main():
    from transformers.models.mamba2 import modeling_mamba2 as hf

    out = {}
    gen = torch.Generator().manual_seed(1234)

    # --- SSD chunk scan, two group settings, ragged length on the second -----------------
    for tag, (b, l, h, p, n, g, chunk) in {"scan_g1": (2, 256, 4, 16, 16, 1, 64),
                                            "scan_g2": (2, 200, 4, 16, 16, 2, 64)}.items():
        dt = torch.exp(torch.empty(b, l, h, dtype=torch.float64).uniform_(math.log(1e-3), math.log(1e-1), generator=gen))
        A = -torch.exp(torch.empty(h, dtype=torch.float64).uniform_(0.0, math.log(16.0), generator=gen))
        X = torch.randn(b, l, h, p, dtype=torch.float64, generator=gen)
        B = torch.randn(b, l, g, n, dtype=torch.float64, generator=gen) / math.sqrt(n)
        C = torch.randn(b, l, g, n, dtype=torch.float64, generator=gen) / math.sqrt(n)
        D = torch.randn(h, dtype=torch.float64, generator=gen)
        S0 = 0.1 * torch.randn(b, h, p, n, dtype=torch.float64, generator=gen)
        # HF's body casts to fp32 internally (.float()), so goldens carry fp32 accuracy.
        y, S = hf.mamba2_chunk_scan(X, dt, A, B, C, chunk, D=D, initial_states=S0, return_final_states=True)
        y0, S_0 = hf.mamba2_chunk_scan(X, dt, A, B, C, chunk, D=D, return_final_states=True)
        for k_, v in dict(dt=dt, A=A, X=X, B=B, C=C, D=D, S0=S0, y=y, S=S, y_noinit=y0, S_noinit=S_0).items():
            out[f"{tag}.{k_}"] = v.numpy()

    # --- single-token selective state update ------------------------------------------------
    b, h, p, n, g = 3, 4, 8, 16, 2
    state = 0.1 * torch.randn(b, h, p, n, generator=gen)
    x = torch.randn(b, h, p, generator=gen)
    dt = torch.exp(torch.empty(b, h).uniform_(math.log(1e-3), math.log(1e-1), generator=gen))
    A = -torch.exp(torch.empty(h).uniform_(0.0, math.log(16.0), generator=gen))
    Bv = torch.randn(b, g, n, generator=gen)
    Cv = torch.randn(b, g, n, generator=gen)
    D = torch.randn(h, generator=gen)
    st = state.clone()
    # HF takes dt/A/D broadcast to (b, h, p[, n]) in its call site; the torch body accepts (b,h)+(h) shapes
    y = hf.mamba2_selective_state_update(st, x, dt[..., None].expand(b, h, p), A[:, None, None].expand(h, p, n),
                                         Bv, Cv, D=D[:, None].expand(h, p))
    for k_, v in dict(state=state, x=x, dt=dt, A=A, B=Bv, C=Cv, D=D, y=y, new_state=st).items():
        out[f"ssu.{k_}"] = v.numpy()

    # --- causal conv1d + silu, layout (b, C, l) ------------------------------------------------
    b, Cc, l, k = 2, 24, 37, 4
    x = torch.randn(b, Cc, l, dtype=torch.float64, generator=gen)
    w = torch.rand(Cc, k, dtype=torch.float64, generator=gen) - 0.5
    bias = torch.rand(Cc, dtype=torch.float64, generator=gen) - 0.5
    y = hf.causal_conv1d_fn(x, w, bias, activation="silu")
    for k_, v in dict(x=x, w=w, bias=bias, y=y).items():
        out[f"conv.{k_}"] = v.numpy()

    # --- gated RMSNorm (HF normalises across the whole hidden size => n_groups = 1) -------------
    d = 48
    norm = hf.MambaRMSNormGated(d, eps=1e-5)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(d, generator=gen))
    x = torch.randn(2, 5, d, generator=gen)
    z = torch.randn(2, 5, d, generator=gen)
    y = norm(x, z)
    for k_, v in dict(x=x, z=z, w=norm.weight.detach(), y=y.detach()).items():
        out[f"norm.{k_}"] = v.numpy()

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hf_goldens.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
