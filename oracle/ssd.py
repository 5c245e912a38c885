"""SSD (state-space duality) scan oracle.  TEST INFRASTRUCTURE ONLY.

Shapes (reference ``mamba2/mamba2_kernel.py:287-296``):
    dt (b, l, h)  -- already softplus'd, positive
    A  (h)        -- negative
    X  (b, l, h, p)
    B, C (b, l, g, n),  h % g == 0, head ``i`` uses group ``i // (h // g)``
    D  (h) or None
    state (b, h, p, n)   -- decode layout, ``mamba2_kernel_inference.py:39``

Pins (tests/test_oracle_ssd.py):
* ``ssd_recurrent_ref`` IS the definition: S_t = exp(A dt_t) S_{t-1} + dt_t x_t (x) B_t,
  y_t = S_t C_t + D x_t  (``mamba2_kernel_inference.py:81,95-102``).  It is checked
  against a scalar pure-Python triple loop on tiny inputs, against the causal
  linear-attention closed form when A -> 0, dt = 1, D = 0, and against HF
  transformers' torch ``mamba2_chunk_scan`` golden vectors.
* ``ssd_chunked_ref`` must equal the recurrence for every chunk size.
* gradients: autograd through either function; ``gradcheck`` in fp64.
"""
import torch


def _expand_groups(t, h):
    """(b, l, g, n) -> (b, l, h, n): head i reads group i // (h // g)
    (``mamba2_kernel.py:131-133``: head_id = group_id * n_heads_per_group + head_id_in_group)."""
    g = t.shape[2]
    if g == h:
        return t
    return t.repeat_interleave(h // g, dim=2)


def ssd_recurrent_ref(dt, A, X, B, C, D=None, initial_state=None):
    """Token-by-token recurrence.  Returns (y (b,l,h,p), final_state (b,h,p,n)).

    Follows ``mamba2_kernel_inference.py:81`` (dA = exp(A*dt)), ``:95-97``
    (S' = S*dA + (dt*x) (x) B) and ``:101-102`` (y = S'.C + D*x).
    Computation dtype = dtype of ``X`` (use fp64 inputs for ground truth).
    """
    b, l, h, p = X.shape
    n = B.shape[-1]
    Bh = _expand_groups(B, h)
    Ch = _expand_groups(C, h)
    S = X.new_zeros(b, h, p, n) if initial_state is None else initial_state.to(X.dtype)
    ys = []
    for t in range(l):
        dA = torch.exp(A * dt[:, t])                                  # (b, h)
        xd = X[:, t] * dt[:, t, :, None]                              # (b, h, p)
        S = S * dA[:, :, None, None] + xd[..., None] * Bh[:, t, :, None, :]
        y = torch.einsum("bhpn,bhn->bhp", S, Ch[:, t])
        if D is not None:
            y = y + D[None, :, None] * X[:, t]
        ys.append(y)
    y = torch.stack(ys, dim=1) if l > 0 else X.new_zeros(b, 0, h, p)
    return y, S


def ssd_chunked_ref(dt, A, X, B, C, D=None, initial_state=None, chunk=128):
    """Chunked (matmul) form.  Returns (y, final_state).

    One pass over chunks carrying the running state, as the reference's device
    loop does (``mamba2_kernel.py:137-169``):
      l = cumsum(A*dt) inside the chunk                     (``:26-28``)
      L[i,j] = exp(l_i - l_j) for i >= j, else 0            (``:32-34``)
      Y = (L o (C B^T)) (dt o X) + (C o e^l) S              (``:54-62``)
      S <- e^{l_last} S + (B o e^{l_last - l})^T (dt o X)   (``:160-163``)
      Y += D X                                              (``:167``)
    A ragged last chunk (l % chunk != 0) is handled by slicing.
    """
    b, l, h, p = X.shape
    n = B.shape[-1]
    Bh = _expand_groups(B, h)
    Ch = _expand_groups(C, h)
    S = X.new_zeros(b, h, p, n) if initial_state is None else initial_state.to(X.dtype)
    outs = []
    for s0 in range(0, l, chunk):
        s1 = min(l, s0 + chunk)
        q = s1 - s0
        dtc = dt[:, s0:s1]                                            # (b, q, h)
        a = A * dtc
        lc = torch.cumsum(a, dim=1)                                   # (b, q, h)
        diff = lc[:, :, None, :] - lc[:, None, :, :]                  # (b, i, j, h)
        mask = torch.ones(q, q, dtype=torch.bool, device=X.device).tril()
        Lm = torch.where(mask[None, :, :, None], torch.exp(torch.where(mask[None, :, :, None], diff, torch.zeros_like(diff))),
                         torch.zeros_like(diff))
        xd = X[:, s0:s1] * dtc[..., None]                             # (b, q, h, p)
        G = torch.einsum("bihn,bjhn->bijh", Ch[:, s0:s1], Bh[:, s0:s1])
        y = torch.einsum("bijh,bjhp->bihp", Lm * G, xd)
        y = y + torch.einsum("bihn,bhpn->bihp", Ch[:, s0:s1] * torch.exp(lc)[..., None], S)
        last = lc[:, -1]                                              # (b, h)
        Bd = Bh[:, s0:s1] * torch.exp(last[:, None] - lc)[..., None]
        S = S * torch.exp(last)[:, :, None, None] + torch.einsum("bjhn,bjhp->bhpn", Bd, xd)
        if D is not None:
            y = y + D[None, None, :, None] * X[:, s0:s1]
        outs.append(y)
    y = torch.cat(outs, dim=1) if outs else X.new_zeros(b, 0, h, p)
    return y, S


def ssd_grads_ref(dt, A, X, B, C, D, dy, initial_state=None, d_final_state=None, chunk=128, fn=None):
    """All SSD gradients by autograd through the oracle (default: chunked form).

    Returns dict with y, final_state, ddt, dA, dX, dB, dC, dD (and dinitial_state
    when an initial state is given).  Shapes follow the reference's backward
    (``mamba2_kernel.py:498-515``): dA and dD are summed over the batch.
    """
    fn = fn or (lambda *a, **k: ssd_chunked_ref(*a, chunk=chunk, **k))
    leaves = [t.detach().clone().requires_grad_(True) for t in (dt, A, X, B, C)]
    Dl = D.detach().clone().requires_grad_(True) if D is not None else None
    S0 = initial_state.detach().clone().requires_grad_(True) if initial_state is not None else None
    y, S = fn(*leaves, Dl, initial_state=S0)
    loss = (y * dy).sum()
    if d_final_state is not None:
        loss = loss + (S * d_final_state).sum()
    wrt = leaves + ([Dl] if Dl is not None else []) + ([S0] if S0 is not None else [])
    grads = list(torch.autograd.grad(loss, wrt, allow_unused=True))
    out = {"y": y.detach(), "final_state": S.detach()}
    for name in ("ddt", "dA", "dX", "dB", "dC"):
        out[name] = grads.pop(0)
    if Dl is not None:
        out["dD"] = grads.pop(0)
    if S0 is not None:
        out["dinitial_state"] = grads.pop(0)
    return out


def make_ssd_inputs(b, l, h, p, n, g, seed=0, dtype=torch.float32, device="cpu"):
    """Seeded synthetic inputs with the distributions the reference's parity
    script uses (``mamba2_kernel.py:555-564``) adjusted as the benchmark
    configuration states: dt = exp(U(log 1e-3, log 1e-1)), A = -exp(U(log 1, log 16)),
    x ~ N(0,1), B, C ~ N(0,1)/sqrt(n), D = 1, dy ~ N(0,1).
    Values are drawn in fp32 on the CPU, rounded to ``dtype`` and returned as
    ``dtype`` tensors (so an fp64 oracle run sees exactly the rounded values).
    """
    import math
    gen = torch.Generator(device="cpu").manual_seed(seed)
    dt = torch.exp(torch.empty(b, l, h).uniform_(math.log(1e-3), math.log(1e-1), generator=gen))
    A = -torch.exp(torch.empty(h).uniform_(0.0, math.log(16.0), generator=gen))
    X = torch.randn(b, l, h, p, generator=gen)
    B = torch.randn(b, l, g, n, generator=gen) / math.sqrt(n)
    C = torch.randn(b, l, g, n, generator=gen) / math.sqrt(n)
    D = torch.ones(h)
    dy = torch.randn(b, l, h, p, generator=gen)
    cast = lambda t: t.to(dtype).to(device)
    return {"dt": cast(dt), "A": A.to(device), "X": cast(X), "B": cast(B), "C": cast(C),
            "D": D.to(device), "dy": cast(dy)}
