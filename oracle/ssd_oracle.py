"""CPU oracle for the Mamba-2 SSD chunk-scan forward and its single-timestep update.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke check and
the benchmark's CPU-baseline leg may import it; the shipped path is the HIP library and
never routes through here.

Provenance.  The reference tree (CarsonBurke/trading_bot_0) no longer contains an SSD
implementation: the only traces are four benchmark row names
(`benchmark_results/bench_20260112_070055.json:7,16,25,34`) and the slot the encoder
occupied (`trading_bots/src/torch/model/trading_model.rs:589-606`, streaming caller
`trading_bots/src/torch/model/stream/live.rs:228-244`).  There is therefore no reference
source, golden vector or test to restate, and no third-party dependency named in
`Cargo.toml`/`Cargo.lock` that holds the arithmetic.  What is restated here is the
published Mamba-2 SSD algorithm (Dao & Gu 2024, "Transformers are SSMs", section 6:
chunked state-space-dual form) under the conventions the task definition fixes:

  h_t = exp(dt_t * A_h) * h_{t-1} + dt_t * x_t (outer) B_t       state  [P, N]
  y_t = h_t . C_t + D_h * x_t                                    (y reads the UPDATED state)

  x  [B, L, H, P]   dt [B, L, H] (already positive; no softplus/bias/clamp in the op)
  A  [H] (< 0)      Bm, Cm [B, L, G, N], head h uses group h // (H // G)
  D  [H] or None    init [B, H, P, N] or None (zero)      final [B, H, P, N]

Pinning.  With no reference vectors, each function is pinned by what the mathematics
fixes (tests/test_oracle.py):
  ssd_sequential   textbook first-order IIR via scipy.signal.lfilter (P=N=1, constant
                   decay); closed-form geometric series for constant inputs; A -> 0-
                   reduces to numpy.cumsum; brute-force quadratic form ssd_quadratic
  chunk_cumsum     numpy.cumsum per chunk (library routine)
  chunk_state      per-tile numpy.einsum and the geometric closed form
  state_passing    scipy.signal.lfilter and final = exp(sum dt*A) * init when S = 0
  chunk_scan       O(Q^2) brute force; composition == ssd_sequential for every chunk size
  ssd_step         L applications == ssd_sequential
The C restatement (ssd_oracle.c) is checked against this file.

All functions compute in `dtype` (default float64) on whatever values they are handed;
for the bf16 mode the caller rounds the inputs to bf16 once and passes the rounded
values, so the oracle measures only the kernel's arithmetic error.
"""
from __future__ import annotations

import numpy as np


def _group_of_head(H: int, G: int) -> np.ndarray:
    if H % G != 0:
        raise ValueError(f"nheads {H} not divisible by ngroups {G}")
    return np.arange(H) // (H // G)


def ssd_sequential(x, dt, A, Bm, Cm, D=None, init=None, dtype=np.float64, reset=None):
    """Definitional recurrence, one timestep at a time.  Ground truth for everything.
    reset [B,L] (optional): a non-zero entry sets that batch row's state to zero before the timestep."""
    x = np.asarray(x, dtype)
    dt = np.asarray(dt, dtype)
    A = np.asarray(A, dtype)
    Bm = np.asarray(Bm, dtype)
    Cm = np.asarray(Cm, dtype)
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    gh = _group_of_head(H, G)
    h = np.zeros((Bsz, H, P, N), dtype) if init is None else np.array(init, dtype)
    y = np.empty((Bsz, L, H, P), dtype)
    for t in range(L):
        if reset is not None:
            h[np.asarray(reset)[:, t] != 0] = 0
        a = np.exp(dt[:, t, :] * A[None, :])                      # [B,H]
        Bt = Bm[:, t, gh, :]                                      # [B,H,N]
        Ct = Cm[:, t, gh, :]
        h = a[:, :, None, None] * h + (dt[:, t, :, None] * x[:, t])[..., None] * Bt[:, :, None, :]
        y[:, t] = np.einsum("bhpn,bhn->bhp", h, Ct)
        if D is not None:
            y[:, t] += np.asarray(D, dtype)[None, :, None] * x[:, t]
    return y, h


def ssd_step(state, x, dt, A, Bm, Cm, D=None, dtype=np.float64):
    """One recurrent update.  state [B,H,P,N] -> (y [B,H,P], new state)."""
    state = np.asarray(state, dtype)
    x = np.asarray(x, dtype)
    dt = np.asarray(dt, dtype)
    A = np.asarray(A, dtype)
    Bm = np.asarray(Bm, dtype)
    Cm = np.asarray(Cm, dtype)
    H = x.shape[1]
    gh = _group_of_head(H, Bm.shape[1])
    a = np.exp(dt * A[None, :])
    new = a[:, :, None, None] * state + (dt[..., None] * x)[..., None] * Bm[:, gh, None, :]
    y = np.einsum("bhpn,bhn->bhp", new, Cm[:, gh, :])
    if D is not None:
        y = y + np.asarray(D, dtype)[None, :, None] * x
    return y, new


# ---------------------------------------------------------------------------------------
# Chunked four-stage form.  Every intermediate is exposed so each HIP stage can be
# compared on its own.
# ---------------------------------------------------------------------------------------

def chunk_cumsum(dt, A, Q, dtype=np.float64):
    """Stage 1.  dA_cs[b,h,c,l] = sum_{i<=l} dt[b,cQ+i,h]*A[h] (restarts every chunk) and
    dt transposed to [B,H,nc,Q].  A ragged tail is padded with dt = 0 (no-op steps)."""
    dt = np.asarray(dt, dtype)
    A = np.asarray(A, dtype)
    Bsz, L, H = dt.shape
    nc = -(-L // Q)
    dtp = np.zeros((Bsz, nc * Q, H), dtype)
    dtp[:, :L] = dt
    dt_c = dtp.reshape(Bsz, nc, Q, H).transpose(0, 3, 1, 2).copy()     # [B,H,nc,Q]
    dA_cs = np.cumsum(dt_c * A[None, :, None, None], axis=-1)
    return dA_cs, dt_c


def _pad_chunks(t, Q):
    Bsz, L = t.shape[:2]
    nc = -(-L // Q)
    if nc * Q != L:
        pad = np.zeros((Bsz, nc * Q - L) + t.shape[2:], t.dtype)
        t = np.concatenate([t, pad], axis=1)
    return t.reshape((Bsz, nc, Q) + t.shape[2:])


def chunk_state(x, Bm, dA_cs, dt_c, dtype=np.float64):
    """Stage 2.  S[b,c,h,p,n] = sum_l exp(dA_cs[c,Q-1]-dA_cs[c,l]) dt[c,l] x[c,l,h,p] B[c,l,g,n]."""
    x = np.asarray(x, dtype)
    Bm = np.asarray(Bm, dtype)
    Q = dA_cs.shape[-1]
    H = x.shape[2]
    gh = _group_of_head(H, Bm.shape[2])
    xc = _pad_chunks(x, Q)                                              # [B,nc,Q,H,P]
    Bc = _pad_chunks(Bm, Q)[:, :, :, gh, :]                             # [B,nc,Q,H,N]
    w = np.exp(dA_cs[..., -1:] - dA_cs) * dt_c                          # [B,H,nc,Q]
    return np.einsum("bhcl,bclhp,bclhn->bchpn", w, xc, Bc)


def state_passing(S, dA_chunk_end, init=None, dtype=np.float64):
    """Stage 3.  prev[c] = state entering chunk c; H_{c+1} = exp(dA_chunk_end[c]) H_c + S_c.
    dA_chunk_end is [B,H,nc] = dA_cs[..., -1]."""
    S = np.asarray(S, dtype)
    Bsz, nc, H, P, N = S.shape
    h = np.zeros((Bsz, H, P, N), dtype) if init is None else np.array(init, dtype)
    prev = np.empty_like(S)
    for c in range(nc):
        prev[:, c] = h
        h = np.exp(dA_chunk_end[:, :, c])[:, :, None, None] * h + S[:, c]
    return prev, h


def chunk_scan(x, Bm, Cm, dA_cs, dt_c, prev, D=None, dtype=np.float64):
    """Stage 4.  y[c,l] = sum_{s<=l} (C[c,l].B[c,s]) exp(dA_cs[l]-dA_cs[s]) dt[s] x[c,s]
    + exp(dA_cs[l]) (prev_c . C[c,l]) + D x[c,l].  The mask is applied before exp."""
    x = np.asarray(x, dtype)
    Bm = np.asarray(Bm, dtype)
    Cm = np.asarray(Cm, dtype)
    Bsz, L, H, P = x.shape
    Q = dA_cs.shape[-1]
    gh = _group_of_head(H, Bm.shape[2])
    xc = _pad_chunks(x, Q)
    Bc = _pad_chunks(Bm, Q)[:, :, :, gh, :]
    Cc = _pad_chunks(Cm, Q)[:, :, :, gh, :]
    CB = np.einsum("bclhn,bcshn->bhcls", Cc, Bc)                        # [B,H,nc,Q,Q]
    diff = dA_cs[..., :, None] - dA_cs[..., None, :]                    # [B,H,nc,l,s]
    mask = np.tril(np.ones((Q, Q), bool))
    lam = np.where(mask, np.exp(np.where(mask, diff, 0.0)), 0.0)
    M = CB * lam * dt_c[..., None, :]
    y = np.einsum("bhcls,bcshp->bclhp", M, xc)
    y += np.einsum("bhcl,bclhn,bchpn->bclhp", np.exp(dA_cs), Cc, np.asarray(prev, dtype))
    if D is not None:
        y += np.asarray(D, dtype)[None, None, None, :, None] * xc
    return y.reshape(Bsz, -1, H, P)[:, :L]


def ssd_chunked(x, dt, A, Bm, Cm, D=None, init=None, chunk=64, dtype=np.float64,
                return_intermediates=False):
    """Stages 1-4 composed."""
    dA_cs, dt_c = chunk_cumsum(dt, A, chunk, dtype)
    S = chunk_state(x, Bm, dA_cs, dt_c, dtype)
    prev, final = state_passing(S, dA_cs[..., -1], init, dtype)
    y = chunk_scan(x, Bm, Cm, dA_cs, dt_c, prev, D, dtype)
    if return_intermediates:
        return y, final, dict(dA_cs=dA_cs, dt_c=dt_c, S=S, prev=prev)
    return y, final


def ssd_quadratic(x, dt, A, Bm, Cm, D=None, init=None, dtype=np.float64):
    """O(L^2) 'attention form' brute force for small L:
    Y = (Lambda o C B^T) diag(dt) X + exp(cum) (init . C) + D X,
    Lambda[i,j] = exp(sum_{k=j+1..i} dt_k A) for j <= i."""
    x = np.asarray(x, dtype)
    dt = np.asarray(dt, dtype)
    A = np.asarray(A, dtype)
    Bm = np.asarray(Bm, dtype)
    Cm = np.asarray(Cm, dtype)
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    gh = _group_of_head(H, G)
    y = np.zeros((Bsz, L, H, P), dtype)
    final = np.zeros((Bsz, H, P, N), dtype)
    for b in range(Bsz):
        for h in range(H):
            g = gh[h]
            dA = dt[b, :, h] * A[h]
            for i in range(L):
                acc = np.zeros(P, dtype)
                for j in range(i + 1):
                    lam = np.exp(dA[j + 1:i + 1].sum())
                    acc += (Cm[b, i, g] @ Bm[b, j, g]) * lam * dt[b, j, h] * x[b, j, h]
                if init is not None:
                    acc += np.exp(dA[:i + 1].sum()) * (np.asarray(init, dtype)[b, h] @ Cm[b, i, g])
                if D is not None:
                    acc += D[h] * x[b, i, h]
                y[b, i, h] = acc
            for j in range(L):
                lam = np.exp(dA[j + 1:].sum())
                final[b, h] += lam * dt[b, j, h] * np.outer(x[b, j, h], Bm[b, j, g])
            if init is not None:
                final[b, h] += np.exp(dA.sum()) * np.asarray(init, dtype)[b, h]
    return y, final


def rel_err(out, ref) -> float:
    """The parity metric: max |out - ref| / rms(ref)."""
    out = np.asarray(out, np.float64)
    ref = np.asarray(ref, np.float64)
    rms = float(np.sqrt(np.mean(ref * ref)))
    return float(np.max(np.abs(out - ref)) / max(rms, 1e-300))
