"""CPU restatement (numpy float64) of the backward pass of the SSD scan.  Test infrastructure only: imported
by tests/ to check the HIP backward (trading_bot_0_amd/csrc/ssd_backward_kernels.hip, ssd_chunk_scan_bwd).
The reference tree holds no source for this path (its historical benchmark case is mamba2_fwd_bwd_train,
benchmark_results/bench_20260112_070055.json:16-23); the arithmetic is the adjoint of the recurrence that
oracle/ssd_oracle.py:ssd_sequential states.  tests/test_oracle_backward.py pins every gradient here against
central differences of that forward, and the decomposition the GPU path uses against this sequential adjoint."""
import numpy as np

from . import ssd_oracle as orc


def ssd_backward_sequential(x, dt, A, Bm, Cm, D, init, dy, dfinal=None, reset=None):
    """Adjoint of ssd_sequential, one timestep at a time, backwards.
    With h_t = a_t h_{t-1} + dt_t x_t (x) B_t, y_t = h_t C_t + D x_t, a_t = exp(dt_t A) and g_t = dLoss/dh_t:
        g_t   = dy_t (x) C_t + a_{t+1} g_{t+1}                    (g_{L-1} also takes dfinal)
        dC_t  = sum_{h in group} dy_t . h_t            dB_t = sum_{h in group} dt_t x_t . g_t
        dx_t  = D dy_t + dt_t g_t B_t                  ddt_t = <g_t, x_t (x) B_t> + A a_t <g_t, h_{t-1}>
        dA    = sum_t dt_t a_t <g_t, h_{t-1}>          dD = sum dy_t x_t        dinit = a_0 g_0
    reset [B,L] (optional) as in ssd_sequential: h_{t-1} is zero for a row that restarts before step t, and its
    adjoint does not reach the steps before.
    Returns a dict with dx, ddt, dA, dB, dC, dD (None without D), dinit, and dA_scale, dD_scale [H]: the 2-norms
    of the terms that dA and dD sum over batch and time (the scale rounding errors of such sums are measured on)."""
    x = np.asarray(x, np.float64)
    dt = np.asarray(dt, np.float64)
    A = np.asarray(A, np.float64)
    Bm = np.asarray(Bm, np.float64)
    Cm = np.asarray(Cm, np.float64)
    dy = np.asarray(dy, np.float64)
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    gh = orc._group_of_head(H, G)
    # forward, keeping every state
    hs = np.empty((L + 1, Bsz, H, P, N))
    hs[0] = 0.0 if init is None else np.asarray(init, np.float64)
    a = np.exp(dt * A[None, None, :])                                   # [B,L,H]
    rs = None if reset is None else (np.asarray(reset) != 0)
    starts = hs if rs is None else np.empty((L, Bsz, H, P, N))          # the state step t starts from
    for t in range(L):
        if rs is not None:
            starts[t] = hs[t]
            starts[t][rs[:, t]] = 0.0
        hs[t + 1] = a[:, t, :, None, None] * starts[t] + (dt[:, t, :, None] * x[:, t])[..., None] * Bm[:, t, gh, None, :]
    dx = np.zeros_like(x)
    ddt = np.zeros_like(dt)
    dBh = np.zeros((Bsz, L, H, N))
    dCh = np.zeros((Bsz, L, H, N))
    dA = np.zeros(H)
    dA_sq = np.zeros(H)
    g = np.zeros((Bsz, H, P, N)) if dfinal is None else np.array(dfinal, np.float64)
    for t in range(L - 1, -1, -1):
        Ct, Bt = Cm[:, t, gh, :], Bm[:, t, gh, :]                        # [B,H,N]
        g = g + dy[:, t][..., None] * Ct[:, :, None, :]                  # adjoint of h_t
        dCh[:, t] = np.einsum("bhp,bhpn->bhn", dy[:, t], hs[t + 1])
        gB = np.einsum("bhpn,bhn->bhp", g, Bt)
        dx[:, t] = dt[:, t, :, None] * gB
        dBh[:, t] = dt[:, t, :, None] * np.einsum("bhpn,bhp->bhn", g, x[:, t])
        gh_prev = np.einsum("bhpn,bhpn->bh", g, starts[t])               # <g_t, h_{t-1}>
        ddt[:, t] = np.einsum("bhp,bhp->bh", gB, x[:, t]) + A[None, :] * a[:, t] * gh_prev
        dA += (dt[:, t] * a[:, t] * gh_prev).sum(0)
        dA_sq += ((dt[:, t] * a[:, t] * gh_prev) ** 2).sum(0)
        g = a[:, t, :, None, None] * g                                   # adjoint of h_{t-1}
        if rs is not None:
            g[rs[:, t]] = 0.0
    out = {"ddt": ddt, "dA": dA, "dinit": g, "dD": None, "dA_scale": np.sqrt(dA_sq), "dD_scale": None}
    if D is not None:
        dx = dx + np.asarray(D, np.float64)[None, None, :, None] * dy
        out["dD"] = np.einsum("blhp,blhp->h", dy, x)
        out["dD_scale"] = np.sqrt(np.einsum("blhp,blhp->h", (dy * x) ** 2, np.ones_like(x)))
    out["dx"] = dx
    hpg = H // G
    out["dB"] = dBh.reshape(Bsz, L, G, hpg, N).sum(3)
    out["dC"] = dCh.reshape(Bsz, L, G, hpg, N).sum(3)
    return out


def scan_general(xr, log_decay, weight, Br, Cr, init=None):
    """The recurrence with decay and input weight given per step instead of derived from dt and A:
    h_t = exp(log_decay_t) h_{t-1} + weight_t x_t (x) B_t, y_t = h_t C_t.  B, C are per head here ([B,L,H,N])."""
    Bsz, L, H, P = xr.shape
    N = Br.shape[3]
    h = np.zeros((Bsz, H, P, N)) if init is None else np.array(init, np.float64)
    y = np.empty((Bsz, L, H, P))
    for t in range(L):
        h = np.exp(log_decay[:, t])[:, :, None, None] * h + (weight[:, t, :, None] * xr[:, t])[..., None] * Br[:, t, :, None, :]
        y[:, t] = np.einsum("bhpn,bhn->bhp", h, Cr[:, t])
    return y, h


def ssd_backward_by_scans(x, dt, A, Bm, Cm, D, init, dy, dfinal=None, final=None):
    """The same gradients as three instances of the forward recurrence with the roles of the operands swapped,
    which is how the GPU path computes them (every heavy step is then the forward's own kernels):
      r   = reversed scan(x <- dy, B <- C, C <- B), decays shifted by one step, unit weights, init <- dfinal
            r_t = g_t B_t;  dx = D dy + dt r;  its final state, decayed by a_0, is dinit
      yB  = the same reversed scan of the transposed state (x <- C, B <- dy, C <- x): yB_t = x_t . g_t
            dB = sum over the group's heads of dt yB
      yC  = forward-time scan of the transposed state (x <- B, B <- x, C <- dy), the forward's own decays and
            weights, init <- init^T: yC_t = dy_t . h_t;  dC = sum over the group's heads of yC
      ddt_t = x_t . r_t + A q_t,  q_t = sum_{u >= t} (C_u . yC_u - dt_u x_u . r_u) + <dfinal, final>,
      dA = sum dt q.   (q_t = a_t <g_t, h_{t-1}> telescopes: a_t <g_t,h_{t-1}> = <g_t,h_t> - dt_t <g_t, x_t (x) B_t>
      and <g_t,h_t> = dy_t . (h_t C_t) + a_{t+1} <g_{t+1}, h_t>.)"""
    x = np.asarray(x, np.float64)
    dt = np.asarray(dt, np.float64)
    A = np.asarray(A, np.float64)
    Bm = np.asarray(Bm, np.float64)
    Cm = np.asarray(Cm, np.float64)
    dy = np.asarray(dy, np.float64)
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    gh = orc._group_of_head(H, G)
    Bh, Ch = Bm[:, :, gh, :], Cm[:, :, gh, :]                            # per head
    rev = lambda v: v[:, ::-1]
    la = dt * A[None, None, :]
    la_rev = np.concatenate([np.zeros((Bsz, 1, H)), rev(la)[:, :-1]], 1)  # step tau decays by a_{L-tau}; a'_0 = 1
    ones = np.ones((Bsz, L, H))
    r_rev, gfin = scan_general(rev(dy), la_rev, ones, rev(Ch), rev(Bh), dfinal)
    r = rev(r_rev)
    dfT = None if dfinal is None else np.swapaxes(np.asarray(dfinal, np.float64), 2, 3)
    yB_rev, _ = scan_general(rev(Ch), la_rev, ones, rev(dy), rev(x), dfT)
    yB = rev(yB_rev)
    inT = None if init is None else np.swapaxes(np.asarray(init, np.float64), 2, 3)
    yC, _ = scan_general(Bh, la, dt, x, dy, inT)
    e1 = np.einsum("blhp,blhp->blh", x, r)
    u = np.einsum("blhn,blhn->blh", Ch, yC) - dt * e1
    q = np.cumsum(u[:, ::-1], 1)[:, ::-1]
    if dfinal is not None:
        q = q + np.einsum("bhpn,bhpn->bh", np.asarray(dfinal, np.float64), np.asarray(final, np.float64))[:, None, :]
    hpg = H // G
    out = {"ddt": e1 + A[None, None, :] * q, "dA": (dt * q).sum((0, 1)), "dD": None,
           "dinit": np.exp(la[:, 0])[:, :, None, None] * gfin,
           "dB": (dt[..., None] * yB).reshape(Bsz, L, G, hpg, N).sum(3),
           "dC": yC.reshape(Bsz, L, G, hpg, N).sum(3)}
    dx = dt[..., None] * r
    if D is not None:
        dx = dx + np.asarray(D, np.float64)[None, None, :, None] * dy
        out["dD"] = np.einsum("blhp,blhp->h", dy, x)
    out["dx"] = dx
    return out
