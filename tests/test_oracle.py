"""Pins the CPU oracle (oracle/ssd_oracle.py, oracle/ssd_oracle.c) with what the mathematics
fixes: library routines (scipy.signal.lfilter, numpy.cumsum, numpy.einsum), closed forms,
brute force on tiny inputs and algebraic invariants.  The reference tree holds no vectors for
this path, so these checks are what stands between a typo in the oracle and a wrong kernel.
Each check is chosen so that a dropped factor, a wrong sign or an off-by-one index fails it."""
import numpy as np
import pytest
from scipy.signal import lfilter

from oracle import ssd_oracle as orc
from oracle import c_oracle

RNG = np.random.default_rng(1234)


def rand_inputs(Bsz=2, L=48, H=4, P=8, N=8, G=2, with_init=True, with_D=True, rng=RNG):
    x = rng.standard_normal((Bsz, L, H, P))
    dt = np.log1p(np.exp(rng.standard_normal((Bsz, L, H)) - 1.0))
    A = -np.exp(rng.uniform(np.log(0.5), np.log(8.0), H))
    Bm = rng.standard_normal((Bsz, L, G, N)) / np.sqrt(N)
    Cm = rng.standard_normal((Bsz, L, G, N)) / np.sqrt(N)
    D = rng.standard_normal(H) if with_D else None
    init = rng.standard_normal((Bsz, H, P, N)) if with_init else None
    return x, dt, A, Bm, Cm, D, init


# ---- ssd_sequential ------------------------------------------------------------------------

def test_sequential_is_textbook_iir_for_scalar_state():
    # P = N = 1, constant dt: h_t = r h_{t-1} + dt x_t B_t ; y_t = C h_t  ==  lfilter([1],[1,-r])
    L = 200
    x = RNG.standard_normal((1, L, 1, 1))
    Bm = RNG.standard_normal((1, L, 1, 1))
    dtv, a = 0.37, -1.3
    dt = np.full((1, L, 1), dtv)
    A = np.array([a])
    Cm = np.ones((1, L, 1, 1))
    y, final = orc.ssd_sequential(x, dt, A, Bm, Cm)
    r = np.exp(dtv * a)
    ref = lfilter([1.0], [1.0, -r], dtv * x[0, :, 0, 0] * Bm[0, :, 0, 0])
    np.testing.assert_allclose(y[0, :, 0, 0], ref, rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(final[0, 0, 0, 0], ref[-1], rtol=1e-12)


def test_sequential_closed_form_constant_inputs():
    # constant dt, x, B: h_t = r^t init + dt x (x) B (1 - r^t)/(1 - r)
    L, P, N = 37, 3, 5
    xv, bv, cv = RNG.standard_normal(P), RNG.standard_normal(N), RNG.standard_normal(N)
    init = RNG.standard_normal((1, 1, P, N))
    dtv, a, d = 0.21, -2.2, 0.7
    x = np.broadcast_to(xv, (1, L, 1, P)).copy()
    Bm = np.broadcast_to(bv, (1, L, 1, N)).copy()
    Cm = np.broadcast_to(cv, (1, L, 1, N)).copy()
    y, final = orc.ssd_sequential(x, np.full((1, L, 1), dtv), np.array([a]), Bm, Cm, np.array([d]), init)
    r = np.exp(dtv * a)
    for t in (1, 2, 17, L):
        h = r ** t * init[0, 0] + dtv * np.outer(xv, bv) * (1 - r ** t) / (1 - r)
        np.testing.assert_allclose(y[0, t - 1, 0], h @ cv + d * xv, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(final[0, 0], h, rtol=1e-11, atol=1e-12)


def test_sequential_zero_decay_rate_is_cumsum():
    # A -> 0-: h_t = init + cumsum(dt x (x) B)
    x, dt, A, Bm, Cm, D, init = rand_inputs(Bsz=1, L=20, H=2, P=3, N=4, G=1)
    A = np.full_like(A, -1e-300)
    y, final = orc.ssd_sequential(x, dt, A, Bm, Cm, None, init)
    outer = np.einsum("blh,blhp,bln->blhpn", dt, x, Bm[:, :, 0])
    h = init[:, None] + np.cumsum(outer, axis=1)
    np.testing.assert_allclose(final, h[:, -1], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(y, np.einsum("blhpn,bln->blhp", h, Cm[:, :, 0]), rtol=1e-12, atol=1e-12)


def test_sequential_equals_quadratic_brute_force():
    x, dt, A, Bm, Cm, D, init = rand_inputs(Bsz=2, L=13, H=4, P=3, N=5, G=2)
    y, final = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init)
    yq, fq = orc.ssd_quadratic(x, dt, A, Bm, Cm, D, init)
    np.testing.assert_allclose(y, yq, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(final, fq, rtol=1e-11, atol=1e-12)


def test_y_reads_the_updated_state():
    # single step from zero state: y_0 = dt (C.B) x + D x  (would be D x if y read h_{t-1})
    x, dt, A, Bm, Cm, D, _ = rand_inputs(Bsz=1, L=1, H=2, P=4, N=6, G=1, with_init=False)
    y, _ = orc.ssd_sequential(x, dt, A, Bm, Cm, D)
    cb = (Cm[0, 0, 0] * Bm[0, 0, 0]).sum()
    ref = dt[0, 0, :, None] * cb * x[0, 0] + D[:, None] * x[0, 0]
    np.testing.assert_allclose(y[0, 0], ref, rtol=1e-12)


# ---- the four stages -----------------------------------------------------------------------

def test_chunk_cumsum_is_numpy_cumsum_per_chunk_with_zero_padded_tail():
    _, dt, A, *_ = rand_inputs(Bsz=2, L=50, H=3)
    Q = 16
    dA_cs, dt_c = orc.chunk_cumsum(dt, A, Q)
    assert dA_cs.shape == (2, 3, 4, 16)
    for c in range(4):
        seg = dt[:, c * Q:(c + 1) * Q]                                   # [B, <=Q, H]
        ref = np.cumsum(seg * A[None, None, :], axis=1).transpose(0, 2, 1)
        n = seg.shape[1]
        np.testing.assert_allclose(dA_cs[:, :, c, :n], ref, rtol=1e-13)
        np.testing.assert_allclose(dt_c[:, :, c, :n], seg.transpose(0, 2, 1))
        if n < Q:  # ragged tail: dt = 0, cumsum stays flat
            assert np.all(dt_c[:, :, c, n:] == 0)
            np.testing.assert_allclose(dA_cs[:, :, c, n:], np.repeat(ref[:, :, -1:], Q - n, axis=2))


def test_chunk_state_tile_einsum_and_geometric_closed_form():
    x, dt, A, Bm, Cm, _, _ = rand_inputs(Bsz=1, L=32, H=2, P=3, N=4, G=1)
    Q = 16
    dA_cs, dt_c = orc.chunk_cumsum(dt, A, Q)
    S = orc.chunk_state(x, Bm, dA_cs, dt_c)
    for c in range(2):
        for h in range(2):
            al = dA_cs[0, h, c]
            w = np.exp(al[-1] - al) * dt_c[0, h, c]
            ref = np.einsum("l,lp,ln->pn", w, x[0, c * Q:(c + 1) * Q, h], Bm[0, c * Q:(c + 1) * Q, 0])
            np.testing.assert_allclose(S[0, c, h], ref, rtol=1e-12, atol=1e-13)
    # constant inputs: S = dt x(x)B (1 - r^Q)/(1 - r)
    xv, bv, dtv, a = RNG.standard_normal(3), RNG.standard_normal(4), 0.3, -1.7
    xc = np.broadcast_to(xv, (1, Q, 1, 3)).copy()
    Bc = np.broadcast_to(bv, (1, Q, 1, 4)).copy()
    dA, dtc = orc.chunk_cumsum(np.full((1, Q, 1), dtv), np.array([a]), Q)
    r = np.exp(dtv * a)
    np.testing.assert_allclose(orc.chunk_state(xc, Bc, dA, dtc)[0, 0, 0],
                               dtv * np.outer(xv, bv) * (1 - r ** Q) / (1 - r), rtol=1e-12)


def test_state_passing_is_lfilter_and_pure_decay():
    nc = 9
    S = RNG.standard_normal((1, nc, 1, 2, 3))
    a_end = np.full((1, 1, nc), -0.4)
    prev, final = orc.state_passing(S, a_end)
    r = np.exp(-0.4)
    for p in range(2):
        for n in range(3):
            ref = lfilter([1.0], [1.0, -r], S[0, :, 0, p, n])          # H_{c+1}
            np.testing.assert_allclose(prev[0, 1:, 0, p, n], ref[:-1], rtol=1e-12)
            np.testing.assert_allclose(final[0, 0, p, n], ref[-1], rtol=1e-12)
    assert np.all(prev[0, 0] == 0)
    # S = 0: final = exp(sum of chunk-end log-decays) * init
    init = RNG.standard_normal((2, 3, 2, 2))
    a_end = -RNG.uniform(0.1, 2.0, (2, 3, 5))
    prev, final = orc.state_passing(np.zeros((2, 5, 3, 2, 2)), a_end, init)
    np.testing.assert_allclose(final, np.exp(a_end.sum(-1))[..., None, None] * init, rtol=1e-12)
    np.testing.assert_allclose(prev[:, 0], init)


def test_chunk_scan_brute_force_loops():
    x, dt, A, Bm, Cm, D, _ = rand_inputs(Bsz=1, L=16, H=2, P=3, N=4, G=1, with_init=False)
    Q = 8
    dA_cs, dt_c = orc.chunk_cumsum(dt, A, Q)
    prev = RNG.standard_normal((1, 2, 2, 3, 4))
    y = orc.chunk_scan(x, Bm, Cm, dA_cs, dt_c, prev, D)
    for c in range(2):
        for h in range(2):
            for l in range(Q):
                t = c * Q + l
                acc = np.exp(dA_cs[0, h, c, l]) * (prev[0, c, h] @ Cm[0, t, 0]) + D[h] * x[0, t, h]
                for s in range(l + 1):
                    ts = c * Q + s
                    acc = acc + (Cm[0, t, 0] @ Bm[0, ts, 0]) * np.exp(dA_cs[0, h, c, l] - dA_cs[0, h, c, s]) \
                        * dt[0, ts, h] * x[0, ts, h]
                np.testing.assert_allclose(y[0, t, h], acc, rtol=1e-11, atol=1e-12)


def test_chunk_scan_does_not_overflow_on_masked_entries():
    # positive exponents above the diagonal (here ~ +900) must be masked before exp
    L, Q = 8, 8
    x, _, _, Bm, Cm, D, _ = rand_inputs(Bsz=1, L=L, H=1, P=2, N=2, G=1, with_init=False)
    dt = np.full((1, L, 1), 2.0)
    A = np.array([-64.0])
    with np.errstate(over="raise", invalid="raise"):
        y, final = orc.ssd_chunked(x, dt, A, Bm, Cm, D, chunk=Q)
    ys, fs = orc.ssd_sequential(x, dt, A, Bm, Cm, D)
    np.testing.assert_allclose(y, ys, rtol=1e-12, atol=1e-300)
    assert np.all(np.isfinite(y))


@pytest.mark.parametrize("Q", [16, 32, 64, 128, 256])
def test_chunked_equals_sequential_for_every_chunk_size(Q):
    x, dt, A, Bm, Cm, D, init = rand_inputs(Bsz=2, L=200, H=4, P=4, N=8, G=2)   # 200 is ragged for all Q
    ys, fs = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init)
    yc, fc = orc.ssd_chunked(x, dt, A, Bm, Cm, D, init, chunk=Q)
    np.testing.assert_allclose(yc, ys, rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(fc, fs, rtol=1e-10, atol=1e-11)


# ---- invariants ----------------------------------------------------------------------------

def test_split_sequence_associativity():
    x, dt, A, Bm, Cm, D, init = rand_inputs(L=60)
    y, f = orc.ssd_chunked(x, dt, A, Bm, Cm, D, init, chunk=16)
    L1 = 23
    y1, f1 = orc.ssd_chunked(x[:, :L1], dt[:, :L1], A, Bm[:, :L1], Cm[:, :L1], D, init, chunk=16)
    y2, f2 = orc.ssd_chunked(x[:, L1:], dt[:, L1:], A, Bm[:, L1:], Cm[:, L1:], D, f1, chunk=16)
    np.testing.assert_allclose(np.concatenate([y1, y2], 1), y, rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(f2, f, rtol=1e-10, atol=1e-11)


def test_linearity_in_x_and_init_and_init_response():
    x, dt, A, Bm, Cm, D, init = rand_inputs(L=40)
    x2, init2 = RNG.standard_normal(x.shape), RNG.standard_normal(init.shape)
    ya, fa = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init)
    yb, fb = orc.ssd_sequential(x2, dt, A, Bm, Cm, D, init2)
    yc, fc = orc.ssd_sequential(2 * x - 3 * x2, dt, A, Bm, Cm, D, 2 * init - 3 * init2)
    np.testing.assert_allclose(yc, 2 * ya - 3 * yb, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(fc, 2 * fa - 3 * fb, rtol=1e-9, atol=1e-10)
    # y(init) - y(0) = exp(global cumsum of dt A) * (init . C_t)
    y0, _ = orc.ssd_sequential(x, dt, A, Bm, Cm, D, None)
    cum = np.cumsum(dt * A[None, None, :], axis=1)                        # [B,L,H]
    gh = np.arange(4) // 2
    ref = np.exp(cum)[..., None] * np.einsum("bhpn,blhn->blhp", init, Cm[:, :, gh])
    np.testing.assert_allclose(ya - y0, ref, rtol=1e-9, atol=1e-10)


def test_zero_dt_rows_are_no_ops():
    x, dt, A, Bm, Cm, D, init = rand_inputs(L=30, with_D=False)
    keep = np.ones(30, bool)
    keep[[4, 5, 17, 29]] = False
    dtz = dt.copy()
    dtz[:, ~keep] = 0.0
    y, f = orc.ssd_sequential(x, dtz, A, Bm, Cm, None, init)
    yk, fk = orc.ssd_sequential(x[:, keep], dt[:, keep], A, Bm[:, keep], Cm[:, keep], None, init)
    np.testing.assert_allclose(y[:, keep], yk, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(f, fk, rtol=1e-11, atol=1e-12)


def test_group_expansion_equivalence():
    x, dt, A, Bm, Cm, D, init = rand_inputs(H=4, G=2)
    y, f = orc.ssd_chunked(x, dt, A, Bm, Cm, D, init, chunk=16)
    ye, fe = orc.ssd_chunked(x, dt, A, np.repeat(Bm, 2, axis=2), np.repeat(Cm, 2, axis=2), D, init, chunk=16)
    np.testing.assert_allclose(y, ye, rtol=1e-12)
    np.testing.assert_allclose(f, fe, rtol=1e-12)


def test_step_applied_L_times_equals_sequential():
    x, dt, A, Bm, Cm, D, init = rand_inputs(L=25)
    ys, fs = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init)
    st = init.copy()
    for t in range(25):
        y, st = orc.ssd_step(st, x[:, t], dt[:, t], A, Bm[:, t], Cm[:, t], D)
        np.testing.assert_allclose(y, ys[:, t], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(st, fs, rtol=1e-11, atol=1e-12)


# ---- C restatement -------------------------------------------------------------------------

def test_c_oracle_matches_numpy_oracle():
    x, dt, A, Bm, Cm, D, init = rand_inputs(Bsz=3, L=70, H=4, P=8, N=16, G=2)
    ys, fs = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init)
    yc, fc = c_oracle.ssd_sequential_c(x, dt, A, Bm, Cm, D, init, nthreads=4)
    np.testing.assert_allclose(yc, ys, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(fc, fs, rtol=1e-11, atol=1e-12)
    y32, f32 = c_oracle.ssd_sequential_c(x, dt, A, Bm, Cm, D, init, dtype=np.float32, nthreads=2)
    assert orc.rel_err(y32, ys) < 1e-5 and orc.rel_err(f32, fs) < 1e-5
    yn, fn = c_oracle.ssd_sequential_c(x, dt, A, Bm, Cm, None, None)
    y0, f0 = orc.ssd_sequential(x, dt, A, Bm, Cm, None, None)
    np.testing.assert_allclose(yn, y0, rtol=1e-11, atol=1e-12)
    y1, s1 = c_oracle.ssd_step_c(init, x[:, 0], dt[:, 0], A, Bm[:, 0], Cm[:, 0], D)
    y1n, s1n = orc.ssd_step(init, x[:, 0], dt[:, 0], A, Bm[:, 0], Cm[:, 0], D)
    np.testing.assert_allclose(y1, y1n, rtol=1e-12)
    np.testing.assert_allclose(s1, s1n, rtol=1e-12)


def test_reset_is_a_fresh_sequence_from_that_timestep():
    """ssd_sequential(reset=...) against the reset-free function: a row with resets at t1 < t2 is the
    concatenation of three independent scans, the later two from a zero state; a reset at t = 0 discards
    the initial state; rows without resets are untouched."""
    x, dt, A, Bm, Cm, D, init = rand_inputs(Bsz=3, L=40)
    reset = np.zeros((3, 40), np.uint8)
    reset[1, [13, 29]] = 1
    reset[2, 0] = 1
    y, f = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init, reset=reset)
    y0, f0 = orc.ssd_sequential(x[:1], dt[:1], A, Bm[:1], Cm[:1], D, init[:1])
    np.testing.assert_array_equal(y[:1], y0)
    np.testing.assert_array_equal(f[:1], f0)
    parts, st = [], init[1:2]
    for a, b in ((0, 13), (13, 29), (29, 40)):
        yp, fp = orc.ssd_sequential(x[1:2, a:b], dt[1:2, a:b], A, Bm[1:2, a:b], Cm[1:2, a:b], D, st)
        parts.append(yp)
        st = None
    np.testing.assert_allclose(y[1:2], np.concatenate(parts, 1), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(f[1:2], fp, rtol=1e-12, atol=1e-13)
    y2, f2 = orc.ssd_sequential(x[2:], dt[2:], A, Bm[2:], Cm[2:], D, None)
    np.testing.assert_allclose(y[2:], y2, rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(f[2:], f2, rtol=1e-12, atol=1e-13)


def test_torch_cpu_restatement_matches_the_oracle():
    """oracle/ssd_torch_cpu.py (the ATen-CPU form bench.py times as the CPU baseline) against the float64
    sequential recurrence: groups, a ragged length, an initial state; float64 to 1e-10, float32 to 1e-4."""
    import torch
    from oracle.ssd_torch_cpu import ssd_chunked_torch
    rng = np.random.default_rng(5)
    Bsz, L, H, P, N, G, Q = 2, 150, 4, 8, 16, 2, 64
    x = rng.standard_normal((Bsz, L, H, P))
    dt = np.log1p(np.exp(rng.standard_normal((Bsz, L, H)) - 2))
    A = -np.exp(rng.uniform(0, np.log(16), H))
    Bm = rng.standard_normal((Bsz, L, G, N)) / 4
    Cm = rng.standard_normal((Bsz, L, G, N)) / 4
    D = rng.standard_normal(H)
    init = rng.standard_normal((Bsz, H, P, N)) * 0.1
    yr, fr = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init)
    t = lambda a, d: torch.from_numpy(np.asarray(a)).to(d)
    for dtype, tol in ((torch.float64, 1e-10), (torch.float32, 1e-4)):
        y, f = ssd_chunked_torch(t(x, dtype), t(dt, dtype), t(A, dtype), t(Bm, dtype), t(Cm, dtype), t(D, dtype),
                                 t(init, dtype), chunk=Q)
        assert orc.rel_err(y.double().numpy(), yr) <= tol and orc.rel_err(f.double().numpy(), fr) <= tol
    y, f = ssd_chunked_torch(t(x, torch.float64), t(dt, torch.float64), t(A, torch.float64), t(Bm, torch.float64),
                             t(Cm, torch.float64), None, None, chunk=32)
    y0, f0 = orc.ssd_sequential(x, dt, A, Bm, Cm)
    assert orc.rel_err(y.numpy(), y0) <= 1e-10 and orc.rel_err(f.numpy(), f0) <= 1e-10
