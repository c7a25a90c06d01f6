"""Pins oracle/mamba2_block_oracle.py with library routines and direct formulas: the causal depthwise conv
against scipy.signal.lfilter per channel, the carried conv state against running the conv over the
concatenated input, softplus and SiLU against their definitions, the gated RMSNorm against an explicit
per-row loop, and the block against its own stages composed by hand."""
import numpy as np
from scipy.signal import lfilter

from oracle import mamba2_block_oracle as blk
from oracle import ssd_oracle as orc

RNG = np.random.default_rng(77)
H, P, N, G, K = 4, 8, 16, 2, 4
DI, GN, C, E = blk.split_widths(H, P, N, G)


def params():
    return dict(conv_w=RNG.standard_normal((C, K)), conv_b=RNG.standard_normal(C), dt_bias=RNG.standard_normal(H))


def test_widths():
    assert (DI, GN, C, E) == (32, 32, 96, 2 * 32 + 2 * 32 + 4)


def test_conv_is_an_fir_filter_per_channel_then_silu_and_split():
    p = params()
    z = RNG.standard_normal((3, 20, E))
    x, Bm, Cm, dt, state = blk.block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G)
    xbc = z[:, :, DI:DI + C]
    ref = np.empty_like(xbc)
    for c in range(C):
        # y[t] = sum_k w[c,k] * in[t-(K-1)+k]  ==  FIR with taps reversed
        ref[:, :, c] = lfilter(p["conv_w"][c, ::-1], [1.0], xbc[:, :, c], axis=1) + p["conv_b"][c]
    ref = ref / (1.0 + np.exp(-ref))
    np.testing.assert_allclose(x.reshape(3, 20, DI), ref[:, :, :DI], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(Bm.reshape(3, 20, GN), ref[:, :, DI:DI + GN], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(Cm.reshape(3, 20, GN), ref[:, :, DI + GN:], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(dt, np.log1p(np.exp(z[:, :, DI + C:] + p["dt_bias"])), rtol=1e-12)
    np.testing.assert_array_equal(state, xbc[:, -(K - 1):])


def test_conv_state_continues_the_sequence_also_for_windows_shorter_than_the_state():
    p = params()
    z = RNG.standard_normal((2, 11, E))
    full = blk.block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G)
    state, outs = None, []
    for a, b in ((0, 5), (5, 6), (6, 8), (8, 11)):          # windows of 5, 1, 2, 3 steps
        x, Bm, Cm, dt, state = blk.block_pre(z[:, a:b], p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, state)
        outs.append((x, Bm, Cm, dt))
    for i in range(4):
        np.testing.assert_allclose(np.concatenate([o[i] for o in outs], 1), full[i], rtol=1e-12, atol=1e-13)
    np.testing.assert_array_equal(state, full[4])


def test_restarts_cut_the_conv_history_like_separate_windows():
    """A window with restarts equals its episodes run as separate windows, each from a zero conv state (the first
    from the carried state), and the state it leaves is the last episode's."""
    p = params()
    L = 23
    z = RNG.standard_normal((3, L, E))
    st = RNG.standard_normal((3, K - 1, C))
    reset = np.zeros((3, L), np.uint8)
    reset[0, [5, 6, 14]] = 1          # back-to-back restarts
    reset[1, [0, L - 1]] = 1          # the first step (drops the carried state) and the last (a one-step episode)
    got = blk.block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, st, reset)
    for b in range(3):
        cuts = [0] + [int(t) for t in np.nonzero(reset[b])[0] if t > 0] + [L]
        state = None if reset[b, 0] else st[b:b + 1]
        pieces = []
        for a, e in zip(cuts[:-1], cuts[1:]):
            pieces.append(blk.block_pre(z[b:b + 1, a:e], p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, state))
            state = None
        for i in range(4):
            np.testing.assert_allclose(got[i][b:b + 1], np.concatenate([q[i] for q in pieces], 1), rtol=1e-12, atol=1e-13)
        np.testing.assert_array_equal(got[4][b:b + 1], pieces[-1][4])
    # no restarts: the mask changes nothing
    plain = blk.block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, st)
    same = blk.block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, st, np.zeros((3, L), np.uint8))
    for a, b_ in zip(plain, same):
        np.testing.assert_array_equal(a, b_)


def test_gated_rmsnorm_row_by_row():
    y = RNG.standard_normal((2, 5, H, P))
    z = RNG.standard_normal((2, 5, E))
    w = RNG.standard_normal(DI)
    out = blk.block_post(y, z, w, 1e-5)
    for b in range(2):
        for t in range(5):
            v = y[b, t].reshape(-1) * (z[b, t, :DI] / (1 + np.exp(-z[b, t, :DI])))
            ref = v / np.sqrt(np.sum(v * v) / DI + 1e-5) * w
            np.testing.assert_allclose(out[b, t], ref, rtol=1e-12, atol=1e-13)


def test_block_is_its_stages_composed_and_streams():
    d_model = 24
    p = params()
    p.update(in_proj=RNG.standard_normal((E, d_model)) / 5, out_proj=RNG.standard_normal((d_model, DI)) / 5,
             A=-np.exp(RNG.uniform(0, 2, H)), D=RNG.standard_normal(H), norm_w=RNG.standard_normal(DI),
             H=H, P=P, N=N, G=G, eps=1e-5)
    u = RNG.standard_normal((2, 17, d_model))
    out, conv, final = blk.block_forward(u, p)
    z = u @ p["in_proj"].T
    x, Bm, Cm, dt, conv2 = blk.block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G)
    y, f2 = orc.ssd_sequential(x, dt, p["A"], Bm, Cm, p["D"])
    np.testing.assert_allclose(out, blk.block_post(y, z, p["norm_w"], 1e-5) @ p["out_proj"].T, rtol=1e-12)
    np.testing.assert_array_equal(conv, conv2)
    np.testing.assert_array_equal(final, f2)
    # a prefix, then one timestep at a time, carrying both states
    o1, cs, ss = blk.block_forward(u[:, :9], p)
    outs = [o1]
    for t in range(9, 17):
        o, cs, ss = blk.block_forward(u[:, t:t + 1], p, cs, ss)
        outs.append(o)
    np.testing.assert_allclose(np.concatenate(outs, 1), out, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(ss, final, rtol=1e-10, atol=1e-12)


def _central(f, a, eps=1e-6):
    """Central differences of the scalar function f with respect to the array a (varied in place)."""
    g = np.zeros_like(a)
    it = np.nditer(a, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        keep = a[i]
        a[i] = keep + eps
        up = f()
        a[i] = keep - eps
        dn = f()
        a[i] = keep
        g[i] = (up - dn) / (2 * eps)
    return g


def test_post_backward_matches_central_differences():
    y = RNG.standard_normal((2, 3, H, P))
    z = RNG.standard_normal((2, 3, E))
    w = RNG.standard_normal(DI)
    dout = RNG.standard_normal((2, 3, DI))
    dy, dz, dw = blk.block_post_bwd(y, z, w, 1e-3, dout)
    loss = lambda: (blk.block_post(y, z, w, 1e-3) * dout).sum()
    np.testing.assert_allclose(dy, _central(loss, y), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(dz, _central(loss, z)[:, :, :DI], rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(dw, _central(loss, w), rtol=1e-6, atol=1e-8)


def test_pre_backward_matches_central_differences_with_state_and_restarts():
    p = params()
    L = 9
    z = RNG.standard_normal((2, L, E))
    st = RNG.standard_normal((2, K - 1, C))
    reset = np.zeros((2, L), np.uint8)
    reset[0, [3, 4]] = 1
    reset[1, L - 2] = 1
    gx, gB, gC = RNG.standard_normal((2, L, H, P)), RNG.standard_normal((2, L, G, N)), RNG.standard_normal((2, L, G, N))
    gdt, gst = RNG.standard_normal((2, L, H)), RNG.standard_normal((2, K - 1, C))
    for rs, gs in ((None, None), (reset, gst)):
        def loss():
            x, Bm, Cm, dt, so = blk.block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, st, rs)
            return (x * gx).sum() + (Bm * gB).sum() + (Cm * gC).sum() + (dt * gdt).sum() + (0.0 if gs is None else (so * gs).sum())
        dxbc, ddt_raw, dcw, dcb, ddb, dst = blk.block_pre_bwd(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, gx, gB, gC,
                                                             gdt, st, rs, gs)
        dz = _central(loss, z)
        np.testing.assert_allclose(dxbc, dz[:, :, DI:DI + C], rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(ddt_raw, dz[:, :, DI + C:], rtol=1e-6, atol=1e-8)
        assert np.abs(dz[:, :, :DI]).max() < 1e-8                      # pre does not read z
        np.testing.assert_allclose(dcw, _central(loss, p["conv_w"]), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(dcb, _central(loss, p["conv_b"]), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(ddb, _central(loss, p["dt_bias"]), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(dst, _central(loss, st), rtol=1e-6, atol=1e-8)


def test_block_backward_matches_central_differences():
    d_model = 6
    p = params()
    p.update(in_proj=RNG.standard_normal((E, d_model)) / 3, out_proj=RNG.standard_normal((d_model, DI)) / 5,
             A=-np.exp(RNG.uniform(0, 1.5, H)), D=RNG.standard_normal(H), norm_w=RNG.standard_normal(DI),
             H=H, P=P, N=N, G=G, eps=1e-3)
    u = RNG.standard_normal((2, 6, d_model))
    dout = RNG.standard_normal((2, 6, d_model))
    reset = np.zeros((2, 6), np.uint8)
    reset[1, 3] = 1
    for rs in (None, reset):
        g = blk.block_backward(u, p, dout, reset=rs)
        loss = lambda: (blk.block_forward(u, p, reset=rs)[0] * dout).sum()
        np.testing.assert_allclose(g["du"], _central(loss, u), rtol=2e-5, atol=1e-7)
        for name, key in (("in_proj", "din_proj"), ("conv_w", "dconv_w"), ("conv_b", "dconv_b"), ("dt_bias", "ddt_bias"),
                          ("A", "dA"), ("D", "dD"), ("norm_w", "dnorm_w"), ("out_proj", "dout_proj")):
            np.testing.assert_allclose(g[key], _central(loss, p[name]), rtol=2e-5, atol=1e-7, err_msg=name)
