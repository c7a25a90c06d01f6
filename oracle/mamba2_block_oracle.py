"""CPU restatement (numpy float64) of the Mamba-2 block stages around the SSD scan, forward and backward.  Test infrastructure
only: imported by tests/ to check the HIP kernels of trading_bot_0_amd/csrc/ssd_block_kernels.hip and the
block assembly of trading_bot_0_amd/block.py.  The reference tree holds no source for this layer (its slot is
trading_bots/src/torch/model/trading_model.rs:589-606); the arithmetic is the published Mamba-2 block:
causal depthwise conv + SiLU on (x, B, C), softplus(dt + bias), SSD, RMSNorm of y*silu(z), two projections.
Every function here is pinned in tests/test_oracle_block.py against library routines or direct formulas; the
backward functions against central differences of the forward ones."""
import numpy as np

from . import ssd_oracle as orc


def silu(v):
    return v / (1.0 + np.exp(-v))


def softplus(v):
    return np.logaddexp(0.0, v)


def split_widths(H, P, N, G):
    DI, GN = H * P, G * N
    return DI, GN, DI + 2 * GN, 2 * DI + 2 * GN + H


def block_pre(zxbcdt, conv_w, conv_b, dt_bias, H, P, N, G, conv_state=None, reset=None):
    """zxbcdt [B,L,E] laid out [z | x | B | C | dt_raw] -> x, Bm, Cm, dt, new conv state [B,d_conv-1,C].
    reset [B,L] (non-zero = an episode boundary before that timestep): from t on, inputs of timesteps before t
    (and the conv state) count as zeros."""
    zxbcdt = np.asarray(zxbcdt, np.float64)
    Bsz, L, E = zxbcdt.shape
    DI, GN, C, E_ = split_widths(H, P, N, G)
    assert E == E_
    K = conv_w.shape[1]
    xbc = zxbcdt[:, :, DI:DI + C]
    hist = np.zeros((Bsz, K - 1, C)) if conv_state is None else np.asarray(conv_state, np.float64)
    full = np.concatenate([hist, xbc], 1)                       # [B, K-1+L, C]
    out = np.zeros((Bsz, L, C))
    cw = np.asarray(conv_w, np.float64)
    if reset is None:
        for k in range(K):                                       # tap K-1 multiplies the current timestep
            out += full[:, k:k + L, :] * cw[None, None, :, k]
        new_state = full[:, L:, :]
    else:
        # last[b,t] = the latest restart at or before t (far in the past: none): a tap at timestep s < last[b,t] is cut
        rs = np.asarray(reset) != 0
        last = np.where(rs, np.arange(L)[None, :], -(10 ** 9))
        last = np.maximum.accumulate(last, axis=1)
        for k in range(K):
            src = np.arange(L) - (K - 1) + k                     # timestep of tap k at every t (negative: the state)
            live = src[None, :] >= last                          # [B, L]
            out += full[:, k:k + L, :] * cw[None, None, :, k] * live[:, :, None]
        # the state after the window: the last K-1 timesteps, those before the window's last restart zeroed
        tail = np.arange(L - (K - 1), L)
        new_state = full[:, L:, :] * (tail[None, :] >= last[:, -1:])[:, :, None]
    out = silu(out + np.asarray(conv_b, np.float64))
    dt = softplus(zxbcdt[:, :, DI + C:] + np.asarray(dt_bias, np.float64))
    x = out[:, :, :DI].reshape(Bsz, L, H, P)
    Bm = out[:, :, DI:DI + GN].reshape(Bsz, L, G, N)
    Cm = out[:, :, DI + GN:].reshape(Bsz, L, G, N)
    return x, Bm, Cm, dt, new_state


def block_post(y, zxbcdt, norm_w, eps):
    """rmsnorm(y * silu(z)) * norm_w over the H*P channels of a timestep."""
    y = np.asarray(y, np.float64)
    Bsz, L = y.shape[:2]
    DI = y.shape[2] * y.shape[3]
    z = np.asarray(zxbcdt, np.float64)[:, :, :DI]
    v = y.reshape(Bsz, L, DI) * silu(z)
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps) * np.asarray(norm_w, np.float64)


def block_forward(u, p, conv_state=None, ssm_state=None, reset=None):
    """Whole block; p is a dict of float64 parameters (in_proj, conv_w, conv_b, dt_bias, A, D, norm_w, out_proj,
    H, P, N, G, eps).  Returns (out, new conv state, final SSM state)."""
    u = np.asarray(u, np.float64)
    zxbcdt = u @ p["in_proj"].T
    x, Bm, Cm, dt, conv = block_pre(zxbcdt, p["conv_w"], p["conv_b"], p["dt_bias"], p["H"], p["P"], p["N"], p["G"],
                                    conv_state, reset)
    y, final = orc.ssd_sequential(x, dt, p["A"], Bm, Cm, p["D"], ssm_state, reset=reset)
    yn = block_post(y, zxbcdt, p["norm_w"], p["eps"])
    return yn @ p["out_proj"].T, conv, final


# ---------------------------------------------------------------------------------------
# Backward pass of the block (what a trainer's update needs around ssd_chunk_scan_bwd)
# ---------------------------------------------------------------------------------------

def dsilu(v):
    sg = 1.0 / (1.0 + np.exp(-v))
    return sg * (1.0 + v * (1.0 - sg))


def block_post_bwd(y, zxbcdt, norm_w, eps, dout):
    """Gradients of block_post: returns dy [B,L,H,P], dz [B,L,H*P], dnorm_w [H*P].
    With v = y silu(z), r = (mean v^2 + eps)^-1/2, out = v r w and g = dout w:  dv = r g - r^3 v mean(g v)."""
    y = np.asarray(y, np.float64)
    Bsz, L, H, P = y.shape
    DI = H * P
    z = np.asarray(zxbcdt, np.float64)[:, :, :DI]
    w = np.asarray(norm_w, np.float64)
    dout = np.asarray(dout, np.float64)
    v = y.reshape(Bsz, L, DI) * silu(z)
    r = 1.0 / np.sqrt((v * v).mean(-1, keepdims=True) + eps)
    g = dout * w
    dv = r * g - r ** 3 * v * (g * v).mean(-1, keepdims=True)
    dy = (dv * silu(z)).reshape(Bsz, L, H, P)
    dz = dv * y.reshape(Bsz, L, DI) * dsilu(z)
    dnorm_w = (dout * v * r).sum((0, 1))
    return dy, dz, dnorm_w


def block_pre_bwd(zxbcdt, conv_w, conv_b, dt_bias, H, P, N, G, dx, dB, dC, ddt, conv_state=None, reset=None,
                  dconv_state_out=None):
    """Gradients of block_pre with respect to its inputs: returns (dxbc [B,L,C] -- the x | B | C channels of
    dzxbcdt --, ddt_raw [B,L,H], dconv_w [C,K], dconv_b [C], ddt_bias [H], dconv_state [B,K-1,C]).
    dconv_state_out (optional) is a gradient on the conv state the forward returned."""
    zxbcdt = np.asarray(zxbcdt, np.float64)
    Bsz, L, E = zxbcdt.shape
    DI, GN, C, _ = split_widths(H, P, N, G)
    cw = np.asarray(conv_w, np.float64)
    K = cw.shape[1]
    xbc = zxbcdt[:, :, DI:DI + C]
    hist = np.zeros((Bsz, K - 1, C)) if conv_state is None else np.asarray(conv_state, np.float64)
    full = np.concatenate([hist, xbc], 1)
    last = np.full((Bsz, L), -(10 ** 9))
    if reset is not None:
        last = np.maximum.accumulate(np.where(np.asarray(reset) != 0, np.arange(L)[None, :], -(10 ** 9)), axis=1)
    pre = np.zeros((Bsz, L, C))
    live = []
    for k in range(K):
        src = np.arange(L) - (K - 1) + k
        lv = (src[None, :] >= last)[:, :, None]
        live.append(lv)
        pre += full[:, k:k + L, :] * cw[None, None, :, k] * lv
    pre += np.asarray(conv_b, np.float64)
    dout = np.concatenate([np.asarray(dx, np.float64).reshape(Bsz, L, DI), np.asarray(dB, np.float64).reshape(Bsz, L, GN),
                           np.asarray(dC, np.float64).reshape(Bsz, L, GN)], -1)
    dpre = dout * dsilu(pre)
    dfull = np.zeros_like(full)
    dconv_w = np.zeros_like(cw)
    for k in range(K):
        dfull[:, k:k + L, :] += dpre * cw[None, None, :, k] * live[k]
        dconv_w[:, k] = (dpre * full[:, k:k + L, :] * live[k]).sum((0, 1))
    if dconv_state_out is not None:
        # the returned state is the last K-1 rows of `full`, those before the window's last restart zeroed
        tail = np.arange(L - (K - 1), L)
        dfull[:, L:, :] += np.asarray(dconv_state_out, np.float64) * (tail[None, :] >= last[:, -1:])[:, :, None]
    raw = zxbcdt[:, :, DI + C:] + np.asarray(dt_bias, np.float64)
    ddt_raw = np.asarray(ddt, np.float64) / (1.0 + np.exp(-raw))
    return dfull[:, K - 1:, :], ddt_raw, dconv_w, dpre.sum((0, 1)), ddt_raw.sum((0, 1)), dfull[:, :K - 1, :]


def block_backward(u, p, dout, conv_state=None, ssm_state=None, reset=None):
    """Gradients of sum(block_forward(u)[0] * dout) with respect to u and every parameter.  Returns a dict: du,
    din_proj, dconv_w, dconv_b, ddt_bias, dA, dD, dnorm_w, dout_proj."""
    from . import ssd_backward_oracle as sbw
    u = np.asarray(u, np.float64)
    dout = np.asarray(dout, np.float64)
    H, P, N, G = p["H"], p["P"], p["N"], p["G"]
    DI, GN, C, E = split_widths(H, P, N, G)
    zxbcdt = u @ p["in_proj"].T
    x, Bm, Cm, dt, _ = block_pre(zxbcdt, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state, reset)
    y, _ = orc.ssd_sequential(x, dt, p["A"], Bm, Cm, p["D"], ssm_state, reset=reset)
    yn = block_post(y, zxbcdt, p["norm_w"], p["eps"])
    dyn = dout @ p["out_proj"]
    dout_proj = np.einsum("blo,bli->oi", dout, yn)
    dy, dz, dnorm_w = block_post_bwd(y, zxbcdt, p["norm_w"], p["eps"], dyn)
    g = sbw.ssd_backward_sequential(x, dt, p["A"], Bm, Cm, p["D"], ssm_state, dy, reset=reset)
    dxbc, ddt_raw, dconv_w, dconv_b, ddt_bias, _ = block_pre_bwd(zxbcdt, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N,
                                                                 G, g["dx"], g["dB"], g["dC"], g["ddt"], conv_state, reset)
    dzx = np.concatenate([dz, dxbc, ddt_raw], -1)
    return dict(du=dzx @ p["in_proj"], din_proj=np.einsum("ble,bld->ed", dzx, u), dconv_w=dconv_w, dconv_b=dconv_b,
                ddt_bias=ddt_bias, dA=g["dA"], dD=g["dD"], dnorm_w=dnorm_w, dout_proj=dout_proj)
