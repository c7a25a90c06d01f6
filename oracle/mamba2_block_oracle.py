"""CPU restatement (numpy float64) of the Mamba-2 block stages around the SSD scan.  Test infrastructure
only: imported by tests/ to check the HIP kernels of trading_bot_0_amd/csrc/ssd_block_kernels.hip and the
block assembly of trading_bot_0_amd/block.py.  The reference tree holds no source for this layer (its slot is
trading_bots/src/torch/model/trading_model.rs:589-606); the arithmetic is the published Mamba-2 block:
causal depthwise conv + SiLU on (x, B, C), softplus(dt + bias), SSD, RMSNorm of y*silu(z), two projections.
Every function here is pinned in tests/test_oracle_block.py against library routines or direct formulas."""
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
