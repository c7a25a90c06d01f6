"""The SSD chunk-scan forward restated with torch CPU tensor ops (ATen CPU, float32): the CPU baseline that
bench.py times next to the GPU numbers.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/ and bench.py's `cpu_baseline` leg import it.

Why this form: the reference has no SSD source left to time (its slot is
`trading_bots/src/torch/model/trading_model.rs:589-606`), but whatever ran there ran on the backend the reference
uses on a CPU device -- ATen CPU in float32 (`trading_bots/src/torch/model/trading_model.rs:140-146`) with the
thread policy the trainer sets, one intra-op thread by default (`trading_bots/src/torch/train/trainer.rs:635-646`).
This file is the four-stage chunked algorithm (per-chunk cumsum, einsum chunk states, sequential state passing,
masked intra-chunk product) in those ops.  It is pinned against the float64 numpy oracle
(tests/test_oracle.py::test_torch_cpu_restatement_matches_the_oracle), which is itself pinned by closed forms.
"""
from __future__ import annotations

import torch


def ssd_chunked_torch(x, dt, A, Bm, Cm, D=None, init=None, chunk=128):
    """x [B,L,H,P], dt [B,L,H], A [H], Bm, Cm [B,L,G,N], D [H] or None, init [B,H,P,N] or None; any float dtype,
    CPU.  Returns (y [B,L,H,P], final [B,H,P,N])."""
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    Q = chunk
    nc = -(-L // Q)
    pad = nc * Q - L
    if pad:
        x = torch.nn.functional.pad(x, (0, 0, 0, 0, 0, pad))
        dt = torch.nn.functional.pad(dt, (0, 0, 0, pad))
        Bm = torch.nn.functional.pad(Bm, (0, 0, 0, 0, 0, pad))
        Cm = torch.nn.functional.pad(Cm, (0, 0, 0, 0, 0, pad))
    rep = H // G
    xc = x.reshape(Bsz, nc, Q, H, P)
    Bc = Bm.reshape(Bsz, nc, Q, G, N)
    Cc = Cm.reshape(Bsz, nc, Q, G, N)
    dtc = dt.reshape(Bsz, nc, Q, H).permute(0, 3, 1, 2)                  # [B,H,nc,Q]
    # stage 1
    cs = torch.cumsum(dtc * A.view(1, H, 1, 1), dim=-1)                  # [B,H,nc,Q]
    # stage 2: S[b,c,h,p,n] = sum_l w[l] x[l,p] B[l,n]
    w = torch.exp(cs[..., -1:] - cs) * dtc                               # [B,H,nc,Q]
    xw = xc * w.permute(0, 2, 3, 1).unsqueeze(-1)                        # [B,nc,Q,H,P]
    S = torch.einsum("bclgrp,bclgn->bcgrpn", xw.reshape(Bsz, nc, Q, G, rep, P), Bc).reshape(Bsz, nc, H, P, N)
    # stage 3
    decay = torch.exp(cs[..., -1])                                       # [B,H,nc]
    h = torch.zeros(Bsz, H, P, N, dtype=x.dtype) if init is None else init.to(x.dtype).clone()
    prev = torch.empty_like(S)
    for c in range(nc):
        prev[:, c] = h
        h = decay[:, :, c, None, None] * h + S[:, c]
    # stage 4
    CB = torch.einsum("bclgn,bcsgn->bcgls", Cc, Bc)                      # [B,nc,G,Q,Q]
    diff = cs.unsqueeze(-1) - cs.unsqueeze(-2)                           # [B,H,nc,l,s]
    mask = torch.ones(Q, Q, dtype=torch.bool).tril()
    lam = torch.exp(diff.masked_fill(~mask, float("-inf")))              # masked before exp
    M = lam * dtc.unsqueeze(-2)                                          # [B,H,nc,l,s]
    M = M.reshape(Bsz, G, rep, nc, Q, Q) * CB.permute(0, 2, 1, 3, 4).unsqueeze(2)
    y = torch.einsum("bgrcls,bcsgrp->bclgrp", M, xc.reshape(Bsz, nc, Q, G, rep, P))
    y = y + torch.einsum("bgrcl,bclgn,bcgrpn->bclgrp", torch.exp(cs).reshape(Bsz, G, rep, nc, Q), Cc,
                         prev.reshape(Bsz, nc, G, rep, P, N))
    y = y.reshape(Bsz, nc * Q, H, P)
    if D is not None:
        y = y + D.view(1, 1, H, 1) * x
    return y[:, :L], h
