"""Seeded synthetic inputs for the five benchmark workloads of the SSD path.

Each workload fixes shapes and input laws; there is no dataset behind the SSD op (the reference
feeds it price-delta features from its CPU environment, `trading_bots/src/torch/env/vec/step.rs:421-445`).
Draw order is always x, dt_raw, A, B, C, D, init, from one torch.Generator seeded with `seed`,
on the device the tensors are wanted on.  In bf16 mode values are drawn in fp32 and rounded to
bf16 once; whoever checks results must consume the rounded values.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Dict, Optional

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    batch: int
    seqlen: int
    nheads: int
    headdim: int
    dstate: int
    ngroups: int
    chunk: int
    dtype: str = "bf16"                 # "bf16" or "f32"
    a_log_range: tuple = (1.0, 16.0)    # A = -exp(U(ln lo, ln hi))
    dt_law: str = "softplus-2"          # "softplus-2" | "per-head-bias" | "mixture"
    x_law: str = "normal"               # "normal" | "student-t3"
    init_std: float = 0.0               # 0 -> no initial state
    stream_steps: int = 0               # single-timestep updates after the prefix scan

    def with_batch(self, batch: int) -> "Workload":
        return replace(self, batch=batch)

    def with_dtype(self, dtype: str) -> "Workload":
        return replace(self, dtype=dtype)

    @property
    def torch_dtype(self) -> torch.dtype:
        return torch.bfloat16 if self.dtype == "bf16" else torch.float32

    @property
    def nchunks(self) -> int:
        return -(-self.seqlen // self.chunk)

    @property
    def units(self) -> int:
        """timestep*batch units of one forward."""
        return self.batch * self.seqlen


WORKLOADS: Dict[str, Workload] = {
    "plumbing_f32": Workload("plumbing_f32", 4, 256, 4, 16, 16, 1, 64, dtype="f32"),
    "policy_bf16": Workload("policy_bf16", 256, 2048, 8, 32, 64, 1, 128),
    "long_lookback_bf16": Workload("long_lookback_bf16", 32, 16384, 16, 64, 128, 2, 256,
                                   dt_law="per-head-bias", init_std=0.1),
    "decay_extreme": Workload("decay_extreme", 64, 4096, 8, 32, 64, 1, 128, a_log_range=(0.01, 64.0),
                              dt_law="mixture", x_law="student-t3"),
    "streamed_bf16": Workload("streamed_bf16", 4096, 2048, 8, 32, 64, 1, 128, stream_steps=64),
}


def _softplus(t: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.softplus(t)


def make_inputs(w: Workload, seed: int = 0, device="cpu", seqlen: Optional[int] = None) -> dict:
    """Returns dict(x, dt, A, B, C, D, init) for workload `w` (init is None when init_std == 0).
    `seqlen` overrides w.seqlen (the streamed workload draws seqlen + stream_steps at once)."""
    L = w.seqlen if seqlen is None else seqlen
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    f32 = dict(dtype=torch.float32, device=device)
    Bsz, H, P, N, G = w.batch, w.nheads, w.headdim, w.dstate, w.ngroups

    def randn(*shape):
        return torch.randn(*shape, generator=g, **f32)

    def rand(*shape):
        return torch.rand(*shape, generator=g, **f32)

    if w.x_law == "normal":
        x = randn(Bsz, L, H, P)
    else:  # Student-t, 3 degrees of freedom: z / sqrt(chi2_3 / 3)
        z = randn(Bsz, L, H, P)
        chi2 = randn(Bsz, L, H, P).square_()
        chi2 += randn(Bsz, L, H, P).square_()
        chi2 += randn(Bsz, L, H, P).square_()
        x = z / torch.sqrt(chi2 / 3.0)
        del z, chi2
    if w.dt_law == "softplus-2":
        dt = _softplus(randn(Bsz, L, H) - 2.0)
    elif w.dt_law == "per-head-bias":
        bias = rand(H) * -4.0
        dt = _softplus(randn(Bsz, L, H) + bias)
    else:  # 90 % near-unity decay, 10 % near-total decay
        small = _softplus(randn(Bsz, L, H) - 4.0)
        large = _softplus(randn(Bsz, L, H) + 3.0)
        dt = torch.where(rand(Bsz, L, H) < 0.9, small, large)
    lo, hi = math.log(w.a_log_range[0]), math.log(w.a_log_range[1])
    A = -torch.exp(rand(H) * (hi - lo) + lo)
    Bm = randn(Bsz, L, G, N) / math.sqrt(N)
    Cm = randn(Bsz, L, G, N) / math.sqrt(N)
    D = randn(H)
    init = randn(Bsz, H, P, N) * w.init_std if w.init_std > 0 else None
    td = w.torch_dtype
    return dict(x=x.to(td), dt=dt.to(td), A=A, B=Bm.to(td), C=Cm.to(td), D=D, init=init)


def algorithmic_bytes_fwd(w: Workload) -> int:
    """Compulsory HBM traffic of one forward: every input read once, every output written once."""
    e = 2 if w.dtype == "bf16" else 4
    Bsz, L, H, P, N, G = w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups
    has_init = 1 if w.init_std > 0 else 0
    return e * (2 * Bsz * L * H * P + Bsz * L * H + 2 * Bsz * L * G * N) + 4 * Bsz * H * P * N * (1 + has_init) + 8 * H


def stage_bytes(w: Workload) -> dict:
    """Algorithmic bytes of each stage run as its own kernel with float32 intermediates."""
    e = 2 if w.dtype == "bf16" else 4
    Bsz, L, H, P, N, G, nc = w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.nchunks
    has_init = 1 if w.init_std > 0 else 0
    blh, st = Bsz * L * H, Bsz * nc * H * P * N
    return {
        "chunk_cumsum": (e + 8) * blh,
        "chunk_state": e * (blh * P + Bsz * L * G * N) + 8 * blh + 4 * st,
        "state_passing": 8 * st + 4 * Bsz * H * nc + 4 * Bsz * H * P * N * (1 + has_init),
        # stages 2+3 in one pass: stage 2's traffic (the chunk-state buffer is written once, with the state
        # entering each chunk) plus the chunk decays and the initial / final states
        "chunk_state_passing": e * (blh * P + Bsz * L * G * N) + 8 * blh + 4 * st + 4 * Bsz * H * nc
                               + 4 * Bsz * H * P * N * (1 + has_init),
        "chunk_scan": e * (2 * blh * P + 2 * Bsz * L * G * N) + 8 * blh + 4 * st,
    }


def stage_flops(w: Workload) -> dict:
    """Dense MFMA flops of stages 2 and 4."""
    Bsz, L, H, P, N, G, Q = w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk
    return {
        "chunk_state": 2 * Bsz * L * H * N * P,
        "chunk_state_passing": 2 * Bsz * L * H * N * P,
        "chunk_scan": 2 * Bsz * L * (G * Q * N + H * Q * P + H * N * P),
    }


def step_bytes(w: Workload) -> int:
    e = 2 if w.dtype == "bf16" else 4
    Bsz, H, P, N, G = w.batch, w.nheads, w.headdim, w.dstate, w.ngroups
    return 8 * Bsz * H * P * N + e * (2 * Bsz * H * P + Bsz * H + 2 * Bsz * G * N)
