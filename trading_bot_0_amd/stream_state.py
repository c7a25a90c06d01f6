"""Streaming state of the SSD encoder: the recurrent memory carried between per-bar calls.

Plays the role the reference's `StreamState` plays for its encoder
(`trading_bots/src/torch/model/trading_model.rs:56-75`; lifecycle reset / detach / build in
`trading_bots/src/torch/model/stream/state.rs:10-21,23-30,52-110`; prefix initialisation then
per-bar step in `trading_bots/src/torch/model/stream/live.rs:257-360`).  Where the reference
keeps a layout ring and recomputes its attention trunk each bar, an SSD encoder keeps one
fp32 tensor [batch, nheads, headdim, dstate] per layer, owned by the caller, zero on reset.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import ssd


@dataclass
class SsdStreamState:
    state: torch.Tensor          # [batch, nheads, headdim, dstate] float32, advanced in place
    initialized: bool = False    # True once a prefix scan (or an explicit state) seeded it

    @classmethod
    def build(cls, batch: int, nheads: int, headdim: int, dstate: int, device="cuda") -> "SsdStreamState":
        """Zero state for `batch` independent streams (cf. build_stream_state, state.rs:52-110)."""
        return cls(torch.zeros((batch, nheads, headdim, dstate), dtype=torch.float32, device=device), False)

    @property
    def batch(self) -> int:
        return self.state.shape[0]

    def reset(self) -> None:
        """Forget everything (cf. StreamState::reset, state.rs:10-21)."""
        self.state.zero_()
        self.initialized = False

    def reset_rows(self, rows: torch.Tensor) -> None:
        """Zero the streams whose environment restarted: `rows` is an int64 index tensor or a bool
        mask over the batch (the rollout resets a subset of envs between steps,
        trading_bots/src/torch/train/rollout.rs:130-135,209-235)."""
        if rows.dtype == torch.bool:
            self.state.mul_((~rows).to(self.state.dtype).view(-1, 1, 1, 1))
        else:
            self.state.index_fill_(0, rows, 0.0)

    def detach(self) -> "SsdStreamState":
        """Cut the state from any autograd history (cf. detach_stream_state, state.rs:23-30)."""
        self.state = self.state.detach()
        return self

    def clone(self) -> "SsdStreamState":
        return SsdStreamState(self.state.clone(), self.initialized)

    def init_from_prefix(self, x, dt, A, Bm, Cm, D=None, chunk: int = 128, workspace=None,
                         y_dtype=None) -> torch.Tensor:
        """Scan a full prefix [B,L,...] and keep its final state (cf. init_from_full_on_device,
        live.rs:322-360).  Continues from the current state when already initialised.  Returns y."""
        if x.shape[0] != self.batch:
            raise ValueError(f"stream state batch size mismatch: state has {self.batch}, input has {x.shape[0]}")
        init = self.state if self.initialized else None
        y, _ = ssd.ssd_chunk_scan(x, dt, A, Bm, Cm, D, chunk=chunk, initial_states=init,
                                  workspace=workspace, final_out=self.state, y_dtype=y_dtype)
        self.initialized = True
        return y

    def step(self, x, dt, A, Bm, Cm, D=None, out: Optional[torch.Tensor] = None, y_dtype=None) -> torch.Tensor:
        """Advance every stream by one timestep (cf. step_uniform_stream_state_on_device,
        live.rs:228-244).  x [B,H,P], dt [B,H], Bm/Cm [B,G,N]; returns y [B,H,P]."""
        if x.shape[0] != self.batch:
            raise ValueError(f"stream state batch size mismatch: state has {self.batch}, input has {x.shape[0]}")
        y = ssd.ssd_step(self.state, x, dt, A, Bm, Cm, D, out=out, y_dtype=y_dtype)
        self.initialized = True
        return y

    def steps(self, x, dt, A, Bm, Cm, D=None, reset: Optional[torch.Tensor] = None,
              out: Optional[torch.Tensor] = None, y_dtype=None) -> torch.Tensor:
        """Advance every stream by T timesteps in one launch, the state staying on chip between them.
        x [B,T,H,P], dt [B,T,H], Bm/Cm [B,T,G,N]; `reset` [B,T] (bool or uint8) zeroes a stream right
        before the marked step, which is the rollout's advance -> reset slots -> forward
        (trading_bots/src/torch/train/rollout.rs:130-135,209-235) without a separate pass over the
        state.  Returns y [B,T,H,P]."""
        if x.shape[0] != self.batch:
            raise ValueError(f"stream state batch size mismatch: state has {self.batch}, input has {x.shape[0]}")
        y = ssd.ssd_steps(self.state, x, dt, A, Bm, Cm, D, reset=reset, out=out, y_dtype=y_dtype)
        self.initialized = True
        return y
