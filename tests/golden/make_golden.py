"""Writes tests/golden/plumbing_f32_seed0.npz: the seed-0 inputs of the plumbing workload
(batch 4, seqlen 256, 4 heads, headdim 16, dstate 16, one group, chunk 64, float32) together
with the oracle's outputs and every stage intermediate, computed in float64.

The reference tree holds no vectors for the SSD path, so these come from this repository's own
oracle (oracle/ssd_oracle.py), which tests/test_oracle.py pins against closed forms and
library routines.  Run from the repository root:  python tests/golden/make_golden.py
"""
import sys
from pathlib import Path

import numpy as np

REPO = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(REPO))

from oracle import ssd_oracle as orc  # noqa: E402
from trading_bot_0_amd.synthetic import WORKLOADS, make_inputs  # noqa: E402


def main():
    w = WORKLOADS["plumbing_f32"]
    inp = make_inputs(w, seed=0, device="cpu")
    x, dt, A, Bm, Cm, D = (inp[k].numpy() for k in ("x", "dt", "A", "B", "C", "D"))
    y, final, mid = orc.ssd_chunked(x, dt, A, Bm, Cm, D, None, chunk=w.chunk, return_intermediates=True)
    ys, fs = orc.ssd_sequential(x, dt, A, Bm, Cm, D, None)
    assert orc.rel_err(y, ys) < 1e-12 and orc.rel_err(final, fs) < 1e-12
    out = Path(__file__).with_name("plumbing_f32_seed0.npz")
    np.savez(out, x=x, dt=dt, A=A, B=Bm, C=Cm, D=D, y=ys, final=fs,
             dA_cs=mid["dA_cs"].astype(np.float32), dt_c=mid["dt_c"].astype(np.float32),
             S=mid["S"].astype(np.float32), prev=mid["prev"].astype(np.float32))
    print(out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
