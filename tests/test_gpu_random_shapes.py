"""Seeded random shapes through the forward -- on whatever kernels the library picks for them -- and the backward
pass, rows against the float64 oracles.  The fixed tests name the shapes the paths were written for; these walk
the space between them (batch sizes either side of the plan's thresholds, ragged lengths, every supported
headdim / dstate / heads-per-group combination, both dtypes, restarts, heavy tails)."""
import numpy as np
import pytest
import torch

from oracle import ssd_backward_oracle as bwd
from oracle import ssd_oracle as orc
from trading_bot_0_amd import SsdError, ssd_chunk_scan, ssd_chunk_scan_backward
from trading_bot_0_amd.synthetic import Workload, make_inputs

from _util import TOL, np64, oracle_scan, rel_err

pytestmark = pytest.mark.gpu


def draw(case):
    rng = np.random.default_rng(1000 + case)
    G = int(rng.choice([1, 2]))
    H = G * int(rng.choice([1, 2, 4, 8]))
    P = int(rng.choice([16, 32, 64]))
    N = int(rng.choice([16, 32, 64, 128]))
    B = int(rng.choice([1, 3, 48, 64, 97, 130, 200]))
    L = int(rng.choice([1, 7, 63, 64, 65, 129, 200, 513, 1000]))
    L = max(1, min(L, int(30e6 // (B * H * P))))
    w = Workload(f"random{case}", B, L, H, P, N, G, int(rng.choice([32, 64, 128, 256])),
                 dtype=str(rng.choice(["bf16", "f32"], p=[0.7, 0.3])), init_std=float(rng.choice([0.0, 0.5])),
                 dt_law=str(rng.choice(["softplus-2", "mixture"])), x_law=str(rng.choice(["normal", "student-t3"])))
    mask = (rng.random((B, L)) < 0.05).astype(np.uint8) if (rng.random() < 0.3 and L > 2) else None
    rows = list(range(B)) if B <= 3 else sorted({0, B - 1, int(rng.integers(0, B))})
    return w, mask, rows, bool(rng.random() < 0.5)


# (case 76: float32, a timestep that decays the state by 2^-64 inside a block of heavy-tailed x -- the shape on which
# separable decay factors across such a block cost float mode 30 ulps on the largest outputs)
@pytest.mark.parametrize("case", list(range(24)) + [76])
def test_random_shape(case):
    w, mask, rows, with_dfinal = draw(case)
    cpu = make_inputs(w, seed=case)
    dev = {k: (None if v is None else v.cuda()) for k, v in cpu.items()}
    sub = {k: (v[rows] if (v is not None and k not in ("A", "D")) else v) for k, v in cpu.items()}
    reset = None if mask is None else torch.from_numpy(mask).cuda()
    tol = TOL[w.torch_dtype]
    try:
        y, fin = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                initial_states=dev["init"], y_dtype=torch.float32 if w.dtype == "bf16" else None,
                                reset=reset)
    except SsdError as e:   # float32 tiles that do not fit the LDS are refused, not mis-computed
        assert e.code == 2 and w.dtype == "f32", str(e)
        return
    torch.cuda.synchronize()
    if mask is None:
        y_ref, f_ref = oracle_scan(sub)
    else:
        y_ref, f_ref = orc.ssd_sequential(np64(sub["x"]), np64(sub["dt"]), np64(sub["A"]), np64(sub["B"]), np64(sub["C"]),
                                          np64(sub["D"]), np64(sub["init"]), reset=mask[rows])
    assert rel_err(y[rows], y_ref) <= tol and rel_err(fin[rows], f_ref) <= tol, f"{w}"
    g = torch.Generator().manual_seed(case + 1000)
    dy = torch.randn(cpu["x"].shape, generator=g).to(w.torch_dtype)
    dfin = torch.randn(w.batch, w.nheads, w.headdim, w.dstate, generator=g) if with_dfinal else None
    try:
        got = ssd_chunk_scan_backward(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], dy.cuda(), chunk=w.chunk,
                                      initial_states=dev["init"], dfinal_states=None if dfin is None else dfin.cuda(),
                                      need_dinitial_states=True, reset=reset)
    except SsdError as e:   # as for the forward: float32 tiles of the largest head sizes do not fit the LDS
        assert e.code == 2 and w.dtype == "f32", str(e)
        return
    torch.cuda.synchronize()
    ref = bwd.ssd_backward_sequential(np64(sub["x"]), np64(sub["dt"]), np64(sub["A"]), np64(sub["B"]), np64(sub["C"]),
                                      np64(sub["D"]), np64(sub["init"]), np64(dy[rows]),
                                      np64(None if dfin is None else dfin[rows]), reset=None if mask is None else mask[rows])
    for k_out, k_ref in (("dx", "dx"), ("ddt", "ddt"), ("dB", "dB"), ("dC", "dC"), ("dinitial_states", "dinit")):
        o = got[k_out][rows].detach().float().cpu().numpy().astype(np.float64)
        r = ref[k_ref]
        allowed = tol * (np.sqrt((r ** 2).mean()) + 1e-300)
        if got[k_out].dtype == torch.bfloat16:   # plus the one rounding the output format costs
            allowed = allowed + 2.0 ** -8 * np.abs(r)
        worst = (np.abs(o - r) / allowed).max()
        assert np.isfinite(worst) and worst <= 1.0, f"{w} {k_out}: {worst:.3g} x the allowance"
