"""Pins of oracle/ssd_backward_oracle.py (CPU only).  The sequential adjoint is checked against central
differences of the forward oracle for every input, with and without D, an initial state, a gradient on the
final state and grouped B/C; the role-swapped decomposition the GPU path uses is checked against the adjoint."""
import numpy as np
import pytest

from oracle import ssd_oracle as orc
from oracle import ssd_backward_oracle as bwd


def _case(seed, Bsz=2, L=7, H=4, P=3, N=5, G=2, with_D=True, with_init=True):
    r = np.random.default_rng(seed)
    x = r.standard_normal((Bsz, L, H, P))
    dt = np.log1p(np.exp(r.standard_normal((Bsz, L, H)) - 1.0))
    A = -np.exp(r.uniform(0.0, np.log(8.0), H))
    Bm = r.standard_normal((Bsz, L, G, N)) / np.sqrt(N)
    Cm = r.standard_normal((Bsz, L, G, N)) / np.sqrt(N)
    D = r.standard_normal(H) if with_D else None
    init = 0.3 * r.standard_normal((Bsz, H, P, N)) if with_init else None
    dy = r.standard_normal((Bsz, L, H, P))
    dfinal = r.standard_normal((Bsz, H, P, N))
    return x, dt, A, Bm, Cm, D, init, dy, dfinal


RESET = None


def _loss(x, dt, A, Bm, Cm, D, init, dy, dfinal):
    y, fin = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init, reset=RESET)
    return (y * dy).sum() + (0.0 if dfinal is None else (fin * dfinal).sum())


def _numeric(args, idx, eps=1e-6):
    base = [None if a is None else np.array(a, np.float64) for a in args]
    g = np.zeros_like(base[idx])
    it = np.nditer(base[idx], flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        keep = base[idx][i]
        base[idx][i] = keep + eps
        up = _loss(*base)
        base[idx][i] = keep - eps
        dn = _loss(*base)
        base[idx][i] = keep
        g[i] = (up - dn) / (2 * eps)
    return g


@pytest.mark.parametrize("with_D,with_init,with_dfinal,G", [(True, True, True, 2), (False, False, False, 1),
                                                            (True, False, True, 4), (False, True, False, 2)])
def test_adjoint_matches_central_differences(with_D, with_init, with_dfinal, G):
    args = list(_case(3, G=G, with_D=with_D, with_init=with_init))
    if not with_dfinal:
        args[8] = None
    got = bwd.ssd_backward_sequential(*args)
    names = {0: "dx", 1: "ddt", 2: "dA", 3: "dB", 4: "dC"}
    if with_D:
        names[5] = "dD"
    if with_init:
        names[6] = "dinit"
    for idx, name in names.items():
        num = _numeric(args, idx)
        scale = max(1.0, np.abs(num).max())
        assert np.abs(got[name] - num).max() < 2e-7 * scale, name
    if not with_D:
        assert got["dD"] is None


def test_dinit_without_initial_state_is_still_the_gradient_at_zero():
    args = list(_case(5, with_init=False))
    got = bwd.ssd_backward_sequential(*args)
    Bsz, L, H, P = args[0].shape
    N = args[3].shape[3]
    args[6] = np.zeros((Bsz, H, P, N))
    num = _numeric(args, 6)
    assert np.abs(got["dinit"] - num).max() < 2e-7 * max(1.0, np.abs(num).max())


@pytest.mark.parametrize("seed,L,G,with_D,with_init,with_dfinal", [(0, 9, 1, True, True, True), (1, 33, 2, False, False, True),
                                                                   (2, 20, 4, True, True, False), (4, 1, 2, True, False, False)])
def test_role_swapped_scans_equal_the_adjoint(seed, L, G, with_D, with_init, with_dfinal):
    x, dt, A, Bm, Cm, D, init, dy, dfinal = _case(seed, L=L, G=G, with_D=with_D, with_init=with_init)
    if not with_dfinal:
        dfinal = None
    _, fin = orc.ssd_sequential(x, dt, A, Bm, Cm, D, init)
    ref = bwd.ssd_backward_sequential(x, dt, A, Bm, Cm, D, init, dy, dfinal)
    got = bwd.ssd_backward_by_scans(x, dt, A, Bm, Cm, D, init, dy, dfinal, fin)
    for k, v in ref.items():
        if k.endswith("_scale"):
            continue
        if v is None:
            assert got[k] is None
        else:
            assert np.abs(got[k] - v).max() < 1e-11 * max(1.0, np.abs(v).max()), k


def test_general_scan_is_the_forward_for_its_own_decays():
    x, dt, A, Bm, Cm, D, init, dy, dfinal = _case(7, G=4)           # G = H: per-head B, C
    y, fin = orc.ssd_sequential(x, dt, A, Bm, Cm, None, init)
    y2, fin2 = bwd.scan_general(x, dt * A[None, None, :], dt, Bm, Cm, init)
    assert np.abs(y - y2).max() < 1e-13 and np.abs(fin - fin2).max() < 1e-13


def test_adjoint_with_restarts_matches_central_differences():
    global RESET
    args = list(_case(11, L=9, G=2))
    RESET = np.zeros((2, 9), np.uint8)
    RESET[0, 4] = 1
    RESET[1, 0] = 1
    RESET[1, 8] = 1
    try:
        got = bwd.ssd_backward_sequential(*args, reset=RESET)
        for idx, name in {0: "dx", 1: "ddt", 2: "dA", 3: "dB", 4: "dC", 5: "dD", 6: "dinit"}.items():
            num = _numeric(args, idx)
            assert np.abs(got[name] - num).max() < 2e-7 * max(1.0, np.abs(num).max()), name
        assert np.abs(got["dinit"][1]).max() == 0.0
    finally:
        RESET = None
