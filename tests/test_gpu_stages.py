"""Each HIP stage on its own against the oracle's intermediates (through the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import ssd_oracle as orc
from trading_bot_0_amd import ssd
from trading_bot_0_amd.synthetic import Workload, make_inputs

from _util import LOG2E, TOL, assert_close, check_y, np64, rel_err, to_dev

pytestmark = pytest.mark.gpu

DT = {"f32": torch.float32, "bf16": torch.bfloat16}

# (batch, seqlen, H, P, N, G, Q) -- plumbing, policy, long-lookback tiles; a ragged tail; small tiles
SHAPES = [
    (2, 256, 4, 16, 16, 1, 64),
    (2, 512, 8, 32, 64, 1, 128),
    (1, 768, 4, 64, 128, 2, 256),
    (3, 200, 6, 8, 32, 3, 32),
    (2, 2112, 8, 32, 64, 1, 128),
    (1, 300, 2, 48, 16, 2, 64),
]


def build(shape, dtype, seed=0, init_std=0.0):
    Bsz, L, H, P, N, G, Q = shape
    w = Workload("t", Bsz, L, H, P, N, G, Q, dtype=dtype, init_std=init_std)
    cpu = make_inputs(w, seed=seed)
    mids = {}
    o = {k: np64(v) for k, v in cpu.items()}
    mids["dA_cs"], mids["dt_c"] = orc.chunk_cumsum(o["dt"], o["A"], Q)
    mids["S"] = orc.chunk_state(o["x"], o["B"], mids["dA_cs"], mids["dt_c"])
    mids["prev"], mids["final"] = orc.state_passing(mids["S"], mids["dA_cs"][..., -1], o["init"])
    mids["y"] = orc.chunk_scan(o["x"], o["B"], o["C"], mids["dA_cs"], mids["dt_c"], mids["prev"], o["D"])
    return w, to_dev(cpu), o, mids


def skip_if_unsupported(shape, dtype):
    """float32 tiles of headdim 64 / dstate 128 / chunk 256 exceed the 160 KiB LDS: the library
    rejects them (tests/test_abi.py checks the error), so there is nothing to compare."""
    if dtype == "f32" and shape[3:5] == (64, 128) and shape[6] == 256:
        pytest.skip("float32 headdim 64 / dstate 128 / chunk 256 does not fit LDS; rejected by the library")


def f32dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def dtcs_dev(mids):
    """The oracle's float64 cumulative sum and dt in the stage-1 output layout [B,H,nc,4,Q]:
    log2(e) * cumsum as an unevaluated float32 pair hi + lo, dt, and the stage-2 weight."""
    al = mids["dA_cs"] * LOG2E
    hi = al.astype(np.float32)
    lo = (al - hi.astype(np.float64)).astype(np.float32)
    w = np.exp(mids["dA_cs"][..., -1:] - mids["dA_cs"]) * mids["dt_c"]
    return f32dev(np.stack([hi, lo, mids["dt_c"].astype(np.float32), w.astype(np.float32)], axis=3))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_chunk_cumsum(shape, dtype):
    w, dev, o, mids = build(shape, dtype)
    dtcs = ssd.chunk_cumsum(dev["dt"], dev["A"], w.chunk)
    torch.cuda.synchronize()
    got = dtcs.cpu().numpy().astype(np.float64)
    hi, lo, d32 = got[:, :, :, 0], got[:, :, :, 1], got[:, :, :, 2]
    # float64 scan split into two floats: the pair carries ~48 bits, hi alone is the rounded sum
    al = mids["dA_cs"] * LOG2E
    assert np.max(np.abs((hi + lo) - al)) <= 1e-11 * max(1.0, np.max(np.abs(al)))
    assert np.max(np.abs(hi - al)) <= 2.0 ** -23 * max(1.0, np.max(np.abs(al)))   # hi alone: a rounded float
    assert np.array_equal(d32, mids["dt_c"]), "dt row is an exact copy"
    w = np.exp(mids["dA_cs"][..., -1:] - mids["dA_cs"]) * mids["dt_c"]
    assert np.max(np.abs(got[:, :, :, 3] - w)) <= 1e-6 * np.max(w), "stage-2 weight row"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_chunk_state(shape, dtype):
    skip_if_unsupported(shape, dtype)
    w, dev, o, mids = build(shape, dtype)
    S = ssd.chunk_state(dev["x"], dev["B"], dtcs_dev(mids))
    torch.cuda.synchronize()
    assert_close(S, mids["S"], DT[dtype], "chunk states")


@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("with_init", [False, True])
@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[1], SHAPES[4], (2, 352, 4, 16, 32, 1, 32), (1, 96, 2, 8, 16, 1, 32)])
def test_state_passing(shape, with_init, in_place):
    w, dev, o, mids = build(shape, "f32", init_std=0.5 if with_init else 0.0)
    S = f32dev(mids["S"])
    prev, final = ssd.state_passing(S, dtcs_dev(mids), dev["init"], in_place=in_place)
    torch.cuda.synchronize()
    if in_place:
        assert prev.data_ptr() == S.data_ptr()
    assert_close(prev, mids["prev"], torch.float32, "prev states")
    assert_close(final, mids["final"], torch.float32, "final states")


@pytest.mark.parametrize("with_init", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES + [(40, 384, 16, 32, 64, 2, 128)])
def test_chunk_state_passing_fused(shape, dtype, with_init):
    """Stages 2+3 in one pass: states entering each chunk and the final state, against the oracle and
    against the two separate stages."""
    skip_if_unsupported(shape, dtype)
    w, dev, o, mids = build(shape, dtype, init_std=0.5 if with_init else 0.0)
    dtcs = dtcs_dev(mids)
    prev, final = ssd.chunk_state_passing(dev["x"], dev["B"], dtcs, dev["init"])
    torch.cuda.synchronize()
    assert_close(prev, mids["prev"], DT[dtype], "fused prev states")
    assert_close(final, mids["final"], DT[dtype], "fused final states")
    prev2, final2 = ssd.state_passing(ssd.chunk_state(dev["x"], dev["B"], dtcs), dtcs, dev["init"])
    assert rel_err(prev, np64(prev2)) <= 1e-5 and rel_err(final, np64(final2)) <= 1e-5
    if with_init:   # the final state may be written over the initial one
        buf = dev["init"].clone()
        lib = ssd.load_library()
        from ctypes import byref
        dims = ssd.SsdDims(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk)
        rc = lib.ssd_chunk_state_passing_fwd(byref(dims), 1 if dtype == "bf16" else 0, dev["x"].data_ptr(),
                                             dev["B"].data_ptr(), dtcs.data_ptr(), buf.data_ptr(), prev2.data_ptr(),
                                             buf.data_ptr(), None)
        assert rc == 0, ssd.last_error(lib)
        torch.cuda.synchronize()
        assert torch.equal(buf, final) and torch.equal(prev2, prev)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_chunk_scan_stage(shape, dtype):
    skip_if_unsupported(shape, dtype)
    w, dev, o, mids = build(shape, dtype, init_std=0.3)
    dtcs, prev = dtcs_dev(mids), f32dev(mids["prev"])
    call = lambda D: (lambda yd: ssd.chunk_scan_stage(dev["x"], dev["B"], dev["C"], dtcs, prev, D, y_dtype=yd))
    _, e = check_y(call(dev["D"]), mids["y"], DT[dtype], "y")
    if dtype == "bf16":   # hi/lo operands leave the arithmetic an order of magnitude inside the bar
        assert e <= 2e-3
    ref0 = mids["y"] - o["D"][None, None, :, None] * o["x"]
    check_y(call(None), ref0, DT[dtype], "y without D")


def test_chunk_scan_stage_special_cases():
    """B = 0 leaves only the readout of the entering state plus D x; zero entering state and
    D = None leave only the masked intra-chunk product."""
    shape = (2, 256, 4, 32, 64, 1, 128)
    w, dev, o, mids = build(shape, "f32", init_std=0.3)
    dtcs, prev = dtcs_dev(mids), f32dev(mids["prev"])
    y = ssd.chunk_scan_stage(dev["x"], torch.zeros_like(dev["B"]), dev["C"], dtcs, prev, dev["D"])
    Cc = o["C"].reshape(2, 2, 128, 1, 64)[:, :, :, 0]
    ref = np.einsum("bhcl,bcln,bchpn->bclhp", np.exp(mids["dA_cs"]), Cc, mids["prev"]).reshape(2, 256, 4, 32)
    ref += o["D"][None, None, :, None] * o["x"]
    assert_close(y, ref, torch.float32, "readout only")
    y = ssd.chunk_scan_stage(dev["x"], dev["B"], dev["C"], dtcs, torch.zeros_like(prev), None)
    ref = orc.chunk_scan(o["x"], o["B"], o["C"], mids["dA_cs"], mids["dt_c"], np.zeros_like(mids["prev"]), None)
    assert_close(y, ref, torch.float32, "intra-chunk only")
