"""The one-pass forward (one kernel, running state in registers) through the C ABI against the float64
oracle: the shapes that pick each of its template instances, ragged tails, initial states, strong decay
(the exact diagonal path), and agreement with the staged kernels."""
import numpy as np
import pytest
import torch

from oracle import ssd_oracle as orc
from trading_bot_0_amd import SsdError, ssd_chunk_scan, ssd_chunk_scan_onepass
from trading_bot_0_amd.synthetic import WORKLOADS, Workload, make_inputs

from _util import assert_close, assert_stored_bf16_close, check_y, np64, oracle_scan, rel_err, to_dev

pytestmark = pytest.mark.gpu


def run(dev, chunk, **kw):
    y, final = ssd_chunk_scan_onepass(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=chunk,
                                      initial_states=dev["init"], **kw)
    torch.cuda.synchronize()
    return y, final


def check(w, seed=0, seqlen=None, drop_D=False):
    cpu = make_inputs(w, seed=seed, seqlen=seqlen)
    if drop_D:
        cpu["D"] = None
    dev = to_dev(cpu)
    yr, fr = oracle_scan(cpu, with_D=not drop_D)
    finals = []

    def call(yd):
        y, f = run(dev, w.chunk, y_dtype=yd)
        finals.append(f)
        return y

    y, ey = check_y(call, yr, w.torch_dtype, f"{w.name} y")
    assert all(torch.equal(f, finals[0]) for f in finals)
    ef = assert_close(finals[0], fr, w.torch_dtype, f"{w.name} final")
    print(f"one-pass {w.name} B={w.batch} L={seqlen or w.seqlen} H={w.nheads} P={w.headdim} N={w.dstate} "
          f"G={w.ngroups} Q={w.chunk}: err_y={ey:.2e} err_final={ef:.2e}")
    return dev, y, finals[0]


SHAPES = {
    # name: (batch, seqlen, nheads, headdim, dstate, ngroups, chunk)  -> instance picked
    "policy": (2, 1024, 8, 32, 64, 1, 128),          # N=64, 8 waves
    "two_groups": (2, 512, 8, 32, 64, 2, 128),       # 4 units per group: 4 waves
    "wide_head": (2, 512, 4, 64, 64, 1, 128),        # two 32-column units per head
    "small_state": (2, 512, 8, 32, 32, 1, 128),      # N=32
    "short_chunk": (2, 512, 8, 32, 64, 1, 64),
    "small_state_short_chunk": (3, 256, 4, 32, 32, 1, 64),   # N=32, 4 waves
    "many_units": (1, 384, 16, 64, 64, 2, 128),      # 16 units per group: two workgroups per (batch, group)
    "wide_state": (2, 320, 8, 32, 128, 1, 128),      # N=128: four waves, one per SIMD
    "long_lookback_heads": (1, 300, 16, 64, 128, 2, 256),   # the long-lookback workload's head sizes, ragged length
}


@pytest.mark.parametrize("name", list(SHAPES))
def test_shapes_against_oracle(name):
    b, l, h, p, n, g, q = SHAPES[name]
    check(Workload(name, b, l, h, p, n, g, q), seed=1)


@pytest.mark.parametrize("seqlen", [1, 31, 128, 129, 300, 1000])
def test_ragged_lengths(seqlen):
    check(Workload("ragged", 2, seqlen, 8, 32, 64, 1, 128, init_std=0.5), seed=seqlen)


def test_no_skip_term_and_initial_state():
    check(Workload("no_D", 2, 384, 8, 32, 64, 1, 128, init_std=1.0), seed=3, drop_D=True)


def test_strong_decay_takes_the_exact_diagonal_path():
    # |A| up to 64 with dt up to ~6: whole blocks decay by far more than 2^-120
    check(WORKLOADS["decay_extreme"].with_batch(2), seed=5, seqlen=1024)
    check(Workload("all_large_dt", 2, 256, 8, 32, 64, 1, 128, a_log_range=(32.0, 64.0), dt_law="mixture",
                   x_law="student-t3"), seed=6)


def test_policy_workload_at_oracle_size():
    check(WORKLOADS["policy_bf16"].with_batch(4))


def test_agrees_with_the_staged_kernels():
    w = WORKLOADS["policy_bf16"].with_batch(4)      # too few sequences for the automatic choice
    dev = to_dev(make_inputs(w, seed=11, seqlen=640))
    y1, f1 = run(dev, w.chunk, y_dtype=torch.float32)
    y2, f2 = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                            y_dtype=torch.float32)
    assert rel_err(y1, y2.double().cpu().numpy()) <= 1e-3
    assert rel_err(f1, f2.double().cpu().numpy()) <= 1e-3


def test_chunk_scan_takes_the_one_pass_path_for_large_batches():
    w = WORKLOADS["policy_bf16"].with_batch(128)     # 128 workgroups of 8 units
    dev = to_dev(make_inputs(w, seed=2, seqlen=256))
    y1, f1 = run(dev, w.chunk)
    y2, f2 = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk)
    assert torch.equal(y1, y2) and torch.equal(f1, f2)


def test_chunk_length_does_not_enter():
    # no workspace layout depends on it: the kernel tiles time by its own block, so every chunk gives the same bits
    w = Workload("chunks", 2, 700, 8, 32, 64, 1, 128, init_std=0.3)
    dev = to_dev(make_inputs(w, seed=9))
    ref = run(dev, 128)
    for chunk in (32, 64, 256):
        y, f = run(dev, chunk)
        assert torch.equal(y, ref[0]) and torch.equal(f, ref[1]), chunk
    with pytest.raises(SsdError):
        run(dev, 100)          # still has to be a chunk length the library accepts


def test_unsupported_shapes_are_refused():
    cases = [
        WORKLOADS["plumbing_f32"],                                  # headdim 16 (float32 inputs)
        Workload("f32_n128", 2, 128, 8, 32, 128, 1, 128, dtype="f32"),  # float32 inputs: state 32 or 64 only
        Workload("f32_units4", 2, 128, 4, 32, 64, 1, 128, dtype="f32"), # float32 inputs: 8 units per group
        Workload("p16", 2, 128, 8, 16, 64, 1, 128),                 # headdim not a multiple of 32
        Workload("n16", 2, 256, 8, 32, 16, 1, 128),                 # state narrower than an MFMA tile
        Workload("units2", 2, 128, 2, 32, 64, 1, 128),              # 2 units per group
    ]
    for w in cases:
        dev = to_dev(make_inputs(w, seed=0))
        with pytest.raises(SsdError) as ei:
            run(dev, w.chunk)
        assert ei.value.code == 2, w.name


FLOAT_SHAPES = {
    "policy": (2, 1024, 8, 32, 64, 1, 128),
    "wide_head": (2, 300, 4, 64, 64, 1, 128),        # two 32-column units per head
    "small_state": (3, 257, 16, 32, 32, 2, 64),      # N=32, two groups
    "many_units": (1, 384, 16, 64, 64, 2, 128),      # 16 units per group: two workgroups per (batch, group)
}


@pytest.mark.parametrize("name", list(FLOAT_SHAPES))
def test_float32_shapes_against_oracle(name):
    """float32 inputs run on their own one-pass kernel (three bf16 terms per operand, tiles of 32 steps)."""
    b, l, h, p, n, g, q = FLOAT_SHAPES[name]
    check(Workload(name, b, l, h, p, n, g, q, dtype="f32"), seed=2)


@pytest.mark.parametrize("seqlen", [1, 31, 32, 33, 100, 1000])
def test_float32_ragged_lengths_initial_state_and_no_skip_term(seqlen):
    check(Workload("ragged_f32", 2, seqlen, 8, 32, 64, 1, 128, dtype="f32", init_std=0.5), seed=seqlen)
    check(Workload("ragged_f32_no_D", 2, seqlen, 8, 32, 64, 1, 128, dtype="f32", init_std=0.5), seed=seqlen + 1, drop_D=True)


def test_float32_strong_decay_and_heavy_tails():
    check(WORKLOADS["decay_extreme"].with_batch(2).with_dtype("f32"), seed=5, seqlen=1024)
    check(Workload("all_large_dt_f32", 2, 256, 8, 32, 64, 1, 128, dtype="f32", a_log_range=(32.0, 64.0), dt_law="mixture",
                   x_law="student-t3"), seed=6)


def test_float32_restarts_inside_a_sequence():
    w = Workload("reset_f32", 3, 500, 8, 32, 64, 1, 128, dtype="f32", init_std=0.5)
    cpu = make_inputs(w, seed=13)
    dev = to_dev(cpu)
    m = (np.random.default_rng(5).random((w.batch, w.seqlen)) < 0.02).astype(np.uint8)
    m[0, 0] = 1          # a restart before the first step: the initial state is not read
    m[1, 31] = m[1, 32] = 1   # either side of a tile boundary
    y, f = run(dev, w.chunk, reset=torch.from_numpy(m).cuda())
    yr, fr = orc.ssd_sequential(np64(cpu["x"]), np64(cpu["dt"]), np64(cpu["A"]), np64(cpu["B"]), np64(cpu["C"]),
                                np64(cpu["D"]), np64(cpu["init"]), reset=m)
    assert_close(y, yr, torch.float32, "reset_f32 y")
    assert_close(f, fr, torch.float32, "reset_f32 final")


def test_float32_large_batches_take_the_one_pass_path():
    w = WORKLOADS["policy_bf16"].with_batch(128).with_dtype("f32")
    dev = to_dev(make_inputs(w, seed=2, seqlen=256))
    y1, f1 = run(dev, w.chunk)
    y2, f2 = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk)
    assert torch.equal(y1, y2) and torch.equal(f1, f2)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_one_pass_kernel_on_a_side_stream_and_inside_a_captured_graph(dtype):
    """Same contract as the staged kernels: nothing allocated, nothing synchronised, so the launch can be
    captured (the reference captures its update, trading_bots/src/torch/train/update.rs:206-330).  Replays
    are interleaved with eager work and each is checked."""
    w = Workload("graph", 4, 320, 8, 32, 64, 1, 128, dtype=dtype, init_std=0.2)
    dev = to_dev(make_inputs(w, seed=8))
    y_ref, f_ref = run(dev, 128)
    out, fin = torch.empty_like(dev["x"]), torch.empty(4, 8, 32, 64, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(dev, 128, out=out, final_out=fin)
    side.synchronize()
    assert torch.equal(out, y_ref) and torch.equal(fin, f_ref)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ssd_chunk_scan_onepass(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=128,
                               initial_states=dev["init"], out=out, final_out=fin)
    x_keep = dev["x"].clone()
    for i in range(4):
        out.fill_(float("nan"))
        fin.fill_(float("nan"))
        dev["x"].copy_(x_keep * 0.5 if i % 2 else x_keep)     # change the captured inputs in place
        graph.replay()
        torch.cuda.synchronize()
        y_e, f_e = run(dev, 128)
        assert torch.equal(out, y_e) and torch.equal(fin, f_e), f"replay {i}"


@pytest.mark.parametrize("seqlen,with_reset", [(2048, False), (1990, True)])
def test_mid_size_batches_run_cut_into_segments(seqlen, with_reset):
    """48 sequences of 2048 steps: too few for one workgroup per 8 units to fill the chip, enough work for the
    one-pass kernel on segments of the sequence to beat the staged kernels.  Rows against the oracle, with an
    initial state, a ragged length and restarts that fall on and next to segment borders."""
    from trading_bot_0_amd.ssd import chunk_scan_segments
    w = Workload("segments", 48, seqlen, 8, 32, 64, 1, 128, init_std=0.5)
    assert chunk_scan_segments(w.batch, seqlen, 8, 32, 64, 1, 128) == 4
    assert chunk_scan_segments(4, 4096, 8, 32, 64, 1, 128) == 1          # little work in total: staged
    assert chunk_scan_segments(256, 2048, 8, 32, 64, 1, 128) == 1        # fills the chip uncut
    dev = make_inputs(w, seed=6, device="cuda")
    reset = None
    m = None
    if with_reset:
        m = (np.random.default_rng(3).random((w.batch, seqlen)) < 0.002).astype(np.uint8)
        for t in (511, 512, 513, 1024, 1535, 1536):
            m[1, t] = 1
        reset = torch.from_numpy(m).cuda()
    y32, final = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                initial_states=dev["init"], y_dtype=torch.float32, reset=reset)
    y16, final16 = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                  initial_states=dev["init"], reset=reset)
    assert torch.equal(y16, y32.to(torch.bfloat16)) and torch.equal(final, final16)
    rows = [0, 1, 47]
    yr, fr = orc.ssd_sequential(*(np64(dev[k][rows]) for k in ("x", "dt")), np64(dev["A"]), np64(dev["B"][rows]),
                                np64(dev["C"][rows]), np64(dev["D"]), np64(dev["init"][rows]),
                                reset=None if m is None else m[rows])
    assert_close(y32[rows], yr, torch.bfloat16, "segmented y (float32 y)")
    assert_close(final[rows], fr, torch.bfloat16, "segmented final")
    # the uncut one-pass kernel gives the same result to rounding
    y1, f1 = ssd_chunk_scan_onepass(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                    initial_states=dev["init"], y_dtype=torch.float32, reset=reset)
    assert rel_err(y32, np64(y1)) <= 1e-4 and rel_err(final, np64(f1)) <= 1e-4


@pytest.mark.parametrize("with_reset", [False, True])
def test_float32_mid_size_batches_run_cut_into_segments(with_reset):
    """48 float32 sequences of 2048 steps: too few workgroups to fill the chip uncut, so the float one-pass kernel runs
    on segments of the sequence (states-only pass, then the forward with the recurrence over the segment states in
    its prologue).  Rows against the oracle at the float bar, and the whole against the uncut kernel."""
    from trading_bot_0_amd.ssd import chunk_scan_segments
    w = Workload("segments_f32", 48, 2048, 8, 32, 64, 1, 128, dtype="f32", init_std=0.5)
    assert chunk_scan_segments(w.batch, w.seqlen, 8, 32, 64, 1, 128, dtype=torch.float32) >= 2
    dev = make_inputs(w, seed=6, device="cuda")
    reset = None
    m = None
    if with_reset:
        m = (np.random.default_rng(3).random((w.batch, w.seqlen)) < 0.002).astype(np.uint8)
        for t in (0, 511, 512, 513, 1024, 1535, 1536):
            m[1, t] = 1
        reset = torch.from_numpy(m).cuda()
    y, final = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                              initial_states=dev["init"], reset=reset)
    rows = [0, 1, 47]
    yr, fr = orc.ssd_sequential(*(np64(dev[k][rows]) for k in ("x", "dt")), np64(dev["A"]), np64(dev["B"][rows]),
                                np64(dev["C"][rows]), np64(dev["D"]), np64(dev["init"][rows]),
                                reset=None if m is None else m[rows])
    assert_close(y[rows], yr, torch.float32, "float segmented y")
    assert_close(final[rows], fr, torch.float32, "float segmented final")
    y1, f1 = ssd_chunk_scan_onepass(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                    initial_states=dev["init"], reset=reset)
    assert rel_err(y, np64(y1)) <= 1e-5 and rel_err(final, np64(f1)) <= 1e-5


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("batch,seqlen", [(288, 512), (272, 2048)])
def test_partial_last_round_runs_as_a_batch_of_its_own(batch, seqlen, dtype):
    """256 workgroups fill the chip; the 32 or 16 sequences beyond run staged (short) or cut into segments (long)
    after the whole round.  Rows of both parts against the oracle, and the whole against the uncut kernel."""
    w = Workload("tail", batch, seqlen, 8, 32, 64, 1, 128, dtype=dtype, init_std=0.5)
    td = w.torch_dtype
    dev = make_inputs(w, seed=9, device="cuda")
    m = (np.random.default_rng(5).random((batch, seqlen)) < 0.002).astype(np.uint8)
    reset = torch.from_numpy(m).cuda()
    yd = torch.float32 if dtype == "bf16" else None
    y32, final = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                initial_states=dev["init"], y_dtype=yd, reset=reset)
    rows = [0, 255, 256, batch - 1]
    yr, fr = orc.ssd_sequential(*(np64(dev[k][rows]) for k in ("x", "dt")), np64(dev["A"]), np64(dev["B"][rows]),
                                np64(dev["C"][rows]), np64(dev["D"]), np64(dev["init"][rows]), reset=m[rows])
    assert_close(y32[rows], yr, td, "tail y (float32 y)")
    assert_close(final[rows], fr, td, "tail final")
    y1, f1 = ssd_chunk_scan_onepass(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                    initial_states=dev["init"], y_dtype=yd, reset=reset)
    assert torch.equal(y32[:256], y1[:256]) and torch.equal(final[:256], f1[:256])     # the whole round is that kernel
    tol = 1e-4 if dtype == "bf16" else 1e-5
    assert rel_err(y32[256:], np64(y1[256:])) <= tol and rel_err(final[256:], np64(f1[256:])) <= tol


@pytest.mark.parametrize("heads", [(4, 32, 64, 1), (2, 64, 64, 1), (8, 32, 32, 2)])
def test_groups_of_four_units_take_the_one_pass_kernel(heads):
    """Four units per group (four heads of 32 columns, two of 64, eight in two groups): workgroups of four waves, two
    to a CU.  The whole-forward entry point picks that path from mid-size batches on (it is the faster one there: 144
    against 263 us for 256 sequences of 2 048 steps) and the staged kernels for small ones; rows against the oracle
    with an initial state, a ragged length and restarts, and the bf16 y as the rounded float32 y."""
    from trading_bot_0_amd.ssd import chunk_scan_is_onepass
    H, P, N, G = heads
    assert chunk_scan_is_onepass(300, 1000, H, P, N, G, 128)
    assert not chunk_scan_is_onepass(16, 1000, H, P, N, G, 128)
    w = Workload("four_units", 300, 1000, H, P, N, G, 128, init_std=0.5)
    dev = make_inputs(w, seed=8, device="cuda")
    m = (np.random.default_rng(4).random((w.batch, w.seqlen)) < 0.003).astype(np.uint8)
    m[2, 0] = 1
    reset = torch.from_numpy(m).cuda()
    y32, final = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                initial_states=dev["init"], y_dtype=torch.float32, reset=reset)
    y16, final16 = ssd_chunk_scan(dev["x"], dev["dt"], dev["A"], dev["B"], dev["C"], dev["D"], chunk=w.chunk,
                                  initial_states=dev["init"], reset=reset)
    assert torch.equal(y16, y32.to(torch.bfloat16)) and torch.equal(final, final16)
    rows = [0, 2, 299]
    yr, fr = orc.ssd_sequential(*(np64(dev[k][rows]) for k in ("x", "dt")), np64(dev["A"]), np64(dev["B"][rows]),
                                np64(dev["C"][rows]), np64(dev["D"]), np64(dev["init"][rows]), reset=m[rows])
    assert_close(y32[rows], yr, torch.bfloat16, "four-wave one-pass y (float32 y)")
    assert_close(final[rows], fr, torch.bfloat16, "four-wave one-pass final")
    assert_stored_bf16_close(y16[rows], yr, "four-wave one-pass stored y")
