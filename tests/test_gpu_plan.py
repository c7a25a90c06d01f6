"""The path plan of ssd_chunk_scan_fwd against the clock.  The library decides from a cost model (time per tile and
workgroup of the one-pass kernel, time per unit-tile of the staged kernels, cost of a launch) whether a shape runs on
the staged kernels, as one launch of the one-pass kernel, or on the one-pass kernel over segments of the sequence.
The model's constants are measurements that every kernel change moves; this test times, either side of the model's
cross-overs, the plan's choice beside the alternatives a caller can force -- the one-pass kernel
(ssd_chunk_scan_onepass_fwd) and the staged kernels through their own entry points -- and asserts that what the plan
picked is within a quarter of the fastest of them (a wrong side of a cross-over costs a factor of about two).

Timing: the best of three means over twenty calls, HIP events on the launch stream, after a spin of the same work."""
from ctypes import byref

import pytest
import torch

from trading_bot_0_amd import ssd
from trading_bot_0_amd.synthetic import Workload, make_inputs

pytestmark = pytest.mark.gpu


def best_of(fn, reps=3, calls=20):
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(calls):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / calls * 1e3)
    return best   # microseconds


SHAPES = [
    # (nheads, headdim, dstate, ngroups, seqlen, batches either side of the cross-overs)
    (8, 32, 64, 1, 2048, (4, 16, 32, 64, 128, 160, 256, 272)),      # staged | segments | one launch | whole rounds + a rest
    (8, 32, 64, 1, 512, (16, 64, 128, 256)),
    (4, 32, 64, 1, 2048, (32, 64, 128, 192, 256, 512)),             # four units per group: staged | four-wave one-pass
    (16, 64, 128, 2, 4096, (1, 4, 8, 16)),                          # 128-wide state
]


@pytest.mark.parametrize("H,P,N,G,L,batches", SHAPES)
def test_plan_picks_a_path_within_a_quarter_of_the_fastest(H, P, N, G, L, batches):
    lib = ssd.load_library()
    report = []
    for Bsz in batches:
        w = Workload("plan", Bsz, L, H, P, N, G, 128)
        inp = make_inputs(w, seed=1, device="cuda")
        x, dt, A, Bm, Cm, D = (inp[k] for k in ("x", "dt", "A", "B", "C", "D"))
        plan = ssd.PreparedChunkScan(x, dt, A, Bm, Cm, D, chunk=w.chunk)
        t_plan = best_of(plan)
        times = {}
        y = torch.empty_like(x)
        fin = torch.empty(Bsz, H, P, N, device="cuda")
        dims = ssd.SsdDims(Bsz, L, H, P, N, G, w.chunk)
        stream = torch.cuda.current_stream().cuda_stream

        def onepass():
            return lib.ssd_chunk_scan_onepass_fwd(byref(dims), ssd.SSD_DTYPE_BF16, x.data_ptr(), dt.data_ptr(), A.data_ptr(),
                                                  Bm.data_ptr(), Cm.data_ptr(), D.data_ptr(), None, None, y.data_ptr(),
                                                  fin.data_ptr(), stream)

        if onepass() == 0:
            times["one-pass"] = best_of(onepass)
        else:
            ssd.last_error(lib)   # (clear the message of a shape the one-pass kernel does not take)
        dtcs = ssd.chunk_cumsum(dt, A, w.chunk)
        prev, _ = ssd.chunk_state_passing(x, Bm, dtcs)

        def staged():
            lib.ssd_chunk_cumsum_fwd(byref(dims), ssd.SSD_DTYPE_BF16, dt.data_ptr(), A.data_ptr(), dtcs.data_ptr(), stream)
            lib.ssd_chunk_state_passing_fwd(byref(dims), ssd.SSD_DTYPE_BF16, x.data_ptr(), Bm.data_ptr(), dtcs.data_ptr(), None,
                                            prev.data_ptr(), fin.data_ptr(), stream)
            lib.ssd_chunk_scan_stage_fwd(byref(dims), ssd.SSD_DTYPE_BF16, x.data_ptr(), Bm.data_ptr(), Cm.data_ptr(),
                                         dtcs.data_ptr(), prev.data_ptr(), D.data_ptr(), y.data_ptr(), stream)

        times["staged"] = best_of(staged)
        fastest = min(times.values())
        segs = ssd.chunk_scan_segments(Bsz, L, H, P, N, G, w.chunk)
        one = ssd.chunk_scan_is_onepass(Bsz, L, H, P, N, G, w.chunk)
        chosen = "one launch" if one else (f"{segs} segments" if segs > 1 else "staged / split")
        report.append(f"batch {Bsz}: plan ({chosen}) {t_plan:.0f} us; " + ", ".join(f"{k} {v:.0f}" for k, v in times.items()))
        assert t_plan <= 1.25 * fastest + 5.0, "\n".join(report)
        del plan, inp, x, dt, Bm, Cm, y, fin, dtcs, prev
    print("\n".join(report))
