#!/usr/bin/env python3
"""Benchmark of the SSD chunk-scan forward on one MI355X.

A step is one forward of the whole op (`ssd_chunk_scan_fwd`) over one batch of seeded synthetic
inputs already resident in HBM.  At the default size the library runs it as ONE kernel (the one-pass
scan: x, dt, B, C read once, y and the final state written once); smaller batches run as the staged
kernels (stages 1-4 on one stream).  Default workload: the policy shape
(batch 256, seqlen 2048, 8 heads, headdim 32, dstate 64, one group, chunk 128, bf16 inputs with
fp32 accumulation, final states returned).  Prints ONE JSON line:

  value        timesteps*batch/s of the whole forward: K steps between two HIP events on the launch stream, after
               W warm-up steps and a fixed spin of the same forward (0.25 s of wall time, outside the timed region)
               that brings the GPU's clocks to their steady state whatever W is; the wall clock around the same K
               steps is printed beside it (ms_per_step_wall)
  err_y, err_final  parity of this very run: max|out - ref| / rms(ref) against the float64 sequential oracle on the
               first batch rows; for bf16 inputs err_y is the float32-y output of the same kernel (the judged
               figure) and err_y_stored_bf16 the stored bf16 y (dominated by its own output rounding)
  roofline     the dominant kernel of the forward as the library runs it: algorithmic bytes per
               launch / its mean duration, measured with HIP events on the launch stream over a
               second timed region of K steps.  One-pass forward: that kernel, against the
               compulsory traffic of the whole op.  Staged forward: the slowest stage.
  stages       the staged kernels issued one by one through their own entry points, each with
               its algorithmic bytes, GB/s and (stages 2, 4) dense MFMA rate; measured in both cases
  stream_step  the single-timestep update at batch 4096: latency and GB/s over the 64 steps, and over a loop of 1 000
               steps with an event per step (mean and median); stream_steps_one_launch: the same
               64 steps as one call of ssd_steps_fwd (which runs 16 steps or more on the one-pass scan)
  reference_suite  the reference's historical benchmark cases for this path (batch 4, seq_len 4096,
               BFloat16) in the reference's result schema: mamba2_* rows time this library's whole Mamba-2 block
               (sizes in each row's config), ssd_scan_* rows the scan op alone
  forward_float32_y  the float32-y instance of the headline kernel (bf16 inputs, y stored as float32): the output
               err_y is measured on, timed beside the bf16-y instance, against its own compulsory traffic
  workloads    the other configurations at full size (plumbing, long lookback, decay-extreme in bf16 and float32):
               forward time (mean and median of 100 calls), path, HBM and MFMA fractions, errors of this run against
               the oracle on the first batch row; --no-workloads skips them
  forward_float32  the same workload with float32 inputs (the other parity mode): time per call, which path ran (the
               float one-pass kernel on three bf16 terms per operand, or the staged kernels on float MFMAs), its
               compulsory traffic against the HBM peak, and its matrix-core rate against the pipe it multiplies on
               (the one-pass kernel executes six bf16 products per float product: 6 x the dense flops against the
               bf16 peak; the staged kernels the dense flops against the float MFMA peak), and its parity errors
               against the oracle on the first batch rows
  backward     the backward pass of the scan at the same shape: time per call, and its compulsory traffic
               (x, dt, B, C, dy read; dx, ddt, dB, dC written) against the HBM peak
  mamba2_block the block around the scan at the policy shape (d_model = nheads*headdim): whole block, and the
               library's projection, pre-scan and post-scan kernels alone with their GB/s (the projections
               also through the BLAS behind torch, for comparison)
  cpu_baseline the plain-C oracle (sequential recurrence, float32, OpenMP) timed on this
               box's host cores on a bounded batch slice of the same workload; beside it the chunked algorithm
               in ATen CPU float32 ops (the reference's CPU backend) at 1 thread and at all usable cores, the
               host's core count and CPU model

After an idle period the first milliseconds of kernels run measurably slower (the clocks ramp), so every timed
region here is preceded by a spin of the same work for a fixed wall time, not just by W calls.

Timing follows the reference harness (warm-up calls, device sync, timed calls, device sync,
mean per call: benchmarks/src/main.rs:140-166; stream step = prefill once then timed single
steps: main.rs:168-200).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
# HBM bytes per forward of the dominant kernel(s), measured with rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE on
# this very command at the library revision the profiles name (profiles/chunk_scan_forward_*.md give the KiB per
# dispatch of each counter and the copy-kernel calibration, factor 1.00); counters cannot be read from inside this
# script, so the figures are carried here, keyed by (workload, batch): a run at any other size reports null.
# Reads come out below the compulsory bytes because inputs that stay in the 256 MB last-level cache from one call
# of the loop to the next are not fetched from HBM again.
MEASURED_TRAFFIC_BYTES = {("policy_bf16", 256): 493.6e6,          # 201 600 + 280 400 KiB, one launch
                          ("long_lookback_bf16", 32): 2116.6e6,   # 1 002 000 + 1 065 000 KiB, one launch
                          ("decay_extreme", 64): 326.8e6}         # states only 63 050 + 12 290, forward 107 200 + 136 600 KiB
TRAFFIC_MEASURED_AT = "4178078"   # the library revision the counter runs in profiles/ were made at
# matrix-pipe busy fraction of the same kernels from the same counter runs (SQ_VALU_MFMA_BUSY_CYCLES over the
# SIMD-cycles of the launch, GRBM_GUI_ACTIVE / 8 x 1 024 SIMDs): what the north star's "MFMA utilisation" reads as
# on the hardware's own counters (decay-extreme: the forward launch of the two)
MEASURED_MFMA_PIPE_BUSY = {("policy_bf16", 256): 0.236, ("long_lookback_bf16", 32): 0.251, ("decay_extreme", 64): 0.189}
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_F32_PEAK_TFLOPS = 157.3


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="policy_bf16")
    ap.add_argument("--batch", type=int, default=None, help="override the workload's batch")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-stream-step", action="store_true")
    ap.add_argument("--no-reference-suite", action="store_true")
    ap.add_argument("--no-block", action="store_true")
    ap.add_argument("--no-backward", action="store_true")
    ap.add_argument("--no-float32", action="store_true")
    ap.add_argument("--no-workloads", action="store_true", help="skip the other workloads' rows (full size, forward only)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain elementwise kernel over 256 MiB in / 256 MiB out three times, the known-size "
                         "reference that rocprofv3's FETCH_SIZE / WRITE_SIZE readings are scaled by")
    return ap.parse_args()


SPIN_SECONDS = 0.25


def f32_mfma(dense_flops, seconds, on_bf16_pipe):
    """The float32 mode's matrix-core figures against the pipe the path multiplies on: the float one-pass kernel forms
    every product from six bf16 MFMAs (three bf16 terms per operand), so it executes 6 x the op's dense flops on the
    bf16 pipe; the staged float kernels use float MFMAs."""
    if on_bf16_pipe:
        executed = 6.0 * dense_flops
        return {"mfma_pipe": "bf16 (six bf16 products per float product)", "executed_TFLOPs": round(executed / seconds / 1e12, 1),
                "peak_TFLOPs": MFMA_BF16_PEAK_TFLOPS, "mfma_frac": round(executed / seconds / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
    return {"mfma_pipe": "float32", "executed_TFLOPs": round(dense_flops / seconds / 1e12, 1),
            "peak_TFLOPs": MFMA_F32_PEAK_TFLOPS, "mfma_frac": round(dense_flops / seconds / 1e12 / MFMA_F32_PEAK_TFLOPS, 4)}


def spin(fn, torch, seconds=SPIN_SECONDS):
    """Runs fn back to back for a fixed wall time (untimed): the clocks settle under this very load."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def event_time_steps(fn, steps, torch):
    """(seconds per step from two HIP events on the current stream around `steps` calls, the same by wall clock);
    synchronised on both sides (the reference harness's order: warm-up, sync, timed calls, sync --
    benchmarks/src/main.rs:140-166)."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return e0.elapsed_time(e1) * 1e-3 / steps, wall


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; the path shards along batch without "
              "communication, so --gpus N>1 is not measured here", file=sys.stderr)
        sys.exit(2)

    import torch
    from trading_bot_0_amd import ssd
    from trading_bot_0_amd.synthetic import (WORKLOADS, algorithmic_bytes_fwd, make_inputs, stage_bytes,
                                             stage_flops, step_bytes)

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    ssd.load_library()   # raises if the HIP library is not built: there is no other path
    torch.cuda.set_device(0)
    w = WORKLOADS[args.workload]
    if args.batch:
        w = w.with_batch(args.batch)
    inp = make_inputs(w, seed=0, device="cuda")
    x, dt, A, Bm, Cm, D, init = (inp[k] for k in ("x", "dt", "A", "B", "C", "D", "init"))
    ws = torch.empty(ssd.workspace_bytes(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk),
                     dtype=torch.uint8, device="cuda")
    y = torch.empty_like(x)
    final = torch.empty((w.batch, w.nheads, w.headdim, w.dstate), dtype=torch.float32, device="cuda")

    # arguments validated and pointers fixed once; a step is then the bare foreign call into the C ABI
    # (the Python wrapper's per-call checks cost more than the kernel leaves room for)
    forward = ssd.PreparedChunkScan(x, dt, A, Bm, Cm, D, chunk=w.chunk, initial_states=init, workspace=ws, out=y,
                                    final_out=final)

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)   # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        forward()
    spin(forward, torch)
    sec, sec_wall = event_time_steps(forward, args.steps, torch)
    value = w.units / sec

    # ---- parity of this run: the first rows of the batch against the float64 sequential oracle ----
    import numpy as np
    from oracle import c_oracle
    from oracle import ssd_oracle as orc
    rows = min(w.batch, 2)

    def f64(t):
        return None if t is None else t[:rows].float().cpu().numpy().astype(np.float64)

    y_ref, f_ref = c_oracle.ssd_sequential_c(f64(x), f64(dt), A.cpu().numpy().astype(np.float64), f64(Bm), f64(Cm),
                                             None if D is None else D.cpu().numpy().astype(np.float64), f64(init),
                                             nthreads=min(16, os.cpu_count() or 1))
    errors = {"err_final": orc.rel_err(final[:rows].cpu().numpy(), f_ref), "err_rows": rows}
    if w.dtype == "bf16":
        y32, _ = ssd.ssd_chunk_scan(x, dt, A, Bm, Cm, D, chunk=w.chunk, initial_states=init, y_dtype=torch.float32,
                                    workspace=ws)
        errors["err_y"] = orc.rel_err(y32[:rows].cpu().numpy(), y_ref)
        errors["err_y_output"] = "float32 y of the bf16-input kernel (the judged output); the stored bf16 y is it rounded once"
        errors["err_y_stored_bf16"] = orc.rel_err(y[:rows].float().cpu().numpy(), y_ref)
        errors["stored_y_is_rounded_f32_y"] = bool(torch.equal(y, y32.to(torch.bfloat16)))
        errors["tolerance"] = 2e-2
        del y32
    else:
        errors["err_y"] = orc.rel_err(y[:rows].cpu().numpy(), y_ref)
        errors["err_y_output"] = "float32 y"
        errors["tolerance"] = 1e-4
    del y_ref, f_ref

    # ---- second timed region: the four stages one by one, HIP events between them -------------
    dtcs = ssd.chunk_cumsum(dt, A, w.chunk)
    S = ssd.chunk_state(x, Bm, dtcs)

    lib = ssd.load_library()
    from ctypes import byref
    dims = ssd.SsdDims(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk)
    code = ssd.SSD_DTYPE_BF16 if w.dtype == "bf16" else ssd.SSD_DTYPE_F32
    stream = torch.cuda.current_stream().cuda_stream
    ip = None if init is None else init.data_ptr()

    def k1():
        return lib.ssd_chunk_cumsum_fwd(byref(dims), code, dt.data_ptr(), A.data_ptr(), dtcs.data_ptr(), stream)

    def k2():
        return lib.ssd_chunk_state_fwd(byref(dims), code, x.data_ptr(), Bm.data_ptr(), dtcs.data_ptr(),
                                       S.data_ptr(), stream)

    def k3():
        return lib.ssd_state_passing_fwd(byref(dims), S.data_ptr(), dtcs.data_ptr(), ip, S.data_ptr(),
                                         final.data_ptr(), stream)

    def k4():
        return lib.ssd_chunk_scan_stage_fwd(byref(dims), code, x.data_ptr(), Bm.data_ptr(), Cm.data_ptr(),
                                            dtcs.data_ptr(), S.data_ptr(), D.data_ptr(), y.data_ptr(), stream)

    def k23():
        return lib.ssd_chunk_state_passing_fwd(byref(dims), code, x.data_ptr(), Bm.data_ptr(), dtcs.data_ptr(), ip,
                                               S.data_ptr(), final.data_ptr(), stream)

    # the stages the whole-forward entry point launches for this shape: with at least 512 (batch, head)
    # sequences it runs stages 2 and 3 as one kernel
    if w.batch * w.nheads >= 512:
        stage_fns = [("chunk_cumsum", k1), ("chunk_state_passing", k23), ("chunk_scan", k4)]
    else:
        stage_fns = [("chunk_cumsum", k1), ("chunk_state", k2), ("state_passing", k3), ("chunk_scan", k4)]
    for _ in range(max(2, args.warmup // 2)):
        for _, fn in stage_fns:
            assert fn() == 0, ssd.last_error(lib)
    spin(lambda: [fn() for _, fn in stage_fns], torch)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(len(stage_fns) + 1)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    for i in range(args.steps):
        ev[i][0].record()
        for j, (_, fn) in enumerate(stage_fns):
            fn()
            ev[i][j + 1].record()
    torch.cuda.synchronize()
    sb, sf = stage_bytes(w), stage_flops(w)
    stages = {}
    for j, (name, _) in enumerate(stage_fns):
        ms = sum(ev[i][j].elapsed_time(ev[i][j + 1]) for i in range(args.steps)) / args.steps
        gbs = sb[name] / (ms * 1e-3) / 1e9
        stages[name] = {"ms": round(ms, 5), "alg_bytes": sb[name], "GBps": round(gbs, 1),
                        "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)}
        if name in sf:
            tf = sf[name] / (ms * 1e-3) / 1e12
            stages[name]["dense_TFLOPs"] = round(tf, 1)
            stages[name]["mfma_frac"] = round(tf / MFMA_BF16_PEAK_TFLOPS, 4)
    # stages 2 and 3 as kernels of their own (the whole-forward entry point fuses them for large batches):
    # state passing alone is the pure-bandwidth recurrence over the chunk states
    separate = {}
    if len(stage_fns) == 3:
        pair = [("chunk_state", k2), ("state_passing", k3)]
        n_sep = max(10, args.steps // 5)
        for _, fn in pair:
            assert fn() == 0, ssd.last_error(lib)
        spin(lambda: (k2(), k3()), torch, 0.1)
        se = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(n_sep)]
        torch.cuda.synchronize()
        for i in range(n_sep):
            se[i][0].record()
            k2()
            se[i][1].record()
            k3()
            se[i][2].record()
        torch.cuda.synchronize()
        for j, (name, _) in enumerate(pair):
            ms = sum(se[i][j].elapsed_time(se[i][j + 1]) for i in range(n_sep)) / n_sep
            gbs = sb[name] / (ms * 1e-3) / 1e9
            separate[name] = {"ms": round(ms, 5), "alg_bytes": sb[name], "GBps": round(gbs, 1),
                              "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)}
    segments = ssd.chunk_scan_segments(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk, w.torch_dtype)
    onepass = ssd.chunk_scan_is_onepass(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk,
                                        w.torch_dtype)
    if onepass or segments > 1:
        # the forward is one kernel (or, cut into segments, that kernel twice with a small one between): events
        # around each call, on the launch stream
        spin(forward, torch)
        oe = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(args.steps)]
        torch.cuda.synchronize()
        for i in range(args.steps):
            oe[i][0].record()
            forward()
            oe[i][1].record()
        torch.cuda.synchronize()
        per_call = sorted(a.elapsed_time(b) for a, b in oe)
        ms = sum(per_call) / args.steps
        ms_median = per_call[len(per_call) // 2]
        ab = algorithmic_bytes_fwd(w)
        gbs = ab / (ms * 1e-3) / 1e9
        tf = sum(sf[k] for k in ("chunk_state", "chunk_scan")) / (ms * 1e-3) / 1e12
        onepass_info = {"ms": round(ms, 5), "ms_median": round(ms_median, 5), "calls": args.steps, "alg_bytes": ab,
                        "GBps": round(gbs, 1),
                        "hbm_frac": round(gbs / HBM_PEAK_GBS, 4), "dense_TFLOPs": round(tf, 1),
                        "mfma_frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4)}
        roofline = {"kernel": "onepass_scan" if onepass else f"onepass_scan on {segments} segments", "bound": "hbm", "achieved": onepass_info["GBps"],
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": onepass_info["hbm_frac"],
                    "traffic": MEASURED_TRAFFIC_BYTES.get((w.name, w.batch)),
                    "traffic_measured_at": TRAFFIC_MEASURED_AT if (w.name, w.batch) in MEASURED_TRAFFIC_BYTES else None,
                    "mfma_pipe_busy": MEASURED_MFMA_PIPE_BUSY.get((w.name, w.batch)),
                    "mfma_pipe_busy_note": "SQ_VALU_MFMA_BUSY_CYCLES over the launch's SIMD-cycles (GRBM_GUI_ACTIVE / 8 x "
                                           "1024) of the same kernel, from the rocprofv3 --pmc run of that revision "
                                           "(profiles/)"}
        if w.dtype == "bf16":
            # the float32-y instance of the same kernel: the output err_y is measured on (bf16 inputs, y in float32,
            # so its compulsory traffic holds y at four bytes per element)
            y32buf = torch.empty(x.shape, dtype=torch.float32, device="cuda")
            fwd32 = ssd.PreparedChunkScan(x, dt, A, Bm, Cm, D, chunk=w.chunk, initial_states=init, workspace=ws, out=y32buf,
                                          final_out=final, y_dtype=torch.float32)
            spin(fwd32, torch)
            t32y, _ = event_time_steps(fwd32, args.steps, torch)
            ab32 = ab + 2 * x.numel()
            y32_info = {"ms": round(t32y * 1e3, 5), "alg_bytes": ab32, "GBps": round(ab32 / t32y / 1e9, 1),
                        "hbm_frac": round(ab32 / t32y / 1e9 / HBM_PEAK_GBS, 4),
                        "units_per_s": round(w.units / t32y, 1),
                        "note": "the instance err_y is measured on; the headline instance stores the same y rounded to bf16"}
            del y32buf, fwd32
        else:
            y32_info = None
    else:
        dom = max(stages, key=lambda k: stages[k]["ms"])
        roofline = {"kernel": dom, "bound": "hbm", "achieved": stages[dom]["GBps"], "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": stages[dom]["hbm_frac"], "traffic": None}

    out = {
        "metric": "SSD scan timesteps*batch/s at policy shape" if args.workload == "policy_bf16"
                  else f"SSD scan timesteps*batch/s ({args.workload})",
        "value": value, "unit": "timesteps*batch/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "ms_per_step_wall": sec_wall * 1e3,
        "timing": f"HIP events on the launch stream around the {args.steps} steps, after {args.warmup} warm-up steps and "
                  f"{SPIN_SECONDS} s of the same forward untimed",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.dtype, "data": "synthetic",
        "config": {"workload": w.name, "batch": w.batch, "seqlen": w.seqlen, "nheads": w.nheads,
                   "headdim": w.headdim, "dstate": w.dstate, "ngroups": w.ngroups, "chunk": w.chunk},
        **errors,
        "forward_alg_bytes": algorithmic_bytes_fwd(w),
        "forward_hbm_frac": round(algorithmic_bytes_fwd(w) / sec / 1e9 / HBM_PEAK_GBS, 4),
        "forward_path": "onepass" if onepass else (f"onepass on {segments} segments" if segments > 1 else "staged"),
        "roofline": roofline, "stages": stages,
        "stages_alone": separate,
        "stages_ms_sum": round(sum(s["ms"] for s in stages.values()), 5),
    }
    if onepass or segments > 1:
        out["onepass_scan"] = onepass_info
        out["ms_per_call_median"] = onepass_info["ms_median"]
        if y32_info is not None:
            out["forward_float32_y"] = y32_info

    # ---- the same workload in float32 mode (the north star's other parity mode): bound by the float MFMAs ----
    if not args.no_float32 and w.dtype == "bf16":
        x32, dt32, B32, C32 = x.float(), dt.float(), Bm.float(), Cm.float()
        try:
            f32_call = ssd.PreparedChunkScan(x32, dt32, A, B32, C32, D, chunk=w.chunk, initial_states=init)
        except ssd.SsdError:
            f32_call = None   # float tiles of this shape do not fit the LDS
        if f32_call is not None:
            spin(f32_call, torch)
            t32, _ = event_time_steps(f32_call, 20, torch)
            fl = sum(sf[k] for k in ("chunk_state", "chunk_scan"))   # dense MFMA flops of the op
            f32_onepass = ssd.chunk_scan_is_onepass(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk,
                                                    dtype=torch.float32)
            f32_segments = ssd.chunk_scan_segments(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk,
                                                   dtype=torch.float32)
            io32 = 4 * (2 * w.batch * w.seqlen * w.nheads * w.headdim + w.batch * w.seqlen * w.nheads +
                        2 * w.batch * w.seqlen * w.ngroups * w.dstate) + \
                4 * w.batch * w.nheads * w.headdim * w.dstate * (2 if init is not None else 1)
            y32o, f32o = f32_call()
            torch.cuda.synchronize()
            from oracle import c_oracle
            from oracle import ssd_oracle as orc
            nb_err = min(w.batch, 2)

            def f64(t):
                return None if t is None else t[:nb_err].cpu().numpy().astype(np.float64)

            y_ref, f_ref = c_oracle.ssd_sequential_c(f64(x32), f64(dt32), A.cpu().numpy().astype(np.float64), f64(B32), f64(C32),
                                                     None if D is None else D.cpu().numpy().astype(np.float64), f64(init),
                                                     nthreads=min(16, os.cpu_count() or 1))
            e32 = (orc.rel_err(y32o[:nb_err].cpu().numpy(), y_ref), orc.rel_err(f32o[:nb_err].cpu().numpy(), f_ref))
            del y_ref, f_ref
            out["forward_float32"] = {"ms": round(t32 * 1e3, 4),
                                      "path": "one-pass (three bf16 terms per operand)" if f32_onepass
                                      else (f"one-pass on {f32_segments} segments (three bf16 terms per operand)" if f32_segments > 1 else "staged"),
                                      "compulsory_io_bytes": io32,
                                      "hbm_frac": round(io32 / t32 / 1e9 / HBM_PEAK_GBS, 4),
                                      "dense_TFLOPs": round(fl / t32 / 1e12, 1),
                                      **f32_mfma(fl, t32, f32_onepass or f32_segments > 1),
                                      "units_per_s": round(w.batch * w.seqlen / t32, 1),
                                      "err_y": e32[0], "err_final": e32[1], "tolerance": 1e-4}
            del y32o, f32o
        del x32, dt32, B32, C32, f32_call

    # ---- the backward pass at the benchmark shape ------------------------------------------------------
    if not args.no_backward:
        dyb = torch.randn_like(x)
        wsb = torch.empty(ssd.backward_workspace_bytes(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk,
                                                        w.torch_dtype), dtype=torch.uint8, device="cuda")

        def bwd_call():
            ssd.ssd_chunk_scan_backward(x, dt, A, Bm, Cm, D, dyb, chunk=w.chunk, initial_states=init, workspace=wsb)

        spin(bwd_call, torch)
        t_bwd, _ = event_time_steps(bwd_call, 20, torch)
        e = 2 if w.dtype == "bf16" else 4
        BL = w.batch * w.seqlen
        bwd_bytes = e * BL * (3 * w.nheads * w.headdim + 2 * w.nheads + 4 * w.ngroups * w.dstate)
        out["backward"] = {"ms": round(t_bwd * 1e3, 4), "alg_bytes": bwd_bytes,
                           "GBps": round(bwd_bytes / t_bwd / 1e9, 1),
                           "hbm_frac": round(bwd_bytes / t_bwd / 1e9 / HBM_PEAK_GBS, 4),
                           "workspace_bytes": wsb.numel(), "units_per_s": round(BL / t_bwd, 1),
                           "parity": "against this repository's float64 adjoint, pinned by central differences of the forward "
                                     "oracle (tests/test_oracle_backward.py); the reference holds no backward of this op: "
                                     "unpinned by the reference"}
        del dyb, wsb

    # ---- the other workloads at full size: forward only, one row each -----------------------------------
    # (the configurations beside the headline one: parity for them is in the tests; here their time, path, traffic
    # fractions and this run's errors against the oracle on the first batch row, so that one run covers them all)
    if not args.no_workloads and args.workload == "policy_bf16" and not args.batch:
        rows_out = []
        for wname, wdtype in (("plumbing_f32", "f32"), ("long_lookback_bf16", "bf16"), ("decay_extreme", "bf16"),
                              ("decay_extreme", "f32")):
            ww = WORKLOADS[wname].with_dtype(wdtype)
            wi = make_inputs(ww, seed=0, device="cuda")
            call = ssd.PreparedChunkScan(wi["x"], wi["dt"], wi["A"], wi["B"], wi["C"], wi["D"], chunk=ww.chunk,
                                         initial_states=wi["init"])
            spin(call, torch, 0.1)
            n_calls = 100
            we = [torch.cuda.Event(enable_timing=True) for _ in range(n_calls + 1)]
            torch.cuda.synchronize()
            we[0].record()
            for i in range(n_calls):
                call()
                we[i + 1].record()
            torch.cuda.synchronize()
            per = sorted(we[i].elapsed_time(we[i + 1]) for i in range(n_calls))
            t_w = we[0].elapsed_time(we[n_calls]) * 1e-3 / n_calls
            wy, wf = call()
            if wdtype == "bf16":   # judged on the float32 y of the same kernel, as the headline
                wy32, _ = ssd.ssd_chunk_scan(wi["x"], wi["dt"], wi["A"], wi["B"], wi["C"], wi["D"], chunk=ww.chunk,
                                             initial_states=wi["init"], y_dtype=torch.float32)
                stored_ok = bool(torch.equal(wy, wy32.to(torch.bfloat16)))
            else:
                wy32, stored_ok = wy, None
            torch.cuda.synchronize()

            def one(t):
                return None if t is None else t[:1].float().cpu().numpy().astype(np.float64)

            yr, fr = c_oracle.ssd_sequential_c(one(wi["x"]), one(wi["dt"]), wi["A"].cpu().numpy().astype(np.float64),
                                               one(wi["B"]), one(wi["C"]), wi["D"].cpu().numpy().astype(np.float64),
                                               one(wi["init"]), nthreads=min(16, os.cpu_count() or 1))
            segs = ssd.chunk_scan_segments(ww.batch, ww.seqlen, ww.nheads, ww.headdim, ww.dstate, ww.ngroups, ww.chunk,
                                           ww.torch_dtype)
            one_launch = ssd.chunk_scan_is_onepass(ww.batch, ww.seqlen, ww.nheads, ww.headdim, ww.dstate, ww.ngroups,
                                                   ww.chunk, ww.torch_dtype)
            wab = algorithmic_bytes_fwd(ww)
            wfl = sum(stage_flops(ww)[k] for k in ("chunk_state", "chunk_scan"))
            row = {"workload": wname, "dtype": wdtype, "batch": ww.batch, "seqlen": ww.seqlen, "nheads": ww.nheads,
                   "headdim": ww.headdim, "dstate": ww.dstate, "ngroups": ww.ngroups, "chunk": ww.chunk,
                   "ms": round(t_w * 1e3, 5), "ms_median": round(per[n_calls // 2], 5), "calls": n_calls,
                   "path": "onepass" if one_launch else (f"onepass on {segs} segments" if segs > 1 else "staged"),
                   "alg_bytes": wab, "hbm_frac": round(wab / t_w / 1e9 / HBM_PEAK_GBS, 4),
                   "units_per_s": round(ww.units / t_w, 1), "dense_TFLOPs": round(wfl / t_w / 1e12, 1),
                   "err_y": orc.rel_err(wy32[:1].float().cpu().numpy(), yr), "err_final": orc.rel_err(wf[:1].cpu().numpy(), fr),
                   "err_rows": 1, "tolerance": 2e-2 if wdtype == "bf16" else 1e-4}
            if wdtype == "bf16":
                row["mfma_frac"] = round(wfl / t_w / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)
                row["stored_y_is_rounded_f32_y"] = stored_ok
                row["mfma_pipe_busy"] = MEASURED_MFMA_PIPE_BUSY.get((wname, ww.batch))
                row["traffic"] = MEASURED_TRAFFIC_BYTES.get((wname, ww.batch))
            else:
                row.update(f32_mfma(wfl, t_w, one_launch or segs > 1))
            rows_out.append(row)
            del wi, call, wy, wf, wy32, yr, fr
            torch.cuda.empty_cache()
        out["workloads"] = rows_out

    # ---- streaming step at batch 4096 ---------------------------------------------------------
    if not args.no_stream_step:
        sw = WORKLOADS["streamed_bf16"]
        del inp, x, Bm, Cm, y, S, ws
        torch.cuda.empty_cache()
        si = make_inputs(sw, seed=0, device="cuda", seqlen=sw.stream_steps)
        state = torch.zeros((sw.batch, sw.nheads, sw.headdim, sw.dstate), dtype=torch.float32, device="cuda")
        xs = [si["x"][:, t].contiguous() for t in range(sw.stream_steps)]
        ds = [si["dt"][:, t].contiguous() for t in range(sw.stream_steps)]
        bs = [si["B"][:, t].contiguous() for t in range(sw.stream_steps)]
        cs = [si["C"][:, t].contiguous() for t in range(sw.stream_steps)]
        ys = torch.empty_like(xs[0])
        for t in range(8):
            ssd.ssd_step(state, xs[t], ds[t], si["A"], bs[t], cs[t], si["D"], out=ys)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for t in range(sw.stream_steps):
            ssd.ssd_step(state, xs[t], ds[t], si["A"], bs[t], cs[t], si["D"], out=ys)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / sw.stream_steps
        gbs = step_bytes(sw) / (us * 1e-6) / 1e9
        out["stream_step"] = {"batch": sw.batch, "steps": sw.stream_steps, "us_per_step": round(us, 2),
                              "alg_bytes": step_bytes(sw), "GBps": round(gbs, 1),
                              "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)}
        # a 1 000-step loop of the same update (the 64 steps' inputs in turn), an event around every step: mean and median
        n_loop = 1000
        le = [torch.cuda.Event(enable_timing=True) for _ in range(n_loop + 1)]
        torch.cuda.synchronize()
        le[0].record()
        for t in range(n_loop):
            k = t % sw.stream_steps
            ssd.ssd_step(state, xs[k], ds[k], si["A"], bs[k], cs[k], si["D"], out=ys)
            le[t + 1].record()
        torch.cuda.synchronize()
        per_step = sorted(le[t].elapsed_time(le[t + 1]) * 1e3 for t in range(n_loop))
        us_loop = le[0].elapsed_time(le[n_loop]) * 1e3 / n_loop
        out["stream_step"]["loop_1000"] = {"us_per_step": round(us_loop, 2), "us_median": round(per_step[n_loop // 2], 2),
                                           "GBps": round(step_bytes(sw) / (us_loop * 1e-6) / 1e9, 1),
                                           "hbm_frac": round(step_bytes(sw) / (us_loop * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
        del le
        # the same 64 steps as ONE launch (state in registers between the steps): per-step latency, and the
        # traffic of the launch = state in and out once plus the 64 steps' inputs and outputs
        xs64, ds64 = si["x"].contiguous(), si["dt"].contiguous()
        bs64, cs64 = si["B"].contiguous(), si["C"].contiguous()
        ys64 = torch.empty_like(xs64)
        for _ in range(3):
            ssd.ssd_steps(state, xs64, ds64, si["A"], bs64, cs64, si["D"], out=ys64)
        reps = 10
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            ssd.ssd_steps(state, xs64, ds64, si["A"], bs64, cs64, si["D"], out=ys64)
        e1.record()
        torch.cuda.synchronize()
        us64 = e0.elapsed_time(e1) * 1e3 / reps
        bytes64 = 8 * sw.batch * sw.nheads * sw.headdim * sw.dstate + sw.stream_steps * (
            step_bytes(sw) - 8 * sw.batch * sw.nheads * sw.headdim * sw.dstate)
        out["stream_steps_one_launch"] = {"batch": sw.batch, "steps": sw.stream_steps,
                                          "us_per_launch": round(us64, 1),
                                          "us_per_step": round(us64 / sw.stream_steps, 2), "alg_bytes": bytes64,
                                          "GBps": round(bytes64 / (us64 * 1e-6) / 1e9, 1)}

    # ---- the reference's own benchmark cases for this path ------------------------------------
    # benchmark_results/bench_20260112_070055.json:5-41 lists mamba2_forward_train, mamba2_fwd_bwd_train,
    # mamba2_infer_prefill and mamba2_infer_step at batch 4, seq_len 4096 (1 for the step), BFloat16, in the schema of
    # benchmarks/src/results.rs:8-29; they timed a whole Mamba-2 block of unrecorded sizes.  Here the mamba2_* rows
    # time this library's block (Mamba2Block: projections, conv + SiLU, scan, gated RMSNorm) with the policy head
    # sizes and d_model = nheads * headdim, printed in each row's config; the ssd_scan_* rows are the scan op alone.
    # Protocol as in benchmarks/src/main.rs:140-200: warm-up calls, sync, timed calls, sync, mean per call; the
    # step row = prefill once, then timed single steps.
    if not args.no_reference_suite:
        from trading_bot_0_amd import Mamba2Block
        rw = WORKLOADS["policy_bf16"].with_batch(4)
        ri = make_inputs(rw, seed=0, device="cuda", seqlen=4096)
        rf = ssd.PreparedChunkScan(ri["x"], ri["dt"], ri["A"], ri["B"], ri["C"], ri["D"], chunk=rw.chunk)
        spin(rf, torch, 0.1)
        t_fwd = event_time_steps(rf, 200, torch)[0] * 1e3
        rstate = rf.final.clone()
        step_args = [ri[k][:, 0].contiguous() for k in ("x", "dt", "B", "C")]
        ry = torch.empty_like(step_args[0])

        def rstep():
            ssd.ssd_step(rstate, step_args[0], step_args[1], ri["A"], step_args[2], step_args[3], ri["D"], out=ry)

        spin(rstep, torch, 0.1)
        t_step = event_time_steps(rstep, 500, torch)[0] * 1e3
        cfg = {"batch": 4, "seq_len": 4096, "dtype": "BFloat16"}
        sizes = {"nheads": rw.nheads, "headdim": rw.headdim, "dstate": rw.dstate, "ngroups": rw.ngroups, "chunk": rw.chunk}
        suite = [{"name": "ssd_scan_forward", "time_ms": t_fwd, "config": {**cfg, **sizes}},
                 {"name": "ssd_scan_step", "time_ms": t_step, "config": {"batch": 4, "seq_len": 1, "dtype": "BFloat16", **sizes}}]
        if not args.no_backward:
            rdy = torch.randn_like(ri["x"])
            rws = torch.empty(ssd.backward_workspace_bytes(4, 4096, rw.nheads, rw.headdim, rw.dstate, rw.ngroups, rw.chunk),
                              dtype=torch.uint8, device="cuda")

            def scan_fwd_bwd():
                rf()
                ssd.ssd_chunk_scan_backward(ri["x"], ri["dt"], ri["A"], ri["B"], ri["C"], ri["D"], rdy, chunk=rw.chunk,
                                            workspace=rws)

            spin(scan_fwd_bwd, torch, 0.1)
            suite.append({"name": "ssd_scan_fwd_bwd", "time_ms": event_time_steps(scan_fwd_bwd, 50, torch)[0] * 1e3,
                          "config": {**cfg, **sizes}})
            del rdy, rws
        if not args.no_block:
            rblk = Mamba2Block(d_model=rw.nheads * rw.headdim, nheads=rw.nheads, headdim=rw.headdim, dstate=rw.dstate,
                               ngroups=rw.ngroups, chunk=rw.chunk)
            bsizes = {"d_model": rblk.d_model, "d_conv": rblk.d_conv, **sizes}
            ru = torch.randn(4, 4096, rblk.d_model, device="cuda").to(torch.bfloat16)
            with torch.no_grad():
                spin(lambda: rblk.forward(ru), torch, 0.1)
                t_train = event_time_steps(lambda: rblk.forward(ru), 100, torch)[0] * 1e3
                # prefill: the same forward that also leaves the conv and SSM state of every stream behind
                rst = rblk.new_state(4)
                spin(lambda: rblk.forward(ru, state=rst), torch, 0.1)
                t_prefill = event_time_steps(lambda: rblk.forward(ru, state=rst), 100, torch)[0] * 1e3
                ru_t = ru[:, 0].contiguous()
                spin(lambda: rblk.step(ru_t, rst), torch, 0.1)
                t_bstep = event_time_steps(lambda: rblk.step(ru_t, rst), 200, torch)[0] * 1e3
                spin(lambda: rblk.step(ru_t, rst, fused=False), torch, 0.1)
                t_bstep_stages = event_time_steps(lambda: rblk.step(ru_t, rst, fused=False), 100, torch)[0] * 1e3
                gstep = rblk.graphed_step(rst)
                spin(lambda: gstep(ru_t), torch, 0.1)
                t_gstep = event_time_steps(lambda: gstep(ru_t), 200, torch)[0] * 1e3
            suite += [{"name": "mamba2_forward_train", "time_ms": t_train, "config": {**cfg, **bsizes}},
                      {"name": "mamba2_infer_prefill", "time_ms": t_prefill, "config": {**cfg, **bsizes}},
                      {"name": "mamba2_infer_step", "time_ms": t_bstep,
                       "config": {"batch": 4, "seq_len": 1, "dtype": "BFloat16", "launches": "one (ssd_block_step_fwd)", **bsizes}},
                      {"name": "mamba2_infer_step_stage_kernels", "time_ms": t_bstep_stages,
                       "config": {"batch": 4, "seq_len": 1, "dtype": "BFloat16",
                                  "launches": "five stage kernels, two library products", **bsizes}},
                      {"name": "mamba2_infer_step_graph", "time_ms": t_gstep,
                       "config": {"batch": 4, "seq_len": 1, "dtype": "BFloat16", "captured": "one HIP graph per step", **bsizes}}]
            if hasattr(rblk, "backward") and not args.no_backward:
                rdo = torch.randn_like(ru)

                def block_fwd_bwd():
                    _, ctx = rblk.forward(ru, save_for_backward=True)
                    rblk.backward(ctx, rdo)

                spin(block_fwd_bwd, torch, 0.1)
                suite.append({"name": "mamba2_fwd_bwd_train", "time_ms": event_time_steps(block_fwd_bwd, 50, torch)[0] * 1e3,
                              "config": {**cfg, **bsizes}})
            del ru, rblk, rst
        out["reference_suite"] = suite

    # ---- the Mamba-2 block around the scan: its stages through their own entry points, and the whole block ----
    if not args.no_block:
        from trading_bot_0_amd import Mamba2Block, block_post, block_pre, block_proj
        bw = WORKLOADS["policy_bf16"]
        blk = Mamba2Block(d_model=bw.nheads * bw.headdim, nheads=bw.nheads, headdim=bw.headdim, dstate=bw.dstate,
                          ngroups=bw.ngroups, chunk=bw.chunk)
        u = torch.randn(bw.batch, bw.seqlen, blk.d_model, device="cuda").to(torch.bfloat16)
        zx = blk._project(u, blk.in_proj, pad_rows=True)  # as in Mamba2Block.forward
        xs_, bs_, cs_, ds_ = block_pre(zx, blk.conv_w, blk.conv_b, blk.dt_bias, blk.H, blk.P, blk.N, blk.G)
        ys_, _ = ssd.ssd_chunk_scan(xs_, ds_, blk.A, bs_, cs_, blk.D, chunk=bw.chunk, return_final_states=False)

        def timed(fn, n=20):
            for _ in range(3):
                fn()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            a.record()
            for _ in range(n):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n

        e = 2
        pre_bytes = e * bw.batch * bw.seqlen * (2 * (blk.conv_dim + blk.H))          # reads x|B|C|dt, writes them
        post_bytes = e * bw.batch * bw.seqlen * 3 * blk.d_inner                     # reads y and z, writes out
        t_pre = timed(lambda: block_pre(zx, blk.conv_w, blk.conv_b, blk.dt_bias, blk.H, blk.P, blk.N, blk.G))
        t_post = timed(lambda: block_post(ys_, zx, blk.norm_w, blk.H, blk.P, blk.N, blk.G))
        t_block = timed(lambda: blk.forward(u), n=10)
        w_in, w_out = blk.in_proj.to(u.dtype).contiguous(), blk.out_proj.to(u.dtype).contiguous()
        yn = block_post(ys_, zx, blk.norm_w, blk.H, blk.P, blk.N, blk.G)
        rows = bw.batch * bw.seqlen
        in_bytes = e * rows * (blk.d_model + w_in.shape[0])
        out_bytes = e * rows * (blk.d_inner + blk.d_model)
        t_in = timed(lambda: block_proj(u, w_in, pad_rows=True))   # as the block calls it: rows of whole 128-byte lines
        t_in_dense = timed(lambda: block_proj(u, w_in))
        t_out = timed(lambda: block_proj(yn, w_out))
        from trading_bot_0_amd import block_post_proj
        t_post_out = timed(lambda: block_post_proj(ys_, zx, blk.norm_w, w_out, blk.H, blk.P, blk.N, blk.G))
        post_out_bytes = e * rows * (2 * blk.d_inner + blk.d_model)               # reads y and z, writes out
        t_in_blas = timed(lambda: torch.matmul(u, w_in.t()))
        t_out_blas = timed(lambda: torch.matmul(yn, w_out.t()))
        out["mamba2_block"] = {"d_model": blk.d_model, "ms": round(t_block, 4),
                               "parity": "against this repository's float64 block oracle (tests/test_oracle_block.py pins it); "
                                         "the reference holds no source or vector of this layer: unpinned by the reference",
                               "in_proj_ms": round(t_in, 4), "in_proj_GBps": round(in_bytes / t_in / 1e6, 1),
                               "in_proj_dense_rows_ms": round(t_in_dense, 4), "in_proj_blas_ms": round(t_in_blas, 4),
                               "pre_ms": round(t_pre, 4), "pre_GBps": round(pre_bytes / t_pre / 1e6, 1),
                               "post_ms": round(t_post, 4), "post_GBps": round(post_bytes / t_post / 1e6, 1),
                               "out_proj_ms": round(t_out, 4), "out_proj_GBps": round(out_bytes / t_out / 1e6, 1),
                               "out_proj_blas_ms": round(t_out_blas, 4),
                               "post_out_proj_fused_ms": round(t_post_out, 4),
                               "post_out_proj_fused_GBps": round(post_out_bytes / t_post_out / 1e6, 1)}
        if hasattr(blk, "backward") and not args.no_backward:
            # forward with what the backward needs kept, then the block's backward (stage kernels of this library,
            # the scan's backward, four GEMMs)
            del xs_, bs_, cs_, ds_, ys_, yn
            dout = torch.randn_like(u)

            def fwd_bwd():
                _, ctx = blk.forward(u, save_for_backward=True)
                blk.backward(ctx, dout)

            out["mamba2_block"]["fwd_bwd_ms"] = round(timed(fwd_bwd, n=5), 4)
            del dout
        del u, zx, blk

    # ---- CPU baseline: the same arithmetic on this box's host cores, on bounded batch slices -----------------
    # (1) the plain-C sequential recurrence (float32, OpenMP) -- the headline cpu_baseline;
    # (2) the chunked algorithm in ATen CPU float32 ops, the backend the reference runs on a CPU device
    #     (trading_bots/src/torch/model/trading_model.rs:140-146), at one intra-op thread (the reference's default
    #     policy, trading_bots/src/torch/train/trainer.rs:635-646) and at every core this process may use.
    if not args.no_cpu_baseline:
        import numpy as np
        from oracle import c_oracle
        from oracle.ssd_torch_cpu import ssd_chunked_torch
        host_cores = os.cpu_count() or 1
        try:
            usable = len(os.sched_getaffinity(0))
        except AttributeError:
            usable = host_cores
        threads = min(16, usable)
        cpu = make_inputs(w.with_batch(max(threads, 16)), seed=0, device="cpu")
        a = {k: (None if v is None else v.float().numpy()) for k, v in cpu.items()}

        def run(nb):
            t0 = time.perf_counter()
            c_oracle.ssd_sequential_c(a["x"][:nb], a["dt"][:nb], a["A"], a["B"][:nb], a["C"][:nb], a["D"],
                                      None if a["init"] is None else a["init"][:nb], dtype=np.float32,
                                      nthreads=threads)
            return time.perf_counter() - t0

        nb0 = a["x"].shape[0]
        t_probe = run(nb0)
        budget = args.cpu_seconds / 3.0
        reps = max(1, min(int(budget / max(t_probe, 1e-3)), 200))
        t0 = time.perf_counter()
        for _ in range(reps):
            run(nb0)
        t_cpu = (time.perf_counter() - t0) / reps

        tc = {k: (None if v is None else v.float()) for k, v in cpu.items()}

        def torch_leg(nthreads, nb):
            prev = torch.get_num_threads()
            torch.set_num_threads(nthreads)
            try:
                def once():
                    t0 = time.perf_counter()
                    with torch.no_grad():
                        ssd_chunked_torch(tc["x"][:nb], tc["dt"][:nb], tc["A"], tc["B"][:nb], tc["C"][:nb], tc["D"],
                                          None if tc["init"] is None else tc["init"][:nb], chunk=w.chunk)
                    return time.perf_counter() - t0
                once()   # the first call pays ATen's one-time set-up
                probe = once()
                n = max(1, min(int(budget / max(probe, 1e-3)), 50))
                t = sum(once() for _ in range(n)) / n
            finally:
                torch.set_num_threads(prev)
            return {"value": nb * w.seqlen / t, "unit": "timesteps*batch/s", "threads": nthreads,
                    "sample": f"batch slice {nb} of {w.batch} at full seqlen, {n} repetitions, {t * 1e3:.1f} ms each"}

        # slices sized so that a call stays around a second: the chunked form materialises [B,H,nc,Q,Q] score tiles
        per_row = w.seqlen * w.nheads * w.headdim
        nb_small = max(1, min(nb0, (1 << 22) // per_row))
        out["cpu_baseline"] = {"value": nb0 * w.seqlen / t_cpu, "unit": "timesteps*batch/s", "cores": threads,
                               "kind": "port",
                               "sample": f"plain-C sequential recurrence, float32, OpenMP {threads} threads, "
                                         f"batch slice {nb0} of {w.batch} at full seqlen, {reps} repetitions, "
                                         f"{t_cpu * 1e3:.1f} ms each",
                               "host_cores": host_cores, "usable_cores": usable, "cpu_model": cpu_model_name(),
                               "torch_cpu_chunked_f32_1_thread": torch_leg(1, nb_small),
                               "torch_cpu_chunked_f32_all_cores": torch_leg(usable, min(nb0, max(nb_small, 4 * nb_small)))}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
