"""Shared helpers of the GPU parity tests: moving synthetic inputs to the device, handing the
oracle exactly the values the kernels see, and the parity metric."""
import numpy as np
import torch

from oracle import c_oracle
from oracle import ssd_oracle as orc

TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}   # max|out-ref| / rms(ref), per the task's bar
ORACLE_THREADS = 16


def np64(t):
    """A tensor's exact values as float64 (bf16 inputs are already rounded once)."""
    return None if t is None else t.detach().float().cpu().numpy().astype(np.float64)


def to_dev(inp, device="cuda"):
    return {k: (None if v is None else v.to(device)) for k, v in inp.items()}


def oracle_scan(inp, with_D=True):
    """Sequential float64 ground truth (C oracle) on the inputs' exact values."""
    return c_oracle.ssd_sequential_c(np64(inp["x"]), np64(inp["dt"]), np64(inp["A"]), np64(inp["B"]),
                                     np64(inp["C"]), np64(inp["D"]) if with_D else None, np64(inp["init"]),
                                     nthreads=ORACLE_THREADS)


def rel_err(out, ref):
    if isinstance(out, torch.Tensor):
        out = out.detach().float().cpu().numpy()
    return orc.rel_err(out, ref)


def assert_close(out, ref, dtype, what):
    e = rel_err(out, ref)
    assert np.isfinite(e) and e <= TOL[dtype], f"{what}: max|err|/rms = {e:.3e} > {TOL[dtype]:.0e}"
    return e
