"""ctypes loader for the plain-C oracle (oracle/ssd_oracle.c).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import c_int, c_int64, c_void_p
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
LIB_PATH = ORACLE_DIR / "libssd_oracle.so"


def build() -> Path:
    subprocess.run(["make", "-C", str(ORACLE_DIR), "-B", "libssd_oracle.so"], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(str(LIB_PATH))
        seq_args = [c_int64] * 6 + [c_void_p] * 9 + [c_int]
        for name in ("ssd_oracle_seq_f64", "ssd_oracle_seq_f32"):
            getattr(lib, name).argtypes = seq_args
            getattr(lib, name).restype = c_int
        lib.ssd_oracle_step_f64.argtypes = [c_int64] * 5 + [c_void_p] * 8
        lib.ssd_oracle_step_f64.restype = c_int
        _lib = lib
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def ssd_sequential_c(x, dt, A, Bm, Cm, D=None, init=None, dtype=np.float64, nthreads=8):
    """Sequential recurrence in C; same contract as ssd_oracle.ssd_sequential."""
    lib = load()
    fn = lib.ssd_oracle_seq_f64 if dtype == np.float64 else lib.ssd_oracle_seq_f32
    c = lambda a: None if a is None else np.ascontiguousarray(a, dtype=dtype)
    x, dt, A, Bm, Cm, D, init = map(c, (x, dt, A, Bm, Cm, D, init))
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    y = np.empty((Bsz, L, H, P), dtype)
    final = np.empty((Bsz, H, P, N), dtype)
    rc = fn(Bsz, L, H, P, N, G, _p(x), _p(dt), _p(A), _p(Bm), _p(Cm), _p(D), _p(init), _p(y), _p(final), nthreads)
    if rc != 0:
        raise RuntimeError(f"C oracle failed with code {rc}")
    return y, final


def ssd_step_c(state, x, dt, A, Bm, Cm, D=None):
    """One update in C (float64).  Returns (y, new_state); `state` is not modified."""
    lib = load()
    c = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.float64)
    st = np.array(state, dtype=np.float64, order="C")
    x, dt, A, Bm, Cm, D = map(c, (x, dt, A, Bm, Cm, D))
    Bsz, H, P, N = st.shape
    y = np.empty((Bsz, H, P), np.float64)
    rc = lib.ssd_oracle_step_f64(Bsz, H, P, N, Bm.shape[1], _p(st), _p(x), _p(dt), _p(A), _p(Bm), _p(Cm), _p(D), _p(y))
    if rc != 0:
        raise RuntimeError(f"C oracle step failed with code {rc}")
    return y, st
