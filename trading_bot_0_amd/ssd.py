"""Host-side operator interface of the SSD path: the functions a model calls, over torch-ROCm
tensors, bound to libssd_hip.so through its C ABI with ctypes.

The shape of this module mirrors how the reference wraps a custom kernel
(`trading_bots/src/torch/fa4.rs:28-47` public op functions, `:145-191` validate-then-call with a
message per violated precondition): `ssd_chunk_scan(...) -> (y, final_states)` is the batched
op that sits in the temporal-encoder slot (`trading_bots/src/torch/model/trading_model.rs:589-606`)
and `ssd_step(state, ...) -> y` is the per-bar streaming update
(`trading_bots/src/torch/model/stream/live.rs:228-244`).  Tensors stay owned by the caller; raw
device pointers are `Tensor.data_ptr()` exactly as the Rust side would pass
(`vendor/torch-sys-0.25.0/src/lib.rs:38`).  torch is used for device memory and the current
stream only -- there is no fallback: without the built library every call raises.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import POINTER, Structure, byref, c_char_p, c_int, c_int64, c_size_t, c_void_p
from typing import Optional, Tuple

import torch

from ._build import LIB_PATH

SSD_DTYPE_F32 = 0
SSD_DTYPE_BF16 = 1
SSD_DTYPE_BF16_Y32 = 2

EXPORTED_SYMBOLS = (
    "ssd_version",
    "ssd_get_and_reset_last_err",
    "ssd_workspace_bytes",
    "ssd_chunk_scan_fwd",
    "ssd_chunk_scan_reset_fwd",
    "ssd_chunk_cumsum_fwd",
    "ssd_chunk_state_fwd",
    "ssd_state_passing_fwd",
    "ssd_chunk_state_passing_fwd",
    "ssd_chunk_scan_onepass_fwd",
    "ssd_chunk_scan_is_onepass",
    "ssd_chunk_scan_segments",
    "ssd_chunk_scan_stage_fwd",
    "ssd_step_fwd",
    "ssd_steps_fwd",
    "ssd_block_pre_fwd",
    "ssd_block_post_fwd",
    "ssd_block_proj_fwd",
    "ssd_chunk_scan_bwd_workspace_bytes",
    "ssd_chunk_scan_bwd",
    "ssd_chunk_scan_noalloc_fwd",
    "ssd_block_pre_reset_fwd",
    "ssd_block_bwd_workspace_bytes",
    "ssd_block_post_bwd",
    "ssd_block_post_bwd_yn",
    "ssd_block_pre_bwd",
    "ssd_block_post_proj_fwd",
    "ssd_block_step_fwd",
)


class SsdError(RuntimeError):
    """A call into libssd_hip returned non-zero; carries the library's message and code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[ssd error {code}] {message}")
        self.code = code
        self.message = message


class SsdDims(Structure):
    _fields_ = [(n, c_int64) for n in ("batch", "seqlen", "nheads", "headdim", "dstate", "ngroups", "chunk")]


class SsdStepDims(Structure):
    _fields_ = [(n, c_int64) for n in ("batch", "nheads", "headdim", "dstate", "ngroups")]


_lib = None
_lib_lock = threading.Lock()
_libc = ctypes.CDLL(None)
_libc.free.argtypes = [c_void_p]
_libc.free.restype = None


def load_library() -> ctypes.CDLL:
    """Loads libssd_hip.so (after torch, so both share one HIP runtime).  Raises if it is not
    built: the HIP path is the only path."""
    global _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "from the repository root (needs hipcc). There is no CPU fallback."
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        P = c_void_p
        lib.ssd_version.argtypes = []
        lib.ssd_version.restype = c_int
        lib.ssd_get_and_reset_last_err.argtypes = []
        lib.ssd_get_and_reset_last_err.restype = c_void_p
        lib.ssd_workspace_bytes.argtypes = [POINTER(SsdDims), POINTER(c_size_t)]
        lib.ssd_chunk_scan_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P, P, P, P, P, P, P, c_size_t, P]
        lib.ssd_chunk_cumsum_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P]
        lib.ssd_chunk_state_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P, P]
        lib.ssd_state_passing_fwd.argtypes = [POINTER(SsdDims), P, P, P, P, P, P]
        lib.ssd_chunk_state_passing_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P, P, P, P]
        lib.ssd_chunk_scan_onepass_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P, P, P, P, P, P, P, P]
        lib.ssd_chunk_scan_reset_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P, P, P, P, P, P, P, P, c_size_t, P]
        lib.ssd_chunk_scan_noalloc_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P, P, P, P, P, P, P, P]
        lib.ssd_chunk_scan_is_onepass.argtypes = [POINTER(SsdDims), c_int, POINTER(c_int)]
        lib.ssd_chunk_scan_segments.argtypes = [POINTER(SsdDims), c_int, POINTER(c_int)]
        lib.ssd_chunk_scan_stage_fwd.argtypes = [POINTER(SsdDims), c_int, P, P, P, P, P, P, P, P]
        lib.ssd_step_fwd.argtypes = [POINTER(SsdStepDims), c_int, P, P, P, P, P, P, P, P, P]
        lib.ssd_steps_fwd.argtypes = [POINTER(SsdStepDims), c_int64, c_int, P, P, P, P, P, P, P, P, P, P]
        lib.ssd_chunk_scan_bwd_workspace_bytes.argtypes = [POINTER(SsdDims), c_int, POINTER(c_size_t)]
        lib.ssd_chunk_scan_bwd.argtypes = [POINTER(SsdDims), c_int] + [P] * 18 + [c_size_t, P]
        for name in EXPORTED_SYMBOLS[2:]:
            getattr(lib, name).restype = c_int   # (argument types of the block stages: block.py)
        _lib = lib
        return lib


def last_error(lib: Optional[ctypes.CDLL] = None) -> Optional[str]:
    """Fetches and clears this thread's error message (freed here, as the Rust side does with
    libc::free, `trading_bots/src/torch/cuda/graph.rs:107-119`)."""
    lib = lib or load_library()
    ptr = lib.ssd_get_and_reset_last_err()
    if not ptr:
        return None
    msg = ctypes.string_at(ptr).decode("utf-8", "replace")
    _libc.free(ptr)
    return msg


def _check(lib, rc: int) -> None:
    if rc != 0:
        raise SsdError(rc, last_error(lib) or "unknown error")


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return SSD_DTYPE_F32
    if t.dtype == torch.bfloat16:
        return SSD_DTYPE_BF16
    raise ValueError(f"SSD tensors must be float32 or bfloat16, got {t.dtype}")


def _out_code(x: torch.Tensor, y_dtype: Optional[torch.dtype]):
    """dtype code of a call whose y is `y_dtype` (default: x's dtype)."""
    code = _dtype_code(x)
    if y_dtype is None or y_dtype == x.dtype:
        return code, x.dtype
    if x.dtype == torch.bfloat16 and y_dtype == torch.float32:
        return SSD_DTYPE_BF16_Y32, y_dtype
    raise ValueError(f"SSD y_dtype {y_dtype} is not available for {x.dtype} inputs")


def _require(t: torch.Tensor, name: str, shape, dtype) -> None:
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"SSD {name} must be a tensor")
    if not t.is_cuda:
        raise ValueError(f"SSD {name} must be on the GPU, got {t.device}")
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"SSD {name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    if t.dtype != dtype:
        raise ValueError(f"SSD {name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"SSD {name} must be contiguous")


def _reset_mask(reset, dims: "SsdDims"):
    """[B,L] uint8 (bool accepted) or None."""
    if reset is None:
        return None
    if reset.dtype == torch.bool:
        reset = reset.view(torch.uint8)
    _require(reset, "reset", (dims.batch, dims.seqlen), torch.uint8)
    return reset


def _scan_dims(x, Bm, chunk) -> SsdDims:
    if x.dim() != 4:
        raise ValueError(f"SSD x must be rank-4 [batch, seqlen, nheads, headdim], got {tuple(x.shape)}")
    if Bm.dim() != 4:
        raise ValueError(f"SSD B must be rank-4 [batch, seqlen, ngroups, dstate], got {tuple(Bm.shape)}")
    Bsz, L, H, P = x.shape
    return SsdDims(Bsz, L, H, P, Bm.shape[3], Bm.shape[2], int(chunk))


def num_chunks(seqlen: int, chunk: int) -> int:
    return -(-seqlen // chunk)


def workspace_bytes(batch, seqlen, nheads, headdim, dstate, ngroups, chunk) -> int:
    lib = load_library()
    out = c_size_t(0)
    _check(lib, lib.ssd_workspace_bytes(byref(SsdDims(batch, seqlen, nheads, headdim, dstate, ngroups, chunk)),
                                        byref(out)))
    return out.value


def _validate_scan_inputs(x, dt, A, Bm, Cm, D, initial_states, dims: SsdDims):
    Bsz, L, H, P, N, G = dims.batch, dims.seqlen, dims.nheads, dims.headdim, dims.dstate, dims.ngroups
    dtype = x.dtype
    _dtype_code(x)
    _require(x, "x", (Bsz, L, H, P), dtype)
    if dt is not None:
        _require(dt, "dt", (Bsz, L, H), dtype)
    if A is not None:
        _require(A, "A", (H,), torch.float32)
    _require(Bm, "B", (Bsz, L, G, N), dtype)
    if Cm is not None:
        _require(Cm, "C", (Bsz, L, G, N), dtype)
    if D is not None:
        _require(D, "D", (H,), torch.float32)
    if initial_states is not None:
        _require(initial_states, "initial_states", (Bsz, H, P, N), torch.float32)
    for name, t in (("dt", dt), ("A", A), ("B", Bm), ("C", Cm), ("D", D), ("initial_states", initial_states)):
        if t is not None and t.device != x.device:
            raise ValueError(f"SSD {name} must be on {x.device}, got {t.device}")


def ssd_chunk_scan(
    x: torch.Tensor,
    dt: torch.Tensor,
    A: torch.Tensor,
    Bm: torch.Tensor,
    Cm: torch.Tensor,
    D: Optional[torch.Tensor] = None,
    chunk: int = 128,
    initial_states: Optional[torch.Tensor] = None,
    return_final_states: bool = True,
    workspace: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    final_out: Optional[torch.Tensor] = None,
    y_dtype: Optional[torch.dtype] = None,
    reset: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """SSD chunk-scan forward.  Returns (y [B,L,H,P] in x's dtype, final_states [B,H,P,N] fp32).
    `reset` [B,L] (uint8 or bool): a non-zero entry restarts that batch row's state from zero before the
    timestep (episode boundaries inside a window).

    `workspace` (uint8, >= workspace_bytes(...)), `out` and `final_out` let a caller that runs
    under stream capture or in a tight loop avoid any allocation.  `y_dtype=torch.float32` with
    bf16 inputs writes y without the output rounding."""
    lib = load_library()
    dims = _scan_dims(x, Bm, chunk)
    _validate_scan_inputs(x, dt, A, Bm, Cm, D, initial_states, dims)
    code, y_dtype = _out_code(x, y_dtype)
    y = torch.empty(x.shape, dtype=y_dtype, device=x.device) if out is None else out
    _require(y, "out", x.shape, y_dtype)
    final = None
    if return_final_states:
        shape = (dims.batch, dims.nheads, dims.headdim, dims.dstate)
        final = torch.empty(shape, dtype=torch.float32, device=x.device) if final_out is None else final_out
        _require(final, "final_out", shape, torch.float32)
    need = c_size_t(0)
    _check(lib, lib.ssd_workspace_bytes(byref(dims), byref(need)))
    if workspace is None:
        workspace = torch.empty(need.value, dtype=torch.uint8, device=x.device)
    elif (not workspace.is_cuda) or workspace.dtype != torch.uint8 or not workspace.is_contiguous():
        raise ValueError("SSD workspace must be a contiguous uint8 GPU tensor")
    reset = _reset_mask(reset, dims)
    rc = lib.ssd_chunk_scan_reset_fwd(byref(dims), code, x.data_ptr(), dt.data_ptr(), A.data_ptr(),
                                      Bm.data_ptr(), Cm.data_ptr(), _ptr(D), _ptr(initial_states), _ptr(reset),
                                      y.data_ptr(), _ptr(final), workspace.data_ptr(), workspace.numel(),
                                      _stream_ptr(x))
    _check(lib, rc)
    return y, final


def ssd_chunk_scan_backward(x, dt, A, Bm, Cm, D, dy, chunk: int = 128, initial_states=None, dfinal_states=None,
                            need_dinitial_states: bool = False, workspace=None, reset=None) -> dict:
    """Gradients of the scan's outputs (y weighted by `dy`, the final state by `dfinal_states`) with respect to
    its inputs; `reset` is the forward's restart mask.  Returns a dict with dx, ddt, dB, dC (input dtype), dA, dD (None without D) and, if asked for,
    dinitial_states (float32)."""
    lib = load_library()
    dims = _scan_dims(x, Bm, chunk)
    _validate_scan_inputs(x, dt, A, Bm, Cm, D, initial_states, dims)
    code = _dtype_code(x)
    _require(dy, "dy", x.shape, x.dtype)
    sshape = (dims.batch, dims.nheads, dims.headdim, dims.dstate)
    if dfinal_states is not None:
        _require(dfinal_states, "dfinal_states", sshape, torch.float32)
    dev = x.device
    out = {"dx": torch.empty_like(x), "ddt": torch.empty_like(dt), "dB": torch.empty_like(Bm), "dC": torch.empty_like(Cm),
           "dA": torch.empty(dims.nheads, dtype=torch.float32, device=dev),
           "dD": None if D is None else torch.empty(dims.nheads, dtype=torch.float32, device=dev),
           "dinitial_states": torch.empty(sshape, dtype=torch.float32, device=dev) if need_dinitial_states else None}
    need = c_size_t(0)
    _check(lib, lib.ssd_chunk_scan_bwd_workspace_bytes(byref(dims), code, byref(need)))
    if workspace is None:
        workspace = torch.empty(need.value, dtype=torch.uint8, device=dev)
    elif (not workspace.is_cuda) or workspace.dtype != torch.uint8 or not workspace.is_contiguous():
        raise ValueError("SSD workspace must be a contiguous uint8 GPU tensor")
    reset = _reset_mask(reset, dims)
    rc = lib.ssd_chunk_scan_bwd(byref(dims), code, x.data_ptr(), dt.data_ptr(), A.data_ptr(), Bm.data_ptr(), Cm.data_ptr(),
                                _ptr(D), _ptr(initial_states), _ptr(reset), dy.data_ptr(), _ptr(dfinal_states),
                                out["dx"].data_ptr(), out["ddt"].data_ptr(), out["dA"].data_ptr(), out["dB"].data_ptr(),
                                out["dC"].data_ptr(), _ptr(out["dD"]), _ptr(out["dinitial_states"]),
                                workspace.data_ptr(), workspace.numel(), _stream_ptr(x))
    _check(lib, rc)
    return out


def backward_workspace_bytes(batch, seqlen, nheads, headdim, dstate, ngroups, chunk, dtype=torch.bfloat16) -> int:
    lib = load_library()
    dims = SsdDims(batch, seqlen, nheads, headdim, dstate, ngroups, chunk)
    need = c_size_t(0)
    code = SSD_DTYPE_F32 if dtype == torch.float32 else SSD_DTYPE_BF16
    _check(lib, lib.ssd_chunk_scan_bwd_workspace_bytes(byref(dims), code, byref(need)))
    return need.value


class PreparedChunkScan:
    """ssd_chunk_scan with everything but the launch done once: shapes validated, outputs and workspace
    allocated, argument pointers fixed.  Calling it launches the forward on the current stream of the
    inputs' device and returns (y, final_states); the tensors it was built from must stay alive and in
    place.  For loops that call the op with the same buffers (benchmarks, graph capture, a serving loop):
    per call it costs one foreign call, where ssd_chunk_scan spends tens of microseconds in Python."""

    def __init__(self, x, dt, A, Bm, Cm, D=None, chunk=128, initial_states=None, return_final_states=True,
                 workspace=None, out=None, final_out=None, y_dtype=None, reset=None):
        self._lib = load_library()
        self._dims = _scan_dims(x, Bm, chunk)
        dims = self._dims
        _validate_scan_inputs(x, dt, A, Bm, Cm, D, initial_states, dims)
        self._code, y_dtype = _out_code(x, y_dtype)
        self.y = torch.empty(x.shape, dtype=y_dtype, device=x.device) if out is None else out
        _require(self.y, "out", x.shape, y_dtype)
        self.final = None
        if return_final_states:
            shape = (dims.batch, dims.nheads, dims.headdim, dims.dstate)
            self.final = torch.empty(shape, dtype=torch.float32, device=x.device) if final_out is None else final_out
            _require(self.final, "final_out", shape, torch.float32)
        need = c_size_t(0)
        _check(self._lib, self._lib.ssd_workspace_bytes(byref(dims), byref(need)))
        if workspace is None:
            workspace = torch.empty(need.value, dtype=torch.uint8, device=x.device)
        elif (not workspace.is_cuda) or workspace.dtype != torch.uint8 or not workspace.is_contiguous():
            raise ValueError("SSD workspace must be a contiguous uint8 GPU tensor")
        reset = _reset_mask(reset, dims)
        self._keep = (x, dt, A, Bm, Cm, D, initial_states, workspace, reset)
        self._device = x.device
        self._args = (x.data_ptr(), dt.data_ptr(), A.data_ptr(), Bm.data_ptr(), Cm.data_ptr(), _ptr(D),
                      _ptr(initial_states), _ptr(reset), self.y.data_ptr(), _ptr(self.final), workspace.data_ptr(),
                      workspace.numel())

    def __call__(self):
        rc = self._lib.ssd_chunk_scan_reset_fwd(byref(self._dims), self._code, *self._args,
                                                torch.cuda.current_stream(self._device).cuda_stream)
        if rc:
            _check(self._lib, rc)
        return self.y, self.final


def chunk_scan_is_onepass(batch, seqlen, nheads, headdim, dstate, ngroups, chunk, dtype=torch.bfloat16) -> bool:
    """Whether ssd_chunk_scan runs this shape as the one-pass kernel (True) or as the staged kernels."""
    lib = load_library()
    dims = SsdDims(batch, seqlen, nheads, headdim, dstate, ngroups, chunk)
    flag = c_int(0)
    code = SSD_DTYPE_BF16 if dtype == torch.bfloat16 else SSD_DTYPE_F32
    _check(lib, lib.ssd_chunk_scan_is_onepass(byref(dims), code, byref(flag)))
    return bool(flag.value)


def chunk_scan_segments(batch, seqlen, nheads, headdim, dstate, ngroups, chunk, dtype=torch.bfloat16) -> int:
    """Into how many segments ssd_chunk_scan cuts the sequences of this shape to run them on the one-pass kernel
    side by side (1 = not cut)."""
    lib = load_library()
    dims = SsdDims(batch, seqlen, nheads, headdim, dstate, ngroups, chunk)
    n = c_int(0)
    code = SSD_DTYPE_BF16 if dtype == torch.bfloat16 else SSD_DTYPE_F32
    _check(lib, lib.ssd_chunk_scan_segments(byref(dims), code, byref(n)))
    return n.value


def ssd_chunk_scan_onepass(
    x: torch.Tensor,
    dt: torch.Tensor,
    A: torch.Tensor,
    Bm: torch.Tensor,
    Cm: torch.Tensor,
    D: Optional[torch.Tensor] = None,
    chunk: int = 128,
    initial_states: Optional[torch.Tensor] = None,
    return_final_states: bool = True,
    out: Optional[torch.Tensor] = None,
    final_out: Optional[torch.Tensor] = None,
    y_dtype: Optional[torch.dtype] = None,
    reset: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """The forward as one kernel and one pass over the inputs (no workspace); same results
    as ssd_chunk_scan, which takes this path by itself when the batch is large enough.  Raises
    SsdError(unsupported) for shapes the one-pass kernel does not cover."""
    lib = load_library()
    dims = _scan_dims(x, Bm, chunk)
    _validate_scan_inputs(x, dt, A, Bm, Cm, D, initial_states, dims)
    code, y_dtype = _out_code(x, y_dtype)
    y = torch.empty(x.shape, dtype=y_dtype, device=x.device) if out is None else out
    _require(y, "out", x.shape, y_dtype)
    final = None
    if return_final_states:
        shape = (dims.batch, dims.nheads, dims.headdim, dims.dstate)
        final = torch.empty(shape, dtype=torch.float32, device=x.device) if final_out is None else final_out
        _require(final, "final_out", shape, torch.float32)
    reset = _reset_mask(reset, dims)
    rc = lib.ssd_chunk_scan_onepass_fwd(byref(dims), code, x.data_ptr(), dt.data_ptr(), A.data_ptr(),
                                        Bm.data_ptr(), Cm.data_ptr(), _ptr(D), _ptr(initial_states), _ptr(reset),
                                        y.data_ptr(), _ptr(final), _stream_ptr(x))
    _check(lib, rc)
    return y, final


# ---- per-stage entry points (testing / profiling) ----------------------------------------

def chunk_cumsum(dt: torch.Tensor, A: torch.Tensor, chunk: int) -> torch.Tensor:
    """Stage 1 -> dtcs [B,H,nc,4,Q] float32: log2(e) * cumulative dt*A as (hi, lo), dt, and the
    stage-2 weight exp(cs[Q-1] - cs[l]) * dt[l]."""
    lib = load_library()
    if dt.dim() != 3:
        raise ValueError(f"SSD dt must be rank-3 [batch, seqlen, nheads], got {tuple(dt.shape)}")
    Bsz, L, H = dt.shape
    _require(dt, "dt", (Bsz, L, H), dt.dtype)
    _require(A, "A", (H,), torch.float32)
    nc = num_chunks(L, chunk)
    dtcs = torch.empty((Bsz, H, nc, 4, chunk), dtype=torch.float32, device=dt.device)
    dims = SsdDims(Bsz, L, H, 32, 64, 1, int(chunk))  # P, N, G do not enter stage 1
    _check(lib, lib.ssd_chunk_cumsum_fwd(byref(dims), _dtype_code(dt), dt.data_ptr(), A.data_ptr(),
                                         dtcs.data_ptr(), _stream_ptr(dt)))
    return dtcs


def _require_dtcs(dtcs, dims: SsdDims):
    nc = num_chunks(dims.seqlen, dims.chunk)
    _require(dtcs, "dtcs", (dims.batch, dims.nheads, nc, 4, dims.chunk), torch.float32)
    return nc


def chunk_state(x, Bm, dtcs):
    """Stage 2 -> chunk states [B,nc,H,P,N] float32."""
    lib = load_library()
    dims = _scan_dims(x, Bm, dtcs.shape[-1])
    _validate_scan_inputs(x, None, None, Bm, None, None, None, dims)
    nc = _require_dtcs(dtcs, dims)
    S = torch.empty((dims.batch, nc, dims.nheads, dims.headdim, dims.dstate), dtype=torch.float32, device=x.device)
    _check(lib, lib.ssd_chunk_state_fwd(byref(dims), _dtype_code(x), x.data_ptr(), Bm.data_ptr(),
                                        dtcs.data_ptr(), S.data_ptr(), _stream_ptr(x)))
    return S


def chunk_state_passing(x, Bm, dtcs, initial_states=None):
    """Stages 2+3 in one pass -> (prev_states [B,nc,H,P,N], final_states [B,H,P,N])."""
    lib = load_library()
    dims = _scan_dims(x, Bm, dtcs.shape[-1])
    _validate_scan_inputs(x, None, None, Bm, None, None, initial_states, dims)
    nc = _require_dtcs(dtcs, dims)
    prev = torch.empty((dims.batch, nc, dims.nheads, dims.headdim, dims.dstate), dtype=torch.float32, device=x.device)
    final = torch.empty((dims.batch, dims.nheads, dims.headdim, dims.dstate), dtype=torch.float32, device=x.device)
    _check(lib, lib.ssd_chunk_state_passing_fwd(byref(dims), _dtype_code(x), x.data_ptr(), Bm.data_ptr(),
                                                dtcs.data_ptr(), _ptr(initial_states), prev.data_ptr(),
                                                final.data_ptr(), _stream_ptr(x)))
    return prev, final


def state_passing(states, dtcs, initial_states=None, in_place: bool = False):
    """Stage 3 -> (prev_states [B,nc,H,P,N], final_states [B,H,P,N])."""
    lib = load_library()
    if states.dim() != 5:
        raise ValueError("SSD chunk states must be rank-5 [batch, nchunks, nheads, headdim, dstate]")
    Bsz, nc, H, P, N = states.shape
    chunk = dtcs.shape[-1]
    _require(states, "chunk_states", (Bsz, nc, H, P, N), torch.float32)
    _require(dtcs, "dtcs", (Bsz, H, nc, 4, chunk), torch.float32)
    if initial_states is not None:
        _require(initial_states, "initial_states", (Bsz, H, P, N), torch.float32)
    prev = states if in_place else torch.empty_like(states)
    final = torch.empty((Bsz, H, P, N), dtype=torch.float32, device=states.device)
    dims = SsdDims(Bsz, nc * chunk, H, P, N, 1, int(chunk))
    _check(lib, lib.ssd_state_passing_fwd(byref(dims), states.data_ptr(), dtcs.data_ptr(), _ptr(initial_states),
                                          prev.data_ptr(), final.data_ptr(), _stream_ptr(states)))
    return prev, final


def chunk_scan_stage(x, Bm, Cm, dtcs, prev_states, D=None, y_dtype=None):
    """Stage 4 -> y [B,L,H,P]."""
    lib = load_library()
    dims = _scan_dims(x, Bm, dtcs.shape[-1])
    _validate_scan_inputs(x, None, None, Bm, Cm, D, None, dims)
    nc = _require_dtcs(dtcs, dims)
    _require(prev_states, "prev_states", (dims.batch, nc, dims.nheads, dims.headdim, dims.dstate), torch.float32)
    code, y_dtype = _out_code(x, y_dtype)
    y = torch.empty(x.shape, dtype=y_dtype, device=x.device)
    _check(lib, lib.ssd_chunk_scan_stage_fwd(byref(dims), code, x.data_ptr(), Bm.data_ptr(), Cm.data_ptr(),
                                             dtcs.data_ptr(), prev_states.data_ptr(), _ptr(D), y.data_ptr(),
                                             _stream_ptr(x)))
    return y


def ssd_step(
    state: torch.Tensor,
    x: torch.Tensor,
    dt: torch.Tensor,
    A: torch.Tensor,
    Bm: torch.Tensor,
    Cm: torch.Tensor,
    D: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    y_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """One recurrent update.  `state` [B,H,P,N] fp32 is advanced in place; returns y [B,H,P]
    (x's dtype, or float32 from bf16 inputs with y_dtype=torch.float32)."""
    lib = load_library()
    if state.dim() != 4:
        raise ValueError(f"SSD state must be rank-4 [batch, nheads, headdim, dstate], got {tuple(state.shape)}")
    if Bm.dim() != 3:
        raise ValueError(f"SSD step B must be rank-3 [batch, ngroups, dstate], got {tuple(Bm.shape)}")
    Bsz, H, P, N = state.shape
    G = Bm.shape[1]
    dtype = x.dtype
    _dtype_code(x)
    _require(state, "state", (Bsz, H, P, N), torch.float32)
    _require(x, "x", (Bsz, H, P), dtype)
    _require(dt, "dt", (Bsz, H), dtype)
    _require(A, "A", (H,), torch.float32)
    _require(Bm, "B", (Bsz, G, N), dtype)
    _require(Cm, "C", (Bsz, G, N), dtype)
    if D is not None:
        _require(D, "D", (H,), torch.float32)
    code, y_dtype = _out_code(x, y_dtype)
    y = torch.empty((Bsz, H, P), dtype=y_dtype, device=x.device) if out is None else out
    _require(y, "out", (Bsz, H, P), y_dtype)
    dims = SsdStepDims(Bsz, H, P, N, G)
    _check(lib, lib.ssd_step_fwd(byref(dims), code, state.data_ptr(), x.data_ptr(), dt.data_ptr(),
                                 A.data_ptr(), Bm.data_ptr(), Cm.data_ptr(), _ptr(D), y.data_ptr(),
                                 _stream_ptr(x)))
    return y


def ssd_steps(
    state: torch.Tensor,
    x: torch.Tensor,
    dt: torch.Tensor,
    A: torch.Tensor,
    Bm: torch.Tensor,
    Cm: torch.Tensor,
    D: Optional[torch.Tensor] = None,
    reset: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    y_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """T consecutive recurrent updates in one launch.  `state` [B,H,P,N] fp32 is advanced in place
    by T steps; x [B,T,H,P], dt [B,T,H], Bm/Cm [B,T,G,N]; returns y [B,T,H,P].  `reset` [B,T] uint8
    or bool: a non-zero entry zeroes that batch row of the state before the step (a rollout's
    "reset some environments, then step")."""
    lib = load_library()
    if state.dim() != 4:
        raise ValueError(f"SSD state must be rank-4 [batch, nheads, headdim, dstate], got {tuple(state.shape)}")
    if x.dim() != 4:
        raise ValueError(f"SSD steps x must be rank-4 [batch, nsteps, nheads, headdim], got {tuple(x.shape)}")
    if Bm.dim() != 4:
        raise ValueError(f"SSD steps B must be rank-4 [batch, nsteps, ngroups, dstate], got {tuple(Bm.shape)}")
    Bsz, H, P, N = state.shape
    T, G = x.shape[1], Bm.shape[2]
    if T < 1:
        raise ValueError("SSD steps needs at least one step")
    dtype = x.dtype
    _dtype_code(x)
    _require(state, "state", (Bsz, H, P, N), torch.float32)
    _require(x, "x", (Bsz, T, H, P), dtype)
    _require(dt, "dt", (Bsz, T, H), dtype)
    _require(A, "A", (H,), torch.float32)
    _require(Bm, "B", (Bsz, T, G, N), dtype)
    _require(Cm, "C", (Bsz, T, G, N), dtype)
    if D is not None:
        _require(D, "D", (H,), torch.float32)
    if reset is not None:
        if reset.dtype == torch.bool:
            reset = reset.view(torch.uint8)
        _require(reset, "reset", (Bsz, T), torch.uint8)
    code, y_dtype = _out_code(x, y_dtype)
    y = torch.empty((Bsz, T, H, P), dtype=y_dtype, device=x.device) if out is None else out
    _require(y, "out", (Bsz, T, H, P), y_dtype)
    dims = SsdStepDims(Bsz, H, P, N, G)
    _check(lib, lib.ssd_steps_fwd(byref(dims), T, code, state.data_ptr(), _ptr(reset), x.data_ptr(), dt.data_ptr(),
                                  A.data_ptr(), Bm.data_ptr(), Cm.data_ptr(), _ptr(D), y.data_ptr(),
                                  _stream_ptr(x)))
    return y
