"""A Mamba-2 block around the SSD scan: in-projection -> causal depthwise conv + SiLU on (x, B, C), softplus on
dt -> SSD scan -> gated RMSNorm -> out-projection.  It is the layer that would sit where the reference's
encoder block sits in `patch_trunk` (`trading_bots/src/torch/model/trading_model.rs:589-606`,
`trading_bots/src/torch/model/blocks/gqa.rs:82-109`), with the conv's streaming state carried next to the SSM
state the way the reference's `StreamState` carries its encoder memory (`trading_model.rs:56-75`).

The two projections are torch matmuls (plain GEMMs); everything between them runs in libssd_hip: the pre-scan
and post-scan kernels bound here and the scan / step of `ssd.py`.
"""
from __future__ import annotations

import math
from ctypes import POINTER, Structure, byref, c_float, c_int, c_int64, c_size_t, c_void_p
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import ssd
from .stream_state import SsdStreamState


class SsdBlockDims(Structure):
    _fields_ = [(n, c_int64) for n in ("batch", "seqlen", "nheads", "headdim", "dstate", "ngroups", "d_conv", "zxbcdt_ld")]


_bound = False


def _lib():
    global _bound
    lib = ssd.load_library()
    if not _bound:
        P = c_void_p
        lib.ssd_block_pre_fwd.argtypes = [POINTER(SsdBlockDims), c_int, P, P, P, P, P, P, P, P, P, P, P]
        lib.ssd_block_post_fwd.argtypes = [POINTER(SsdBlockDims), c_int, P, P, P, c_float, P, P]
        lib.ssd_block_proj_fwd.argtypes = [c_int64, c_int64, c_int64, c_int64, c_int, P, P, P, P]
        lib.ssd_block_post_proj_fwd.argtypes = [POINTER(SsdBlockDims), c_int, P, P, P, c_float, P, c_int64, c_int64, P, P]
        lib.ssd_block_post_proj_fwd.restype = c_int
        lib.ssd_block_step_fwd.argtypes = [POINTER(SsdBlockDims), c_int, c_int64, P, P, P, P, P, P, P, P, c_float, P, P, P, P, P]
        lib.ssd_block_step_fwd.restype = c_int
        lib.ssd_block_pre_reset_fwd.argtypes = [POINTER(SsdBlockDims), c_int, P, P, P, P, P, P, P, P, P, P, P, P]
        lib.ssd_block_pre_reset_fwd.restype = c_int
        lib.ssd_block_bwd_workspace_bytes.argtypes = [POINTER(SsdBlockDims), c_int, POINTER(c_size_t)]
        lib.ssd_block_post_bwd.argtypes = [POINTER(SsdBlockDims), c_int, P, P, P, c_float, P, P, P, P, P, c_size_t, P]
        lib.ssd_block_post_bwd_yn.argtypes = [POINTER(SsdBlockDims), c_int, P, P, P, c_float, P, P, P, P, P, P, c_size_t, P]
        lib.ssd_block_pre_bwd.argtypes = [POINTER(SsdBlockDims), c_int] + [P] * 17 + [c_size_t, P]
        for name in ("ssd_block_bwd_workspace_bytes", "ssd_block_post_bwd", "ssd_block_post_bwd_yn", "ssd_block_pre_bwd"):
            getattr(lib, name).restype = c_int
        lib.ssd_block_pre_fwd.restype = c_int
        lib.ssd_block_post_fwd.restype = c_int
        lib.ssd_block_proj_fwd.restype = c_int
        _bound = True
    return lib


def _weight_gradient(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """a^T b in float32 for tall a [rows, E] (its rows may be a view into wider ones) and b [rows, D]: a sum over all
    rows of the batch and the sequence.  As one GEMM the BLAS behind torch sees a contraction hundreds of thousands
    long against outputs a few hundred wide and runs it at a fifth of its rate, so the rows are cut into equal slabs,
    multiplied as one batched GEMM with float32 outputs, and the slabs' products added in order (measured on MI355X,
    524 288 rows: 648 x 256 outputs 1 333 -> 232 us, 256 x 256 outputs 1 059 -> 129 us; the float32 partial products also
    make the result more accurate than the single GEMM's bf16 output)."""
    rows = a.shape[0]
    slabs = 1
    while slabs < 128 and rows % (2 * slabs) == 0 and rows // (2 * slabs) >= 4096:
        slabs *= 2
    if slabs == 1 or a.dtype == torch.float32:
        return torch.matmul(a.t(), b).float()
    a3 = a.unflatten(0, (slabs, rows // slabs))
    b3 = b.unflatten(0, (slabs, rows // slabs))
    return torch.bmm(a3.transpose(1, 2), b3, out_dtype=torch.float32).sum(0)


def in_proj_width(nheads, headdim, dstate, ngroups) -> int:
    return 2 * nheads * headdim + 2 * ngroups * dstate + nheads


def _row_stride(zxbcdt) -> int:
    """The row stride of zxbcdt [B,L,E]: dense, or the first E columns of a buffer with padded rows (what
    `block_proj(..., pad_rows=True)` returns)."""
    Bsz, L, E = zxbcdt.shape
    ld = zxbcdt.stride(1) if L > 1 else (zxbcdt.stride(0) if Bsz > 1 else E)
    if zxbcdt.data_ptr() % 16:
        raise ValueError("zxbcdt must be 16-byte aligned")
    if zxbcdt.is_contiguous():
        return E
    if zxbcdt.stride(2) != 1 or ld < E or (L > 1 and Bsz > 1 and zxbcdt.stride(0) != L * ld):
        raise ValueError(f"zxbcdt must be contiguous or have evenly padded rows, got strides {zxbcdt.stride()}")
    return ld


def block_pre(zxbcdt, conv_w, conv_b, dt_bias, nheads, headdim, dstate, ngroups, conv_state=None,
              return_conv_state=False, reset=None, conv_state_out=None):
    """zxbcdt [B,L,E] (rows dense or evenly padded) -> (x [B,L,H,P], Bm, Cm [B,L,G,N], dt [B,L,H][, conv state
    [B,d_conv-1,C]]).  `reset` [B,L] (uint8 or bool): a non-zero entry cuts the filter's history before that
    timestep.  `conv_state_out`: where to write the new conv state (may be `conv_state` itself for seqlen 1)."""
    lib = _lib()
    if zxbcdt.dim() != 3:
        raise ValueError(f"block input must be rank-3 [batch, seqlen, channels], got {tuple(zxbcdt.shape)}")
    Bsz, L, E = zxbcdt.shape
    H, P, N, G = nheads, headdim, dstate, ngroups
    C = H * P + 2 * G * N
    if E != in_proj_width(H, P, N, G):
        raise ValueError(f"block input must have {in_proj_width(H, P, N, G)} channels, got {E}")
    dtype = zxbcdt.dtype
    code = ssd._dtype_code(zxbcdt)
    if not zxbcdt.is_cuda:
        raise ValueError("zxbcdt must be a GPU tensor")
    ld = _row_stride(zxbcdt)
    if conv_w.dim() != 2 or conv_w.shape[0] != C:
        raise ValueError(f"conv_w must be [{C}, d_conv], got {tuple(conv_w.shape)}")
    d_conv = conv_w.shape[1]
    ssd._require(conv_w, "conv_w", (C, d_conv), torch.float32)
    ssd._require(conv_b, "conv_b", (C,), torch.float32)
    ssd._require(dt_bias, "dt_bias", (H,), torch.float32)
    if conv_state is not None:
        ssd._require(conv_state, "conv_state", (Bsz, d_conv - 1, C), dtype)
    dev = zxbcdt.device
    x = torch.empty((Bsz, L, H, P), dtype=dtype, device=dev)
    Bm = torch.empty((Bsz, L, G, N), dtype=dtype, device=dev)
    Cm = torch.empty((Bsz, L, G, N), dtype=dtype, device=dev)
    dt = torch.empty((Bsz, L, H), dtype=dtype, device=dev)
    new_state = None
    if conv_state_out is not None:
        ssd._require(conv_state_out, "conv_state_out", (Bsz, d_conv - 1, C), dtype)
        new_state, return_conv_state = conv_state_out, True
    elif return_conv_state:
        new_state = torch.empty((Bsz, d_conv - 1, C), dtype=dtype, device=dev)
    if reset is not None:
        if reset.dtype == torch.bool:
            reset = reset.view(torch.uint8)
        ssd._require(reset, "reset", (Bsz, L), torch.uint8)
    dims = SsdBlockDims(Bsz, L, H, P, N, G, d_conv, ld)
    ssd._check(lib, lib.ssd_block_pre_reset_fwd(byref(dims), code, zxbcdt.data_ptr(), conv_w.data_ptr(),
                                                conv_b.data_ptr(), dt_bias.data_ptr(), ssd._ptr(conv_state),
                                                ssd._ptr(new_state), ssd._ptr(reset), x.data_ptr(), Bm.data_ptr(),
                                                Cm.data_ptr(), dt.data_ptr(), ssd._stream_ptr(zxbcdt)))
    return (x, Bm, Cm, dt, new_state) if return_conv_state else (x, Bm, Cm, dt)


def block_post(y, zxbcdt, norm_w, nheads, headdim, dstate, ngroups, eps=1e-5):
    """out [B,L,H*P] = rmsnorm(y * silu(z)) * norm_w; y [B,L,H,P] in the activation dtype or float32."""
    lib = _lib()
    Bsz, L, E = zxbcdt.shape
    H, P, N, G = nheads, headdim, dstate, ngroups
    dtype = zxbcdt.dtype
    code = ssd._dtype_code(zxbcdt)
    if y.dtype != dtype:
        if not (dtype == torch.bfloat16 and y.dtype == torch.float32):
            raise ValueError(f"block y must be {dtype} (or float32 with bf16 activations), got {y.dtype}")
        code = ssd.SSD_DTYPE_BF16_Y32
    if not zxbcdt.is_cuda or E != in_proj_width(H, P, N, G):
        raise ValueError(f"zxbcdt must be a GPU tensor with {in_proj_width(H, P, N, G)} channels, got {tuple(zxbcdt.shape)}")
    ld = _row_stride(zxbcdt)
    ssd._require(y, "y", (Bsz, L, H, P), y.dtype)
    ssd._require(norm_w, "norm_w", (H * P,), torch.float32)
    out = torch.empty((Bsz, L, H * P), dtype=dtype, device=zxbcdt.device)
    dims = SsdBlockDims(Bsz, L, H, P, N, G, 4, ld)
    ssd._check(lib, lib.ssd_block_post_fwd(byref(dims), code, y.data_ptr(), zxbcdt.data_ptr(), norm_w.data_ptr(),
                                           c_float(eps), out.data_ptr(), ssd._stream_ptr(zxbcdt)))
    return out


def block_post_proj_supported(y: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether `block_post_proj` takes these tensors (else `block_post`, then the projection)."""
    return (y.is_cuda and y.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.shape[1] in (128, 256) and weight.shape[0] % 8 == 0 and weight.shape[0] <= 256)


def block_post_proj(y, zxbcdt, norm_w, weight, nheads, headdim, dstate, ngroups, eps=1e-5):
    """out [B,L,out_features] = (rmsnorm(y * silu(z)) * norm_w) . weight^T as one kernel (bf16; weight
    [out_features, H*P]): `block_post` and the out-projection without the normalised rows going to memory between."""
    lib = _lib()
    Bsz, L, E = zxbcdt.shape
    H, P, N, G = nheads, headdim, dstate, ngroups
    if not zxbcdt.is_cuda or E != in_proj_width(H, P, N, G):
        raise ValueError(f"zxbcdt must be a GPU tensor with {in_proj_width(H, P, N, G)} channels, got {tuple(zxbcdt.shape)}")
    if zxbcdt.dtype != torch.bfloat16 or y.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise ValueError("block_post_proj takes bfloat16 tensors")
    ld = _row_stride(zxbcdt)
    ssd._require(y, "y", (Bsz, L, H, P), torch.bfloat16)
    ssd._require(norm_w, "norm_w", (H * P,), torch.float32)
    if weight.dim() != 2 or weight.shape[1] != H * P or not weight.is_contiguous():
        raise ValueError(f"weight must be contiguous [out_features, {H * P}], got {tuple(weight.shape)}")
    out = torch.empty((Bsz, L, weight.shape[0]), dtype=torch.bfloat16, device=zxbcdt.device)
    dims = SsdBlockDims(Bsz, L, H, P, N, G, 4, ld)
    ssd._check(lib, lib.ssd_block_post_proj_fwd(byref(dims), ssd.SSD_DTYPE_BF16, y.data_ptr(), zxbcdt.data_ptr(),
                                                norm_w.data_ptr(), c_float(eps), weight.data_ptr(), weight.shape[0], 0,
                                                out.data_ptr(), ssd._stream_ptr(zxbcdt)))
    return out


# batches up to which one workgroup per stream (each reading both weight matrices whole) beats the stage kernels
FUSED_STEP_MAX_BATCH = 64


def block_step_supported(u_t: torch.Tensor, d_inner: int, dstate: int) -> bool:
    """Whether `block_step` takes this step (else the stage kernels, one launch each)."""
    return (u_t.is_cuda and u_t.dtype in (torch.bfloat16, torch.float32) and u_t.dim() == 2
            and u_t.shape[1] in (128, 256) and d_inner in (128, 256) and dstate % 16 == 0)


def block_step(u_t, w_in, conv_w, conv_b, dt_bias, A, D, norm_w, w_out, conv_state, ssm_state, nheads, headdim, dstate,
               ngroups, eps=1e-5, out=None):
    """One timestep of the whole block for every stream as one launch: u_t [B,d_model] -> out [B,d_model]; `conv_state`
    [B,d_conv-1,C] (activation dtype) and `ssm_state` [B,H,P,N] (float32) advance in place.  w_in [E,d_model] and
    w_out [d_model,H*P] in the activation dtype."""
    lib = _lib()
    Bsz, d_model = u_t.shape
    H, P, N, G = nheads, headdim, dstate, ngroups
    C = H * P + 2 * G * N
    E = in_proj_width(H, P, N, G)
    dtype = u_t.dtype
    code = ssd._dtype_code(u_t)
    d_conv = conv_w.shape[1]
    ssd._require(u_t, "u_t", (Bsz, d_model), dtype)
    ssd._require(w_in, "w_in", (E, d_model), dtype)
    ssd._require(w_out, "w_out", (d_model, H * P), dtype)
    ssd._require(conv_w, "conv_w", (C, d_conv), torch.float32)
    ssd._require(conv_b, "conv_b", (C,), torch.float32)
    ssd._require(dt_bias, "dt_bias", (H,), torch.float32)
    ssd._require(A, "A", (H,), torch.float32)
    if D is not None:
        ssd._require(D, "D", (H,), torch.float32)
    ssd._require(norm_w, "norm_w", (H * P,), torch.float32)
    ssd._require(conv_state, "conv_state", (Bsz, d_conv - 1, C), dtype)
    ssd._require(ssm_state, "ssm_state", (Bsz, H, P, N), torch.float32)
    if out is None:
        out = torch.empty((Bsz, d_model), dtype=dtype, device=u_t.device)
    else:
        ssd._require(out, "out", (Bsz, d_model), dtype)
    dims = SsdBlockDims(Bsz, 1, H, P, N, G, d_conv, 0)
    ssd._check(lib, lib.ssd_block_step_fwd(byref(dims), code, d_model, u_t.data_ptr(), w_in.data_ptr(), conv_w.data_ptr(),
                                           conv_b.data_ptr(), dt_bias.data_ptr(), A.data_ptr(), ssd._ptr(D),
                                           norm_w.data_ptr(), c_float(eps), w_out.data_ptr(), conv_state.data_ptr(),
                                           ssm_state.data_ptr(), out.data_ptr(), ssd._stream_ptr(u_t)))
    return out


def block_bwd_workspace(batch, seqlen, nheads, headdim, dstate, ngroups, d_conv=4, dtype=torch.bfloat16, device="cuda"):
    """Scratch for the partial sums of block_post_bwd / block_pre_bwd (one buffer serves both calls of a pass)."""
    lib = _lib()
    need = c_size_t(0)
    dims = SsdBlockDims(batch, seqlen, nheads, headdim, dstate, ngroups, d_conv, 0)
    code = ssd.SSD_DTYPE_F32 if dtype == torch.float32 else ssd.SSD_DTYPE_BF16
    ssd._check(lib, lib.ssd_block_bwd_workspace_bytes(byref(dims), code, byref(need)))
    return torch.empty(need.value, dtype=torch.uint8, device=device)


def block_post_bwd(y, zxbcdt, norm_w, dout, dzxbcdt, nheads, headdim, dstate, ngroups, eps=1e-5, workspace=None,
                   d_conv=4, yn_out=None):
    """Gradients of block_post: returns (dy [B,L,H,P], dnorm_w [H*P]) and writes dz into the z channels of dzxbcdt
    (a tensor laid out like zxbcdt, same row stride).  `d_conv` is the block's filter length: the library sizes the
    scratch both backward calls of a pass share from it, so it must be the one `workspace` was sized with.
    With `yn_out` [B,L,H*P] (zxbcdt's dtype) the call also writes the forward's normalised rows into it, bit for bit
    what `block_post` returns (for a forward that ran `block_post_proj` and kept none)."""
    lib = _lib()
    Bsz, L, E = zxbcdt.shape
    H, P, N, G = nheads, headdim, dstate, ngroups
    dtype = zxbcdt.dtype
    code = ssd._dtype_code(zxbcdt)
    if y.dtype != dtype:
        if not (dtype == torch.bfloat16 and y.dtype == torch.float32):
            raise ValueError(f"block y must be {dtype} (or float32 with bf16 activations), got {y.dtype}")
        code = ssd.SSD_DTYPE_BF16_Y32
    ld = _row_stride(zxbcdt)
    if tuple(dzxbcdt.shape) != (Bsz, L, E) or dzxbcdt.dtype != dtype or _row_stride(dzxbcdt) != ld:
        raise ValueError("dzxbcdt must have zxbcdt's shape, dtype and row stride")
    ssd._require(y, "y", (Bsz, L, H, P), y.dtype)
    ssd._require(dout, "dout", (Bsz, L, H * P), dtype)
    ssd._require(norm_w, "norm_w", (H * P,), torch.float32)
    dy = torch.empty((Bsz, L, H, P), dtype=dtype, device=zxbcdt.device)
    dnorm_w = torch.empty(H * P, dtype=torch.float32, device=zxbcdt.device)
    if workspace is None:
        workspace = block_bwd_workspace(Bsz, L, H, P, N, G, d_conv, dtype, zxbcdt.device)
    dims = SsdBlockDims(Bsz, L, H, P, N, G, d_conv, ld)
    if yn_out is not None:
        ssd._require(yn_out, "yn_out", (Bsz, L, H * P), dtype)
    ssd._check(lib, lib.ssd_block_post_bwd_yn(byref(dims), code, y.data_ptr(), zxbcdt.data_ptr(), norm_w.data_ptr(), c_float(eps),
                                              dout.data_ptr(), dy.data_ptr(), dzxbcdt.data_ptr(), dnorm_w.data_ptr(),
                                              None if yn_out is None else yn_out.data_ptr(),
                                              workspace.data_ptr(), workspace.numel(), ssd._stream_ptr(zxbcdt)))
    return dy, dnorm_w


def block_pre_bwd(zxbcdt, conv_w, conv_b, dt_bias, dx, dB, dC, ddt, dzxbcdt, nheads, headdim, dstate, ngroups,
                  conv_state=None, reset=None, dconv_state_out=None, need_dconv_state=False, workspace=None):
    """Gradients of block_pre: writes the x | B | C | dt channels of dzxbcdt and returns (dconv_w [C,d_conv],
    dconv_b [C], ddt_bias [H], dconv_state [B,d_conv-1,C] or None)."""
    lib = _lib()
    Bsz, L, E = zxbcdt.shape
    H, P, N, G = nheads, headdim, dstate, ngroups
    C = H * P + 2 * G * N
    dtype = zxbcdt.dtype
    code = ssd._dtype_code(zxbcdt)
    ld = _row_stride(zxbcdt)
    d_conv = conv_w.shape[1]
    if tuple(dzxbcdt.shape) != (Bsz, L, E) or dzxbcdt.dtype != dtype or _row_stride(dzxbcdt) != ld:
        raise ValueError("dzxbcdt must have zxbcdt's shape, dtype and row stride")
    ssd._require(conv_w, "conv_w", (C, d_conv), torch.float32)
    ssd._require(conv_b, "conv_b", (C,), torch.float32)
    ssd._require(dt_bias, "dt_bias", (H,), torch.float32)
    ssd._require(dx, "dx", (Bsz, L, H, P), dtype)
    ssd._require(dB, "dB", (Bsz, L, G, N), dtype)
    ssd._require(dC, "dC", (Bsz, L, G, N), dtype)
    ssd._require(ddt, "ddt", (Bsz, L, H), dtype)
    for name, t in (("conv_state", conv_state), ("dconv_state_out", dconv_state_out)):
        if t is not None:
            ssd._require(t, name, (Bsz, d_conv - 1, C), dtype)
    if reset is not None:
        if reset.dtype == torch.bool:
            reset = reset.view(torch.uint8)
        ssd._require(reset, "reset", (Bsz, L), torch.uint8)
    dev = zxbcdt.device
    dconv_w = torch.empty((C, d_conv), dtype=torch.float32, device=dev)
    dconv_b = torch.empty(C, dtype=torch.float32, device=dev)
    ddt_bias = torch.empty(H, dtype=torch.float32, device=dev)
    dstate = torch.empty((Bsz, d_conv - 1, C), dtype=dtype, device=dev) if need_dconv_state else None
    if workspace is None:
        workspace = block_bwd_workspace(Bsz, L, H, P, N, G, d_conv, dtype, dev)
    dims = SsdBlockDims(Bsz, L, H, P, N, G, d_conv, ld)
    ssd._check(lib, lib.ssd_block_pre_bwd(byref(dims), code, zxbcdt.data_ptr(), conv_w.data_ptr(), conv_b.data_ptr(),
                                          dt_bias.data_ptr(), ssd._ptr(conv_state), ssd._ptr(reset), dx.data_ptr(),
                                          dB.data_ptr(), dC.data_ptr(), ddt.data_ptr(), ssd._ptr(dconv_state_out),
                                          dzxbcdt.data_ptr(), dconv_w.data_ptr(), dconv_b.data_ptr(), ddt_bias.data_ptr(),
                                          ssd._ptr(dstate), workspace.data_ptr(), workspace.numel(),
                                          ssd._stream_ptr(zxbcdt)))
    return dconv_w, dconv_b, ddt_bias, dstate


def block_proj_supported(u: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether `block_proj` takes this product (else the caller's BLAS does it)."""
    return (u.is_cuda and u.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and u.shape[-1] in (128, 256)
            and weight.shape[0] % 8 == 0 and u.numel() > 0)


def block_proj(u: torch.Tensor, weight: torch.Tensor, pad_rows: bool = False) -> torch.Tensor:
    """u [..., in_features] (bf16) times weight [out_features, in_features]^T -> [..., out_features] (bf16), float32
    accumulation: the block's in- and out-projection as one memory-bound kernel.  With pad_rows the result is the
    first out_features columns of a buffer whose rows are a multiple of 128 bytes apart (a non-contiguous view that
    `block_pre` and `block_post` take): every line the kernel writes is then a whole one."""
    lib = _lib()
    if u.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise ValueError(f"block_proj takes bfloat16 tensors, got {u.dtype} and {weight.dtype}")
    if weight.dim() != 2 or u.shape[-1] != weight.shape[1]:
        raise ValueError(f"block_proj: u [..., {u.shape[-1]}] does not match weight {tuple(weight.shape)}")
    if not u.is_contiguous() or not weight.is_contiguous():
        raise ValueError("block_proj takes contiguous tensors")
    rows = u.numel() // u.shape[-1]
    width = weight.shape[0]
    ld = (width + 63) // 64 * 64 if pad_rows else width
    out = torch.empty(u.shape[:-1] + (ld,), dtype=torch.bfloat16, device=u.device)
    ssd._check(lib, lib.ssd_block_proj_fwd(rows, u.shape[-1], width, ld, ssd.SSD_DTYPE_BF16, u.data_ptr(),
                                           weight.data_ptr(), out.data_ptr(), ssd._stream_ptr(u)))
    return out[..., :width] if ld != width else out


@dataclass
class Mamba2StreamState:
    """Streaming memory of one block: the conv's last d_conv-1 inputs and the SSM state."""
    conv: torch.Tensor          # [B, d_conv-1, H*P + 2*G*N], activation dtype
    ssm: SsdStreamState         # [B, H, P, N] float32

    def reset(self) -> None:
        self.conv.zero_()
        self.ssm.reset()

    def reset_rows(self, rows: torch.Tensor) -> None:
        if rows.dtype == torch.bool:
            self.conv.mul_((~rows).to(self.conv.dtype).view(-1, 1, 1))
        else:
            self.conv.index_fill_(0, rows, 0.0)
        self.ssm.reset_rows(rows)


class Mamba2Block:
    """Parameters and forward of one block.  Parameters are float32 masters; the projections run in the
    activation dtype of the input (bf16 on the GPU, as the reference policy runs,
    `trading_bots/src/torch/model/trading_model.rs:140-146`)."""

    def __init__(self, d_model, nheads, headdim, dstate, ngroups=1, d_conv=4, chunk=128, eps=1e-5, device="cuda",
                 seed=0):
        self.d_model, self.H, self.P, self.N, self.G = d_model, nheads, headdim, dstate, ngroups
        self.d_conv, self.chunk, self.eps = d_conv, chunk, eps
        self.d_inner = nheads * headdim
        self.conv_dim = self.d_inner + 2 * ngroups * dstate
        E = in_proj_width(nheads, headdim, dstate, ngroups)
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)

        def rnd(*shape, scale=1.0):
            return (torch.randn(*shape, generator=g) * scale).to(device)

        self.in_proj = rnd(E, d_model, scale=1.0 / math.sqrt(d_model))
        self.conv_w = rnd(self.conv_dim, d_conv, scale=1.0 / math.sqrt(d_conv))
        self.conv_b = rnd(self.conv_dim, scale=0.1)
        # dt after softplus spread over [1e-3, 1e-1] (log-uniform), as Mamba-2 initialises it
        dt0 = torch.exp(torch.rand(nheads, generator=g) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3))
        self.dt_bias = (dt0 + torch.log(-torch.expm1(-dt0))).to(device)
        self.A_log = torch.log(torch.rand(nheads, generator=g) * 15.0 + 1.0).to(device)
        self.D = torch.ones(nheads, device=device)
        self.norm_w = torch.ones(self.d_inner, device=device)
        self.out_proj = rnd(d_model, self.d_inner, scale=1.0 / math.sqrt(self.d_inner))

    @property
    def A(self) -> torch.Tensor:
        return -torch.exp(self.A_log)

    def new_state(self, batch, dtype=torch.bfloat16) -> Mamba2StreamState:
        conv = torch.zeros((batch, self.d_conv - 1, self.conv_dim), dtype=dtype, device=self.in_proj.device)
        return Mamba2StreamState(conv, SsdStreamState.build(batch, self.H, self.P, self.N, device=self.in_proj.device))

    def forward(self, u: torch.Tensor, state: Optional[Mamba2StreamState] = None,
                reset: Optional[torch.Tensor] = None, save_for_backward: bool = False):
        """u [B,L,d_model] -> [B,L,d_model].  With `state`, continues from it and leaves it at the end of the
        window (a prefix scan; then `step` per bar).  `reset` [B,L]: episode boundaries inside the window -- a
        non-zero entry restarts both the SSM state and the conv's history before that timestep, exactly what
        `Mamba2StreamState.reset_rows` does between two steps of a stream.  With `save_for_backward` (windows
        without a carried state) returns (out, ctx) for `backward`."""
        if u.dim() != 3 or u.shape[2] != self.d_model:
            raise ValueError(f"block input must be [batch, seqlen, {self.d_model}], got {tuple(u.shape)}")
        if reset is not None and state is not None:
            raise ValueError("restarts inside the window and a carried conv state cannot be combined")
        zxbcdt = self._project(u, self._weights(u.dtype)[0], pad_rows=True)  # internal to the block: rows of whole lines
        if state is None:
            x, Bm, Cm, dt = block_pre(zxbcdt, self.conv_w, self.conv_b, self.dt_bias, self.H, self.P, self.N, self.G,
                                      reset=reset)
            y, _ = ssd.ssd_chunk_scan(x, dt, self.A, Bm, Cm, self.D, chunk=self.chunk, return_final_states=False,
                                      reset=reset)
        else:
            x, Bm, Cm, dt, conv = block_pre(zxbcdt, self.conv_w, self.conv_b, self.dt_bias, self.H, self.P, self.N,
                                            self.G, conv_state=state.conv, return_conv_state=True)
            state.conv = conv
            y = state.ssm.init_from_prefix(x, dt, self.A, Bm, Cm, self.D, chunk=self.chunk)
        w_out = self._weights(u.dtype)[1]
        if save_for_backward and state is not None:
            raise ValueError("backward through a window that continues a carried state is not supported")
        if block_post_proj_supported(y, w_out) and y.numel() // self.d_inner >= 8192:
            # gate, norm and out-projection as one kernel: the normalised rows never reach memory (the backward pass
            # needs them for one weight gradient only, and has its post stage write them on the way: yn=None)
            out = block_post_proj(y, zxbcdt, self.norm_w, w_out, self.H, self.P, self.N, self.G, self.eps)
            yn = None
        else:
            yn = block_post(y, zxbcdt, self.norm_w, self.H, self.P, self.N, self.G, self.eps)
            out = self._project(yn, w_out)
        if save_for_backward:
            return out, dict(u=u, zxbcdt=zxbcdt, x=x, Bm=Bm, Cm=Cm, dt=dt, y=y, yn=yn, reset=reset)
        return out

    def backward(self, ctx: dict, dout: torch.Tensor) -> dict:
        """Gradients of sum(out * dout) with respect to the input and every parameter, from the tensors `forward`
        kept: two GEMMs per projection (torch), the library's post, scan and pre backward kernels between them.
        Returns du [B,L,d_model] and float32 din_proj, dconv_w, dconv_b, ddt_bias, dA, dA_log, dD, dnorm_w, dout_proj."""
        u, zxbcdt, y, yn, reset = ctx["u"], ctx["zxbcdt"], ctx["y"], ctx["yn"], ctx["reset"]
        x, Bm, Cm, dt = ctx["x"], ctx["Bm"], ctx["Cm"], ctx["dt"]
        Bsz, L, _ = u.shape
        act = u.dtype
        E = in_proj_width(self.H, self.P, self.N, self.G)
        w_in, w_out = self._weights(act)
        dout2 = dout.reshape(Bsz * L, self.d_model)
        dyn = self._project(dout2, self._out_proj_transposed(act)).view(Bsz, L, self.d_inner)
        # (a forward that ran gate, norm and out-projection as one kernel kept no normalised rows: post_bwd writes them)
        yn_new = None if yn is not None else torch.empty((Bsz, L, self.d_inner), dtype=act, device=u.device)
        # the gradient of zxbcdt, with zxbcdt's own (padded) row stride
        ld = _row_stride(zxbcdt)
        dbuf = torch.empty((Bsz, L, ld), dtype=act, device=u.device)
        dzx = dbuf[..., :E] if ld != E else dbuf
        ws = block_bwd_workspace(Bsz, L, self.H, self.P, self.N, self.G, self.d_conv, act, u.device)
        dy, dnorm_w = block_post_bwd(y, zxbcdt, self.norm_w, dyn, dzx, self.H, self.P, self.N, self.G, self.eps, workspace=ws,
                                     d_conv=self.d_conv, yn_out=yn_new)
        dout_proj = _weight_gradient(dout2, (yn if yn is not None else yn_new).reshape(Bsz * L, self.d_inner))
        g = ssd.ssd_chunk_scan_backward(x, dt, self.A, Bm, Cm, self.D, dy, chunk=self.chunk, reset=reset)
        dconv_w, dconv_b, ddt_bias, _ = block_pre_bwd(zxbcdt, self.conv_w, self.conv_b, self.dt_bias, g["dx"], g["dB"],
                                                      g["dC"], g["ddt"], dzx, self.H, self.P, self.N, self.G, reset=reset,
                                                      workspace=ws)
        dz2 = dbuf.view(Bsz * L, ld)[:, :E]
        du = torch.matmul(dz2, w_in).view(Bsz, L, self.d_model)
        din_proj = _weight_gradient(dz2, u.reshape(Bsz * L, self.d_model))
        return dict(du=du, din_proj=din_proj, dconv_w=dconv_w, dconv_b=dconv_b, ddt_bias=ddt_bias, dA=g["dA"],
                    dA_log=g["dA"] * self.A, dD=g["dD"], dnorm_w=dnorm_w, dout_proj=dout_proj)

    def _project(self, u: torch.Tensor, weight: torch.Tensor, pad_rows: bool = False) -> torch.Tensor:
        """u . weight^T in the activation dtype: the library's kernel where it takes the shape (bf16, in_features 128
        or 256, a tall u), else the BLAS behind torch."""
        w = weight.to(u.dtype)
        u = u.contiguous()
        if block_proj_supported(u, w) and u.numel() // u.shape[-1] >= 16384:
            return block_proj(u, w.contiguous(), pad_rows=pad_rows)
        return torch.matmul(u, w.t()).contiguous()

    def _weights(self, dtype: torch.dtype):
        """The two projection matrices in the activation dtype, converted once per dtype (and again when a master
        copy has been modified in place)."""
        key = (dtype, self.in_proj._version, self.out_proj._version, self.in_proj.data_ptr(), self.out_proj.data_ptr())
        cached = getattr(self, "_weights_cache", None)
        if cached is None or cached[0] != key:
            w_out = self.out_proj.to(dtype).contiguous()
            cached = (key, self.in_proj.to(dtype).contiguous(), w_out, w_out.t().contiguous())
            self._weights_cache = cached
        return cached[1], cached[2]

    def _out_proj_transposed(self, dtype: torch.dtype) -> torch.Tensor:
        """out_proj^T [d_inner, d_model] in the activation dtype (the backward's dyn = dout . out_proj is then a
        product of the forward's form, which the library's projection kernel takes), cached with the others."""
        self._weights(dtype)
        return self._weights_cache[3]

    def _A_cached(self) -> torch.Tensor:
        """-exp(A_log), computed once per version of A_log (a launch of its own otherwise, per step)."""
        key = (self.A_log._version, self.A_log.data_ptr())
        cached = getattr(self, "_A_cache", None)
        if cached is None or cached[0] != key:
            cached = (key, -torch.exp(self.A_log))
            self._A_cache = cached
        return cached[1]

    def step(self, u_t: torch.Tensor, state: Mamba2StreamState, fused: Optional[bool] = None) -> torch.Tensor:
        """One timestep for every stream: u_t [B,d_model] -> [B,d_model]; advances `state` in place.  `fused`: run the
        step as one launch (default: for batches up to FUSED_STEP_MAX_BATCH of shapes the fused kernel takes) or as the
        stage kernels with the projections on the BLAS behind torch."""
        if u_t.dim() != 2 or u_t.shape[1] != self.d_model:
            raise ValueError(f"block step input must be [batch, {self.d_model}], got {tuple(u_t.shape)}")
        w_in, w_out = self._weights(u_t.dtype)
        if fused is None:
            fused = u_t.shape[0] <= FUSED_STEP_MAX_BATCH and block_step_supported(u_t, self.d_inner, self.N)
        if fused:   # the whole step as one launch: what a step costs at a few streams is issuing its launches
            return block_step(u_t.contiguous(), w_in, self.conv_w, self.conv_b, self.dt_bias, self._A_cached(), self.D,
                              self.norm_w, w_out, state.conv, state.ssm.state, self.H, self.P, self.N, self.G, self.eps)
        zxbcdt = torch.matmul(u_t, w_in.t()).unsqueeze(1).contiguous()
        x, Bm, Cm, dt, _ = block_pre(zxbcdt, self.conv_w, self.conv_b, self.dt_bias, self.H, self.P, self.N,
                                     self.G, conv_state=state.conv, conv_state_out=state.conv)  # in place
        y = state.ssm.step(x[:, 0], dt[:, 0], self.A, Bm[:, 0], Cm[:, 0], self.D)
        yn = block_post(y.unsqueeze(1), zxbcdt, self.norm_w, self.H, self.P, self.N, self.G, self.eps)
        return torch.matmul(yn[:, 0], w_out.t())

    def graphed_step(self, state: Mamba2StreamState, dtype: torch.dtype = torch.bfloat16) -> "GraphedBlockStep":
        """`step` for `state`'s streams captured once in a HIP graph and replayed per bar: at a few streams a step
        is five launches of a few microseconds each and the host's time to issue them is what a step costs (the
        reference captures its launch-bound loops the same way, trading_bots/src/torch/cuda/graph.rs)."""
        return GraphedBlockStep(self, state, dtype)



class GraphedBlockStep:
    """A captured `Mamba2Block.step` over fixed buffers.  Calling it copies the bar's input into the captured input
    buffer, replays the graph and returns the captured output buffer (overwritten by the next call).  The state it
    was built for advances in place, as with `step`; the block's parameters are read at replay time, except the
    projection matrices, whose activation-dtype copies are made at capture."""

    def __init__(self, block: Mamba2Block, state: Mamba2StreamState, dtype: torch.dtype):
        batch = state.conv.shape[0]
        dev = state.conv.device
        self.u = torch.zeros((batch, block.d_model), dtype=dtype, device=dev)
        # what the warm-up steps below do to the state is undone afterwards
        conv_keep, ssm_keep = state.conv.clone(), state.ssm.state.clone()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            for _ in range(2):  # library handles, kernel modules and the weights' copies exist before the capture
                block.step(self.u, state)
        torch.cuda.current_stream(dev).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.out = block.step(self.u, state)
        state.conv.copy_(conv_keep)
        state.ssm.state.copy_(ssm_keep)

    def __call__(self, u_t: torch.Tensor) -> torch.Tensor:
        self.u.copy_(u_t)
        self.graph.replay()
        return self.out
