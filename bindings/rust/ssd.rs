//! Rust binding of libssd_hip (`include/ssd_hip.h`): the file a maintainer of CarsonBurke/trading_bot_0 would add
//! as `trading_bots/src/torch/ssd.rs`.  It follows the tree's own wrapper of a custom kernel,
//! `trading_bots/src/torch/fa4.rs:28-47` (public op functions over `&Tensor`) and `:145-191` (validate, then call,
//! one message per violated precondition), and fetches the library's thread-local error string the way
//! `trading_bots/src/torch/cuda/graph.rs:107-119` does for the torch shim.
//!
//! Source only: the image this library is built in has no Rust toolchain, so this file is checked mechanically
//! against the header instead (every `extern "C"` prototype below: name, parameter count, pointer constness and
//! pointee / integer kinds) by `tests/test_abi.py`.
//!
//! Link (in `trading_bots/build.rs`, next to the libtorch rpath lines):
//! `cargo:rustc-link-search=native=<dir of libssd_hip.so>`, `cargo:rustc-link-lib=dylib=ssd_hip`,
//! `cargo:rustc-link-arg=-Wl,-rpath,<dir>`.

use anyhow::{bail, Result};
use std::ffi::{c_char, c_int, c_void, CStr};
use tch::{Kind, Tensor};

pub const SSD_DTYPE_F32: c_int = 0;
pub const SSD_DTYPE_BF16: c_int = 1;
/// bf16 inputs, y written as f32 (same arithmetic, no output rounding)
pub const SSD_DTYPE_BF16_Y32: c_int = 2;
/// scratch that `ssd_chunk_scan_noalloc_fwd` can draw on (part of the library's device code)
pub const SSD_STATIC_SCRATCH_BYTES: usize = 64 << 20;

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct SsdDims {
    pub batch: i64,
    pub seqlen: i64,
    pub nheads: i64,
    pub headdim: i64,
    pub dstate: i64,
    pub ngroups: i64,
    pub chunk: i64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct SsdStepDims {
    pub batch: i64,
    pub nheads: i64,
    pub headdim: i64,
    pub dstate: i64,
    pub ngroups: i64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct SsdBlockDims {
    pub batch: i64,
    pub seqlen: i64,
    pub nheads: i64,
    pub headdim: i64,
    pub dstate: i64,
    pub ngroups: i64,
    pub d_conv: i64,
    /// row stride of zxbcdt in elements, 0 = dense
    pub zxbcdt_ld: i64,
}

extern "C" {
    pub fn ssd_version() -> c_int;
    pub fn ssd_get_and_reset_last_err() -> *mut c_char;
    pub fn ssd_workspace_bytes(dims: *const SsdDims, out_bytes: *mut usize) -> c_int;
    pub fn ssd_chunk_scan_fwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, dt: *const c_void,
        a: *const f32, bm: *const c_void, cm: *const c_void, d: *const f32, initial_states: *const f32,
        y: *mut c_void, final_states: *mut f32, workspace: *mut c_void, workspace_bytes: usize,
        hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_cumsum_fwd(dims: *const SsdDims, dtype: c_int, dt: *const c_void, a: *const f32,
        dtcs: *mut f32, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_state_fwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, bm: *const c_void,
        dtcs: *const f32, chunk_states: *mut f32, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_state_passing_fwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, bm: *const c_void,
        dtcs: *const f32, initial_states: *const f32, prev_states: *mut f32, final_states: *mut f32,
        hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_scan_onepass_fwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, dt: *const c_void,
        a: *const f32, bm: *const c_void, cm: *const c_void, d: *const f32, initial_states: *const f32,
        reset: *const u8, y: *mut c_void, final_states: *mut f32, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_scan_reset_fwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, dt: *const c_void,
        a: *const f32, bm: *const c_void, cm: *const c_void, d: *const f32, initial_states: *const f32,
        reset: *const u8, y: *mut c_void, final_states: *mut f32, workspace: *mut c_void, workspace_bytes: usize,
        hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_scan_noalloc_fwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, dt: *const c_void,
        a: *const f32, bm: *const c_void, cm: *const c_void, d: *const f32, initial_states: *const f32,
        reset: *const u8, y: *mut c_void, final_states: *mut f32, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_scan_is_onepass(dims: *const SsdDims, dtype: c_int, is_onepass: *mut c_int) -> c_int;
    pub fn ssd_chunk_scan_segments(dims: *const SsdDims, dtype: c_int, segments: *mut c_int) -> c_int;
    pub fn ssd_state_passing_fwd(dims: *const SsdDims, chunk_states: *const f32, dtcs: *const f32,
        initial_states: *const f32, prev_states: *mut f32, final_states: *mut f32, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_scan_stage_fwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, bm: *const c_void,
        cm: *const c_void, dtcs: *const f32, prev_states: *const f32, d: *const f32, y: *mut c_void,
        hip_stream: *mut c_void) -> c_int;
    pub fn ssd_step_fwd(dims: *const SsdStepDims, dtype: c_int, state: *mut f32, x: *const c_void,
        dt: *const c_void, a: *const f32, bm: *const c_void, cm: *const c_void, d: *const f32, y: *mut c_void,
        hip_stream: *mut c_void) -> c_int;
    pub fn ssd_steps_fwd(dims: *const SsdStepDims, nsteps: i64, dtype: c_int, state: *mut f32, reset: *const u8,
        x: *const c_void, dt: *const c_void, a: *const f32, bm: *const c_void, cm: *const c_void, d: *const f32,
        y: *mut c_void, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_chunk_scan_bwd_workspace_bytes(dims: *const SsdDims, dtype: c_int, out_bytes: *mut usize) -> c_int;
    pub fn ssd_chunk_scan_bwd(dims: *const SsdDims, dtype: c_int, x: *const c_void, dt: *const c_void,
        a: *const f32, bm: *const c_void, cm: *const c_void, d: *const f32, initial_states: *const f32,
        reset: *const u8, dy: *const c_void, dfinal_states: *const f32, dx: *mut c_void, ddt: *mut c_void,
        da: *mut f32, db: *mut c_void, dc: *mut c_void, dd: *mut f32, dinitial_states: *mut f32,
        workspace: *mut c_void, workspace_bytes: usize, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_pre_fwd(dims: *const SsdBlockDims, dtype: c_int, zxbcdt: *const c_void, conv_w: *const f32,
        conv_b: *const f32, dt_bias: *const f32, conv_state_in: *const c_void, conv_state_out: *mut c_void,
        x: *mut c_void, bm: *mut c_void, cm: *mut c_void, dt: *mut c_void, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_pre_reset_fwd(dims: *const SsdBlockDims, dtype: c_int, zxbcdt: *const c_void,
        conv_w: *const f32, conv_b: *const f32, dt_bias: *const f32, conv_state_in: *const c_void,
        conv_state_out: *mut c_void, reset: *const u8, x: *mut c_void, bm: *mut c_void, cm: *mut c_void,
        dt: *mut c_void, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_proj_fwd(rows: i64, in_features: i64, out_features: i64, out_ld: i64, dtype: c_int,
        u: *const c_void, w: *const c_void, out: *mut c_void, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_post_fwd(dims: *const SsdBlockDims, dtype: c_int, y: *const c_void, zxbcdt: *const c_void,
        norm_w: *const f32, eps: f32, out: *mut c_void, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_post_proj_fwd(dims: *const SsdBlockDims, dtype: c_int, y: *const c_void, zxbcdt: *const c_void,
        norm_w: *const f32, eps: f32, w: *const c_void, out_features: i64, out_ld: i64, out: *mut c_void,
        hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_step_fwd(dims: *const SsdBlockDims, dtype: c_int, d_model: i64, u: *const c_void, w_in: *const c_void,
        conv_w: *const f32, conv_b: *const f32, dt_bias: *const f32, a: *const f32, d: *const f32, norm_w: *const f32,
        eps: f32, w_out: *const c_void, conv_state: *mut c_void, ssm_state: *mut f32, out: *mut c_void,
        hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_bwd_workspace_bytes(dims: *const SsdBlockDims, dtype: c_int, out_bytes: *mut usize) -> c_int;
    pub fn ssd_block_post_bwd(dims: *const SsdBlockDims, dtype: c_int, y: *const c_void, zxbcdt: *const c_void,
        norm_w: *const f32, eps: f32, dout: *const c_void, dy: *mut c_void, dzxbcdt: *mut c_void, dnorm_w: *mut f32,
        workspace: *mut c_void, workspace_bytes: usize, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_post_bwd_yn(dims: *const SsdBlockDims, dtype: c_int, y: *const c_void, zxbcdt: *const c_void,
        norm_w: *const f32, eps: f32, dout: *const c_void, dy: *mut c_void, dzxbcdt: *mut c_void, dnorm_w: *mut f32,
        yn_out: *mut c_void, workspace: *mut c_void, workspace_bytes: usize, hip_stream: *mut c_void) -> c_int;
    pub fn ssd_block_pre_bwd(dims: *const SsdBlockDims, dtype: c_int, zxbcdt: *const c_void, conv_w: *const f32,
        conv_b: *const f32, dt_bias: *const f32, conv_state_in: *const c_void, reset: *const u8, dx: *const c_void,
        db: *const c_void, dc: *const c_void, ddt: *const c_void, dconv_state_out: *const c_void,
        dzxbcdt: *mut c_void, dconv_w: *mut f32, dconv_b: *mut f32, ddt_bias: *mut f32,
        dconv_state_in: *mut c_void, workspace: *mut c_void, workspace_bytes: usize, hip_stream: *mut c_void) -> c_int;
}

/// Maps a return code to `anyhow`, with the library's message (malloc'd; freed here).
fn check(rc: c_int) -> Result<()> {
    if rc == 0 {
        return Ok(());
    }
    let p = unsafe { ssd_get_and_reset_last_err() };
    let msg = if p.is_null() {
        "unknown".to_string()
    } else {
        let s = unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned();
        unsafe { libc::free(p as *mut c_void) };
        s
    };
    bail!("ssd error {rc}: {msg}")
}

fn dtype_code(t: &Tensor) -> Result<c_int> {
    match t.kind() {
        Kind::Float => Ok(SSD_DTYPE_F32),
        Kind::BFloat16 => Ok(SSD_DTYPE_BF16),
        k => bail!("SSD tensors must be f32 or bf16, got {k:?}"),
    }
}

fn opt_f32(t: Option<&Tensor>) -> *const f32 {
    t.map_or(std::ptr::null(), |t| t.data_ptr() as *const f32)
}

fn opt_u8(t: Option<&Tensor>) -> *const u8 {
    t.map_or(std::ptr::null(), |t| t.data_ptr() as *const u8)
}

/// A raw HIP stream handle (`hipStream_t`) as the library takes it; `None` is the legacy default stream.
pub type StreamHandle = Option<*mut c_void>;

fn stream_ptr(stream: StreamHandle) -> *mut c_void {
    stream.unwrap_or(std::ptr::null_mut())
}

extern "C" {
    /// The getter this binding needs from the vendored torch shim (`vendor/torch-sys-0.25.0/libtch/torch_api.{h,cpp}`,
    /// next to the graph stream-scope helpers at `torch_api.cpp:408-464`): the raw handle of the calling thread's
    /// current stream on `device_index`, i.e. the capture stream while `at_cuda_graph_stream_begin` is in scope.
    /// INTEGRATION.md gives the patch.  Errors go to the shim's thread-local `torch_last_err`, as for its other calls.
    pub fn at_cuda_current_stream(device_index: i64) -> *mut c_void;
}

/// The current stream of `device` for the calling thread: pass it to the wrappers below so that the kernels land
/// on the stream torch's own work is on (and inside a graph capture, `train/update.rs:206-330`).
pub fn current_stream(device: tch::Device) -> Result<StreamHandle> {
    match device {
        tch::Device::Cuda(index) => {
            let handle = unsafe { at_cuda_current_stream(index as i64) };
            // the shim's own error slot, read the way `torch/cuda/graph.rs:107-119` reads it
            let err = unsafe { torch_sys::get_and_reset_last_err() };
            if !err.is_null() {
                let msg = unsafe { CStr::from_ptr(err) }.to_string_lossy().into_owned();
                unsafe { libc::free(err.cast()) };
                bail!("at_cuda_current_stream: {msg}");
            }
            Ok(Some(handle))
        }
        other => bail!("SSD runs on a GPU stream, got device {other:?}"),
    }
}

fn require(name: &str, t: &Tensor, shape: &[i64], kind: Kind) -> Result<()> {
    if !t.device().is_cuda() {
        bail!("SSD {name} must be on the GPU, got {:?}", t.device());
    }
    if t.size() != shape {
        bail!("SSD {name} must have shape {shape:?}, got {:?}", t.size());
    }
    if t.kind() != kind {
        bail!("SSD {name} must be {kind:?}, got {:?}", t.kind());
    }
    if !t.is_contiguous() {
        bail!("SSD {name} must be contiguous");
    }
    Ok(())
}

fn scan_dims(x: &Tensor, b: &Tensor, chunk: i64) -> Result<SsdDims> {
    let (xs, bs) = (x.size(), b.size());
    if xs.len() != 4 {
        bail!("SSD x must be rank-4 [batch, seqlen, nheads, headdim], got {xs:?}");
    }
    if bs.len() != 4 {
        bail!("SSD B must be rank-4 [batch, seqlen, ngroups, dstate], got {bs:?}");
    }
    Ok(SsdDims { batch: xs[0], seqlen: xs[1], nheads: xs[2], headdim: xs[3], dstate: bs[3], ngroups: bs[2], chunk })
}

fn validate_scan(dims: &SsdDims, x: &Tensor, dt: &Tensor, a: &Tensor, b: &Tensor, c: &Tensor, d: Option<&Tensor>,
                 initial_states: Option<&Tensor>, reset: Option<&Tensor>) -> Result<()> {
    let k = x.kind();
    require("x", x, &[dims.batch, dims.seqlen, dims.nheads, dims.headdim], k)?;
    require("dt", dt, &[dims.batch, dims.seqlen, dims.nheads], k)?;
    require("A", a, &[dims.nheads], Kind::Float)?;
    require("B", b, &[dims.batch, dims.seqlen, dims.ngroups, dims.dstate], k)?;
    require("C", c, &[dims.batch, dims.seqlen, dims.ngroups, dims.dstate], k)?;
    if let Some(d) = d {
        require("D", d, &[dims.nheads], Kind::Float)?;
    }
    if let Some(s) = initial_states {
        require("initial_states", s, &[dims.batch, dims.nheads, dims.headdim, dims.dstate], Kind::Float)?;
    }
    if let Some(r) = reset {
        require("reset", r, &[dims.batch, dims.seqlen], Kind::Uint8)?;
    }
    Ok(())
}

/// SSD chunk-scan forward: y `[B,L,H,P]` (x's kind) and final states `[B,H,P,N]` f32.
/// `reset` `[B,L]` u8: a non-zero entry restarts that row's state from zero before the timestep.
/// `stream`: where the kernels are issued -- `current_stream(x.device())?` for torch's current stream (what a caller
/// inside the captured update must pass), `None` for the legacy default stream.
pub fn ssd_chunk_scan(x: &Tensor, dt: &Tensor, a: &Tensor, b: &Tensor, c: &Tensor, d: Option<&Tensor>, chunk: i64,
                      initial_states: Option<&Tensor>, reset: Option<&Tensor>, stream: StreamHandle)
                      -> Result<(Tensor, Tensor)> {
    let dims = scan_dims(x, b, chunk)?;
    validate_scan(&dims, x, dt, a, b, c, d, initial_states, reset)?;
    let mut need = 0usize;
    check(unsafe { ssd_workspace_bytes(&dims, &mut need) })?;
    let ws = Tensor::empty([need as i64], (Kind::Uint8, x.device()));
    let y = Tensor::empty_like(x);
    let fin = Tensor::empty([dims.batch, dims.nheads, dims.headdim, dims.dstate], (Kind::Float, x.device()));
    check(unsafe {
        ssd_chunk_scan_reset_fwd(&dims, dtype_code(x)?, x.data_ptr(), dt.data_ptr(), a.data_ptr() as *const f32,
                                 b.data_ptr(), c.data_ptr(), opt_f32(d), opt_f32(initial_states), opt_u8(reset),
                                 y.data_ptr(), fin.data_ptr() as *mut f32, ws.data_ptr(), need, stream_ptr(stream))
    })?;
    Ok((y, fin))
}

/// The same into caller-owned outputs and without any allocation (graph capture, serving loops): scratch comes
/// from the library's static array, so shapes whose workspace exceeds `SSD_STATIC_SCRATCH_BYTES` are refused
/// unless they run as one launch of the one-pass kernel.  Calls that overlap on one GPU race on that array.
pub fn ssd_chunk_scan_noalloc(x: &Tensor, dt: &Tensor, a: &Tensor, b: &Tensor, c: &Tensor, d: Option<&Tensor>,
                              chunk: i64, initial_states: Option<&Tensor>, reset: Option<&Tensor>, y: &mut Tensor,
                              final_states: &mut Tensor, stream: StreamHandle) -> Result<()> {
    let dims = scan_dims(x, b, chunk)?;
    validate_scan(&dims, x, dt, a, b, c, d, initial_states, reset)?;
    require("y", y, &x.size(), x.kind())?;
    require("final_states", final_states, &[dims.batch, dims.nheads, dims.headdim, dims.dstate], Kind::Float)?;
    check(unsafe {
        ssd_chunk_scan_noalloc_fwd(&dims, dtype_code(x)?, x.data_ptr(), dt.data_ptr(), a.data_ptr() as *const f32,
                                   b.data_ptr(), c.data_ptr(), opt_f32(d), opt_f32(initial_states), opt_u8(reset),
                                   y.data_ptr(), final_states.data_ptr() as *mut f32, stream_ptr(stream))
    })
}

/// Advances `state` `[B,H,P,N]` f32 in place by one timestep; returns y `[B,H,P]`.
pub fn ssd_step(state: &mut Tensor, x: &Tensor, dt: &Tensor, a: &Tensor, b: &Tensor, c: &Tensor,
                d: Option<&Tensor>, stream: StreamHandle) -> Result<Tensor> {
    let (ss, bs) = (state.size(), b.size());
    if ss.len() != 4 || bs.len() != 3 {
        bail!("SSD state must be [B,H,P,N] and B [B,G,N], got {ss:?} and {bs:?}");
    }
    let dims = SsdStepDims { batch: ss[0], nheads: ss[1], headdim: ss[2], dstate: ss[3], ngroups: bs[1] };
    require("state", state, &ss, Kind::Float)?;
    require("x", x, &[ss[0], ss[1], ss[2]], x.kind())?;
    let y = Tensor::empty_like(x);
    check(unsafe {
        ssd_step_fwd(&dims, dtype_code(x)?, state.data_ptr() as *mut f32, x.data_ptr(), dt.data_ptr(),
                     a.data_ptr() as *const f32, b.data_ptr(), c.data_ptr(), opt_f32(d), y.data_ptr(),
                     stream_ptr(stream))
    })?;
    Ok(y)
}

/// `nsteps` timesteps in one launch (inputs `[B,T,...]`), `reset` `[B,T]` u8 marking rows to zero right before a
/// step: the rollout's advance -> reset slots -> forward (`train/rollout.rs:209-235`) as one call.
pub fn ssd_steps(state: &mut Tensor, x: &Tensor, dt: &Tensor, a: &Tensor, b: &Tensor, c: &Tensor, d: Option<&Tensor>,
                 reset: Option<&Tensor>, stream: StreamHandle) -> Result<Tensor> {
    let (ss, xs, bs) = (state.size(), x.size(), b.size());
    if ss.len() != 4 || xs.len() != 4 || bs.len() != 4 {
        bail!("SSD steps: state [B,H,P,N], x [B,T,H,P], B [B,T,G,N], got {ss:?}, {xs:?}, {bs:?}");
    }
    let dims = SsdStepDims { batch: ss[0], nheads: ss[1], headdim: ss[2], dstate: ss[3], ngroups: bs[2] };
    let y = Tensor::empty_like(x);
    check(unsafe {
        ssd_steps_fwd(&dims, xs[1], dtype_code(x)?, state.data_ptr() as *mut f32, opt_u8(reset), x.data_ptr(),
                      dt.data_ptr(), a.data_ptr() as *const f32, b.data_ptr(), c.data_ptr(), opt_f32(d), y.data_ptr(),
                      stream_ptr(stream))
    })?;
    Ok(y)
}

/// Gradients of the scan (what a custom autograd function's `backward` would call).
pub struct SsdGrads {
    pub dx: Tensor,
    pub ddt: Tensor,
    pub da: Tensor,
    pub db: Tensor,
    pub dc: Tensor,
    pub dd: Option<Tensor>,
    pub dinitial_states: Option<Tensor>,
}

pub fn ssd_chunk_scan_backward(x: &Tensor, dt: &Tensor, a: &Tensor, b: &Tensor, c: &Tensor, d: Option<&Tensor>,
                               dy: &Tensor, chunk: i64, initial_states: Option<&Tensor>, reset: Option<&Tensor>,
                               dfinal_states: Option<&Tensor>, need_dinitial_states: bool, stream: StreamHandle)
                               -> Result<SsdGrads> {
    let dims = scan_dims(x, b, chunk)?;
    validate_scan(&dims, x, dt, a, b, c, d, initial_states, reset)?;
    require("dy", dy, &x.size(), x.kind())?;
    let code = dtype_code(x)?;
    let mut need = 0usize;
    check(unsafe { ssd_chunk_scan_bwd_workspace_bytes(&dims, code, &mut need) })?;
    let dev = x.device();
    let ws = Tensor::empty([need as i64], (Kind::Uint8, dev));
    let state_shape = [dims.batch, dims.nheads, dims.headdim, dims.dstate];
    let g = SsdGrads {
        dx: Tensor::empty_like(x),
        ddt: Tensor::empty_like(dt),
        da: Tensor::empty([dims.nheads], (Kind::Float, dev)),
        db: Tensor::empty_like(b),
        dc: Tensor::empty_like(c),
        dd: d.map(|_| Tensor::empty([dims.nheads], (Kind::Float, dev))),
        dinitial_states: if need_dinitial_states { Some(Tensor::empty(state_shape, (Kind::Float, dev))) } else { None },
    };
    let opt_mut = |t: &Option<Tensor>| t.as_ref().map_or(std::ptr::null_mut(), |t| t.data_ptr() as *mut f32);
    check(unsafe {
        ssd_chunk_scan_bwd(&dims, code, x.data_ptr(), dt.data_ptr(), a.data_ptr() as *const f32, b.data_ptr(),
                           c.data_ptr(), opt_f32(d), opt_f32(initial_states), opt_u8(reset), dy.data_ptr(),
                           opt_f32(dfinal_states), g.dx.data_ptr(), g.ddt.data_ptr(), g.da.data_ptr() as *mut f32,
                           g.db.data_ptr(), g.dc.data_ptr(), opt_mut(&g.dd), opt_mut(&g.dinitial_states),
                           ws.data_ptr(), need, stream_ptr(stream))
    })?;
    Ok(g)
}
