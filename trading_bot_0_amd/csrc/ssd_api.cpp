// C ABI of libssd_hip: argument validation, error slot, workspace carving, stage sequencing.
// Conventions follow the reference's own extern "C" shim (thread-local malloc'd error string,
// vendor/torch-sys-0.25.0/libtch/torch_api.h:18-24,33 and torch_api.cpp:32,84-88) and its op
// wrappers' validate-then-call shape (trading_bots/src/torch/fa4.rs:145-191).
#include "../../include/ssd_hip.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include <atomic>

#include "ssd_launch.h"

// Scratch of ssd_chunk_scan_noalloc_fwd: device memory that exists from the moment the library's code object is
// loaded on a GPU until the process ends, so that entry point never allocates.  Every call on a GPU shares that GPU's
// copy; host code reaches it only through the address hipGetSymbolAddress returns (static_scratch_address below).
constexpr size_t kStaticScratchBytes = (size_t)64 << 20;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

namespace {

thread_local char *g_last_err = nullptr;

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    free(g_last_err);
    g_last_err = strdup(buf);
    return code;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

#define REQUIRE_PTR(name)                                                                      \
    do {                                                                                       \
        if ((name) == nullptr) return fail(SSD_ERR_INVALID, "ssd: " #name " must not be NULL"); \
        if (!aligned16(name)) return fail(SSD_ERR_INVALID, "ssd: " #name " must be 16-byte aligned"); \
    } while (0)
#define OPTIONAL_PTR(name)                                                                     \
    do {                                                                                       \
        if ((name) != nullptr && !aligned16(name))                                             \
            return fail(SSD_ERR_INVALID, "ssd: " #name " must be 16-byte aligned");            \
    } while (0)

int check_dtype(int dtype) {
    if (dtype != SSD_DTYPE_F32 && dtype != SSD_DTYPE_BF16 && dtype != SSD_DTYPE_BF16_Y32)
        return fail(SSD_ERR_INVALID,
                    "ssd: dtype must be 0 (float32), 1 (bfloat16) or 2 (bfloat16 with float32 y), got %d", dtype);
    return SSD_OK;
}

int check_state_dims(int64_t H, int64_t P, int64_t N, int64_t G) {
    if (H <= 0 || P <= 0 || N <= 0 || G <= 0)
        return fail(SSD_ERR_INVALID, "ssd: nheads, headdim, dstate, ngroups must be positive, got %lld %lld %lld %lld",
                    (long long)H, (long long)P, (long long)N, (long long)G);
    if (H % G != 0)
        return fail(SSD_ERR_INVALID, "ssd: nheads (%lld) must be divisible by ngroups (%lld)", (long long)H,
                    (long long)G);
    if (N != 16 && N != 32 && N != 64 && N != 128)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: dstate must be 16, 32, 64 or 128, got %lld", (long long)N);
    if (P % 8 != 0 || P > 64)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: headdim must be a multiple of 8 and at most 64, got %lld",
                    (long long)P);
    return SSD_OK;
}

// Validates dims and converts them to the launchers' 32-bit shape.
int make_shape(const ssd_dims *d, int dtype, ssd::ScanShape *out) {
    if (d == nullptr) return fail(SSD_ERR_INVALID, "ssd: dims must not be NULL");
    if (int rc = check_dtype(dtype)) return rc;
    if (d->batch <= 0 || d->seqlen <= 0 || d->chunk <= 0)
        return fail(SSD_ERR_INVALID, "ssd: batch, seqlen, chunk must be positive, got %lld %lld %lld",
                    (long long)d->batch, (long long)d->seqlen, (long long)d->chunk);
    if (int rc = check_state_dims(d->nheads, d->headdim, d->dstate, d->ngroups)) return rc;
    if (d->chunk != 32 && d->chunk != 64 && d->chunk != 128 && d->chunk != 256)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: chunk must be 32, 64, 128 or 256, got %lld", (long long)d->chunk);
    if (d->nheads > 1024) return fail(SSD_ERR_UNSUPPORTED, "ssd: nheads must be at most 1024");
    const int64_t nc = (d->seqlen + d->chunk - 1) / d->chunk;
    const int64_t kmax = 0x7fffffff;
    if (d->batch * nc * d->nheads > kmax || d->batch * d->seqlen > kmax ||
        d->batch * d->nheads * (d->headdim * d->dstate / 4) / 256 + 1 > kmax)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: batch*nchunks*nheads or batch*seqlen exceeds 2^31-1");
    ssd::ScanShape s{(int)d->batch, (int)d->seqlen, (int)d->nheads, (int)d->headdim,
                     (int)d->dstate, (int)d->ngroups, (int)d->chunk, (int)nc};
    const int eb = dtype == SSD_DTYPE_F32 ? 4 : 2;
    if (ssd::chunk_scan_lds_bytes(s, eb) > ssd::kLdsLimitBytes || ssd::chunk_state_lds_bytes(s, eb) > ssd::kLdsLimitBytes)
        return fail(SSD_ERR_UNSUPPORTED,
                    "ssd: headdim %lld / dstate %lld / chunk %lld needs more than 160 KiB of LDS in %s mode",
                    (long long)d->headdim, (long long)d->dstate, (long long)d->chunk, eb == 2 ? "bf16" : "float32");
    if (ssd::chunk_cumsum_lds_bytes(s) > ssd::kLdsLimitBytes)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: nheads %lld with chunk %lld needs more than 160 KiB of LDS in stage 1",
                    (long long)d->nheads, (long long)d->chunk);
    *out = s;
    return SSD_OK;
}

// The fused stage 2+3 kernel parallelises over (batch, head) sequences only; below this many sequences
// the separate stages, which parallelise over chunks as well, fill the chip better.
constexpr int64_t kFusedStatePassingMinSequences = 512;
// The one-pass kernel runs one workgroup per 8 units of 32 head-dim columns and is parallel over sequences
// only; below this many workgroups the staged kernels (parallel over chunks too) fill the chip better.
constexpr int64_t kOnePassMinWorkgroups = 96;

struct Workspace {
    size_t dtcs_off, st_off, total;
};

Workspace carve(const ssd::ScanShape &s) {
    Workspace w;
    const size_t dtcs = (size_t)s.B * s.H * s.nc * 4 * s.Q * sizeof(float);
    const size_t st = (size_t)s.B * s.nc * s.H * s.P * s.N * sizeof(float);
    w.dtcs_off = 0;
    w.st_off = align_up(dtcs, 256);
    w.total = w.st_off + align_up(st, 256);
    return w;
}

bool takes_one_pass(const ssd::ScanShape &s, int dtype) {
    int segments;
    return ssd::fused_scan_plan(s, dtype, &segments) == 1;
}

int hip_fail(hipError_t e, const char *what) {
    return fail(SSD_ERR_RUNTIME, "ssd: %s failed: %s", what, hipGetErrorString(e));
}

// Device address of g_static_scratch on the current device.  In host code the array's name is only a handle for the
// runtime's symbol lookup, not a device address, and every GPU holds its own copy at its own address: the address
// is looked up once per device, with that device current, and kept.  Lock-free: two threads that race on a
// device's first call look up the same address and store the same value.
constexpr int kMaxDevices = 64;
std::atomic<void *> g_static_scratch_ptr[kMaxDevices];

int static_scratch_address(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(SSD_ERR_UNSUPPORTED, "ssd: device index %d is beyond %d", dev, kMaxDevices - 1);
    void *p = g_static_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress of the static scratch array");
        if (p == nullptr) return fail(SSD_ERR_RUNTIME, "ssd: the static scratch array has no device address");
        g_static_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return SSD_OK;
}

// Stages 1-4 one after the other.  mode as for launch_chunk_cumsum (0 = the forward's decays and weights).
int run_staged(const ssd::ScanShape &s, int dtype, const void *x, const void *dt, const float *A, const void *Bm,
               const void *Cm, const float *D, const float *initial_states, const uint8_t *reset, int mode, void *y,
               float *final_states, float *dtcs, float *states, hipStream_t st, int dt_len = 0) {
    hipError_t e = ssd::launch_chunk_cumsum(s, dtype, dt, A, reset, dtcs, st, mode, dt_len);
    if (e != hipSuccess) return hip_fail(e, "chunk_cumsum launch");
    ssd::ScanShape sp = s;  // for the kernels that read the initial state
    if (mode == 0) sp.fresh = reset;
    if ((int64_t)s.B * s.H >= kFusedStatePassingMinSequences) {
        // enough (b,h) sequences to fill the chip: stages 2 and 3 in one pass, states carried on chip
        e = ssd::launch_chunk_state_scan(sp, dtype, x, Bm, dtcs, initial_states, states, final_states, st);
        if (e != hipSuccess) return hip_fail(e, "chunk_state_passing launch");
    } else {
        e = ssd::launch_chunk_state(s, dtype, x, Bm, dtcs, states, st);
        if (e != hipSuccess) return hip_fail(e, "chunk_state launch");
        e = ssd::launch_state_passing(sp, states, dtcs, initial_states, states, final_states, st);  // in place
        if (e != hipSuccess) return hip_fail(e, "state_passing launch");
    }
    e = ssd::launch_chunk_scan(s, dtype, x, Bm, Cm, dtcs, states, D, y, st);
    if (e != hipSuccess) return hip_fail(e, "chunk_scan launch");
    return SSD_OK;
}

// Workspace of the backward pass: the scan workspace (its three scans have the same number of chunks, heads and
// state elements; the two transposed scans keep their chunk states for the anchors, so there is a second state
// array), the gathered operands (reversed ones padded to whole chunks) and the scans' float outputs.
struct BwdWorkspace {
    size_t scan_off, states2, dy_rev, x_rev, c_rev_g, b_rev_g, c_rev_h, b_fwd_h, r_rev, yb_rev, yc, gfin, gfin_t, ffin_t,
        init_t, dfin_t, e1, dd, u, parts, anchor, da_part, dt_parts, a_parts, total;
};

// Which kernels a backward pass of a given shape runs on (a function of shape and dtype only: the workspace is laid
// out for it).
struct BwdPlan {
    bool fast_r;        // the adjoint scan on the one-pass kernel (else staged, with gathered operands)
    bool fast_t;        // the two transposed scans on the one-pass kernel
    bool sum_on_chip;   // ... on its transposed kinds, which sum dB and dC over a group's heads themselves
    bool rows_in_scan;  // the adjoint scan with the row products in its epilogue (writes dx; no float r)
    int anchor_stride;  // tiles between two meetings of the transposed scans' states (the decay gradient's anchors)
};

// The decay gradient is anchored where the two transposed scans' states meet; between two anchors it sums the
// per-step terms, whose rounding errors add up with the square root of the distance.  Meeting at every tile costs
// a state per head and tile written by one scan and read by the other (at the policy shape 0.54 GB each way, a tenth
// of the pass's time); in bf16 mode, where the gradient is rounded to 8 bits, runs of 512 steps stay three orders of
// magnitude below that rounding.
constexpr int kBf16AnchorStride = 8;

BwdPlan plan_bwd(const ssd::ScanShape &s, const ssd::ScanShape &sT, int dtype) {
    const int inner = dtype == SSD_DTYPE_F32 ? SSD_DTYPE_F32 : SSD_DTYPE_BF16_Y32;  // the scans write float y
    // The one-pass kernel reverses time itself (reads the forward tensors, writes its output in forward order), reads
    // an x that a group's heads share in place and writes the state entering every 64-step tile, which is what the
    // staged kernels leave in their state array.
    auto one_pass = [&](const ssd::ScanShape &shape) {
        const int waves = ssd::fused_scan_waves(shape, inner);
        if (waves == 0 || shape.Q != 64) return false;
        const int64_t groups = (int64_t)shape.B * shape.G * ((shape.H / shape.G) * (shape.P / 32) / waves);
        return (waves == 8 && groups >= kOnePassMinWorkgroups) || (waves == 2 && groups >= 4 * kOnePassMinWorkgroups);
    };
    BwdPlan p;
    // bf16, headdim 32, eight heads per group, enough workgroups
    p.sum_on_chip = inner != SSD_DTYPE_F32 && ssd::transposed_scan_supported(sT, s.G) &&
                    (int64_t)s.B * (s.H / 8) * (s.N / 32) >= kOnePassMinWorkgroups;
    p.fast_r = one_pass(s);  // (the padded length does not enter)
    p.fast_t = p.sum_on_chip || one_pass(sT);
    p.rows_in_scan = p.sum_on_chip && p.fast_r && ssd::adjoint_rows_scan_supported(s);
    p.anchor_stride = (p.rows_in_scan && ssd::bwd_ddt_anchor_stride_supported(s, (s.N + 31) / 32)) ? kBf16AnchorStride : 1;
    return p;
}

BwdWorkspace carve_bwd(const ssd::ScanShape &s, const ssd::ScanShape &sT, int elem_bytes, const BwdPlan &plan) {
    BwdWorkspace w;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off += align_up(bytes, 256);
        return at;
    };
    auto take_if = [&](bool used, size_t bytes) { return take(used ? bytes : 0); };
    const size_t BL = (size_t)s.B * s.L, BLp = (size_t)s.B * s.nc * s.Q;  // true and padded rows
    const size_t HP = (size_t)s.H * s.P, HN = (size_t)s.H * s.N, GN = (size_t)s.G * s.N;
    const size_t st = (size_t)s.B * s.H * s.P * s.N * sizeof(float);
    // (the transposed scans of a 128-wide state run on twice the heads: more stage-1 rows, the same state elements)
    // (... or, where no scan of the pass runs on the staged kernels, the tile states one transposed scan keeps for
    // the other)
    w.scan_off = take(plan.anchor_stride > 1 ? (size_t)(s.nc / plan.anchor_stride + 1) * st
                                             : sT.H > s.H ? carve(sT).total : carve(s).total);
    w.states2 = take_if(!plan.sum_on_chip, (size_t)s.nc * st);
    w.dy_rev = take_if(!plan.fast_r || !plan.fast_t, BLp * HP * elem_bytes);
    w.x_rev = take_if(!plan.fast_t, BLp * HP * elem_bytes);
    w.c_rev_g = take_if(!plan.fast_r, BLp * GN * elem_bytes);
    w.b_rev_g = take_if(!plan.fast_r, BLp * GN * elem_bytes);
    w.c_rev_h = take_if(!plan.fast_t, BLp * HN * elem_bytes);
    w.b_fwd_h = take_if(!plan.fast_t, BL * HN * elem_bytes);
    w.r_rev = take_if(!plan.rows_in_scan, BLp * HP * sizeof(float));
    w.yb_rev = take_if(!plan.sum_on_chip, BLp * HN * sizeof(float));
    w.yc = take_if(!plan.sum_on_chip, BL * HN * sizeof(float));
    w.gfin = take(st);
    w.gfin_t = take(st);
    w.ffin_t = take(st);
    w.init_t = take(st);
    w.dfin_t = take(st);
    w.e1 = take(2 * BL * s.H * sizeof(float));  // or the (e1, dd) pairs of the adjoint scan with row products
    w.dd = take(BL * s.H * sizeof(float));
    w.u = take(BL * s.H * sizeof(float));
    w.parts = take(BL * s.H * (size_t)((s.N + 31) / 32) * sizeof(float));
    w.anchor = take((size_t)s.B * (s.nc + 1) * s.H * sizeof(double) * (size_t)((s.N + 31) / 32));  // or its pieces
    w.da_part = take((size_t)2 * s.B * s.nc * s.H * sizeof(double));  // and the parts of dD behind them
    // dt and A once per part of a head, for the transposed scans of a state scanned in parts
    w.dt_parts = take_if(sT.H > s.H, BL * sT.H * elem_bytes);
    w.a_parts = take_if(sT.H > s.H, (size_t)sT.H * sizeof(float));
    w.total = off;
    return w;
}

constexpr int64_t kBackwardChunk = 64;

// The backward pass runs the forward's stage kernels on the transposed state ([N,P] per head, B and C per head),
// so the transposed shape must be one they take as well.
int make_bwd_shapes(const ssd_dims *dims, int dtype, ssd::ScanShape *s, ssd::ScanShape *sT) {
    if (dims == nullptr) return fail(SSD_ERR_INVALID, "ssd: dims must not be NULL");
    if (dtype != SSD_DTYPE_F32 && dtype != SSD_DTYPE_BF16)
        return fail(SSD_ERR_INVALID, "ssd: the backward pass takes dtype 0 (float32) or 1 (bfloat16), got %d", dtype);
    // The pass tiles time by at most kBackwardChunk steps whatever chunk the caller names (it owns its workspace
    // layout): the decay gradient sums rounding errors over a chunk, see ssd_backward_kernels.hip.
    ssd_dims own = *dims;
    if (own.chunk > kBackwardChunk) own.chunk = kBackwardChunk;
    if (int rc = make_shape(&own, dtype, s)) return rc;
    if (dims->headdim < 16 || (dims->headdim & (dims->headdim - 1)) != 0)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: the backward pass needs headdim 16, 32 or 64, got %lld", (long long)dims->headdim);
    // The transposed state is [dstate, headdim] per head, and the stage kernels take a head-dim of at most 64: a
    // 128-wide state is scanned as two parts of 64 rows, i.e. as twice as many heads in groups of two that share
    // their B and C operands -- the same memory, read as [.., 2 nheads, 64, ..].
    const int64_t parts = dims->dstate > 64 ? 2 : 1;
    const ssd_dims t = {dims->batch, dims->seqlen, dims->nheads * parts, dims->dstate / parts, dims->headdim, dims->nheads,
                        own.chunk};
    return make_shape(&t, dtype, sT);
}

}  // namespace

extern "C" {

int ssd_version(void) { return 100; }

char *ssd_get_and_reset_last_err(void) {
    char *tmp = g_last_err;
    g_last_err = nullptr;
    return tmp;
}

int ssd_workspace_bytes(const ssd_dims *dims, size_t *out_bytes) {
    if (out_bytes == nullptr) return fail(SSD_ERR_INVALID, "ssd: out_bytes must not be NULL");
    ssd::ScanShape s;
    // the workspace layout does not depend on dtype; validate with the tighter float32 LDS bound
    // only when asked to run, so use bf16 here
    if (int rc = make_shape(dims, SSD_DTYPE_BF16, &s)) return rc;
    *out_bytes = carve(s).total;
    return SSD_OK;
}

int ssd_chunk_cumsum_fwd(const ssd_dims *dims, int dtype, const void *dt, const float *A, float *dtcs,
                         void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(dt);
    REQUIRE_PTR(A);
    REQUIRE_PTR(dtcs);
    hipError_t e = ssd::launch_chunk_cumsum(s, dtype, dt, A, nullptr, dtcs, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "chunk_cumsum launch");
}

int ssd_chunk_state_fwd(const ssd_dims *dims, int dtype, const void *x, const void *Bm, const float *dtcs,
                        float *chunk_states, void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(x);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(dtcs);
    REQUIRE_PTR(chunk_states);
    hipError_t e = ssd::launch_chunk_state(s, dtype, x, Bm, dtcs, chunk_states, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "chunk_state launch");
}

int ssd_chunk_state_passing_fwd(const ssd_dims *dims, int dtype, const void *x, const void *Bm, const float *dtcs,
                                const float *initial_states, float *prev_states, float *final_states,
                                void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(x);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(dtcs);
    REQUIRE_PTR(prev_states);
    OPTIONAL_PTR(initial_states);
    OPTIONAL_PTR(final_states);
    hipError_t e = ssd::launch_chunk_state_scan(s, dtype, x, Bm, dtcs, initial_states, prev_states, final_states,
                                                (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "chunk_state_passing launch");
}

int ssd_state_passing_fwd(const ssd_dims *dims, const float *chunk_states, const float *dtcs,
                          const float *initial_states, float *prev_states, float *final_states,
                          void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, SSD_DTYPE_BF16, &s)) return rc;
    REQUIRE_PTR(chunk_states);
    REQUIRE_PTR(dtcs);
    REQUIRE_PTR(prev_states);
    OPTIONAL_PTR(initial_states);
    OPTIONAL_PTR(final_states);
    hipError_t e = ssd::launch_state_passing(s, chunk_states, dtcs, initial_states, prev_states, final_states,
                                             (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "state_passing launch");
}

int ssd_chunk_scan_stage_fwd(const ssd_dims *dims, int dtype, const void *x, const void *Bm, const void *Cm,
                             const float *dtcs, const float *prev_states, const float *D, void *y,
                             void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(x);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(Cm);
    REQUIRE_PTR(dtcs);
    REQUIRE_PTR(prev_states);
    REQUIRE_PTR(y);
    OPTIONAL_PTR(D);
    hipError_t e = ssd::launch_chunk_scan(s, dtype, x, Bm, Cm, dtcs, prev_states, D, y, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "chunk_scan launch");
}

int ssd_chunk_scan_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                       const void *Bm, const void *Cm, const float *D, const float *initial_states, void *y,
                       float *final_states, void *workspace, size_t workspace_bytes, void *hip_stream) {
    return ssd_chunk_scan_reset_fwd(dims, dtype, x, dt, A, Bm, Cm, D, initial_states, nullptr, y, final_states,
                                    workspace, workspace_bytes, hip_stream);
}

// Scratch of the forward on segments: the segments' decays [B, S, H], then their states [B, S, H, P, N] (fewer than the
// chunk states the workspace is sized for)
size_t segment_decay_bytes(const ssd::ScanShape &s, int segments) {
    return align_up((size_t)s.B * segments * s.H * sizeof(float), 256);
}

// What the forward of this shape uses of its workspace: nothing as one launch of the one-pass kernel, the segment
// states and decays on segments, everything carve() lays out on the staged kernels (or with a partial last round).
size_t scan_scratch_bytes(const ssd::ScanShape &s, int dtype) {
    int segments = 1;
    const int plan = ssd::fused_scan_plan(s, dtype, &segments);
    if (plan == 1 && ssd::fused_scan_tail_rows(s, dtype) == 0) return 0;
    if (plan == 2)
        return segment_decay_bytes(s, segments) + (size_t)s.B * segments * s.H * s.P * s.N * sizeof(float);
    return carve(s).total;
}

// The forward proper, arguments checked: the way the plan says for this shape, with `workspace` (carve(s).total bytes,
// or anything at all when scan_scratch_bytes says the shape needs none) as scratch.
static int scan_forward(const ssd::ScanShape &s, int dtype, const void *x, const void *dt, const float *A, const void *Bm,
                        const void *Cm, const float *D, const float *initial_states, const uint8_t *reset, void *y,
                        float *final_states, void *workspace, hipStream_t st) {
    const Workspace w = carve(s);
    char *base = static_cast<char *>(workspace);
    float *dtcs = reinterpret_cast<float *>(base + w.dtcs_off);
    float *states = reinterpret_cast<float *>(base + w.st_off);
    // One batch of sequences, the way the plan says.  The workspace is carved for the whole batch and so holds any
    // part of it.
    auto forward = [&](const ssd::ScanShape &part, const void *px, const void *pdt, const void *pb, const void *pc,
                       const float *pinit, const uint8_t *preset, void *py, float *pfinal) -> int {
        int segments = 1;
        const int plan = ssd::fused_scan_plan(part, dtype, &segments);
        hipError_t e;
        if (plan == 1) {
            e = ssd::launch_fused_scan(part, dtype, px, pdt, A, pb, pc, D, pinit, preset, py, pfinal, st);
            return e == hipSuccess ? SSD_OK : hip_fail(e, "one-pass scan launch");
        }
        if (plan == 2) {
            // too few sequences for one workgroup per 8 units to fill the chip, but long ones: the one-pass kernel
            // on segments of the sequence; the segment states (fewer than the chunk states) and decays use the
            // workspace
            float *seg_decay = reinterpret_cast<float *>(base);
            float *seg_states = reinterpret_cast<float *>(base + segment_decay_bytes(part, segments));
            e = ssd::launch_fused_scan_segmented(part, dtype, segments, px, pdt, A, pb, pc, D, pinit, preset, py, pfinal,
                                                 seg_states, seg_decay, st);
            return e == hipSuccess ? SSD_OK : hip_fail(e, "segmented one-pass scan launch");
        }
        return run_staged(part, dtype, px, pdt, A, pb, pc, D, pinit, preset, 0, py, pfinal, dtcs, states, st);
    };
    // A batch that fills the chip some whole number of times and a bit: the whole rounds run as one launch of the
    // one-pass kernel, the rest as a batch of its own (cut into segments or staged, as the plan says for it) -- a
    // last round of a few workgroups would cost as long as a full one.
    const int tail_rows = ssd::fused_scan_tail_rows(s, dtype);
    if (tail_rows > 0) {
        const int main_rows = s.B - tail_rows;
        const size_t eb = dtype == SSD_DTYPE_F32 ? 4 : 2, yb = dtype == SSD_DTYPE_BF16 ? 2 : 4;
        const size_t row_x = (size_t)s.L * s.H * s.P, row_dt = (size_t)s.L * s.H, row_bc = (size_t)s.L * s.G * s.N;
        const size_t row_st = (size_t)s.H * s.P * s.N;
        auto off = [](const void *p, size_t bytes) { return p ? static_cast<const char *>(p) + bytes : nullptr; };
        ssd::ScanShape head = s, tail = s;
        head.B = main_rows;
        tail.B = tail_rows;
        if (int rc = forward(head, x, dt, Bm, Cm, initial_states, reset, y, final_states)) return rc;
        return forward(tail, off(x, main_rows * row_x * eb), off(dt, main_rows * row_dt * eb), off(Bm, main_rows * row_bc * eb),
                       off(Cm, main_rows * row_bc * eb),
                       reinterpret_cast<const float *>(off(initial_states, main_rows * row_st * 4)),
                       reinterpret_cast<const uint8_t *>(off(reset, (size_t)main_rows * s.L)),
                       const_cast<char *>(off(y, main_rows * row_x * yb)),
                       reinterpret_cast<float *>(const_cast<char *>(off(final_states, main_rows * row_st * 4))));
    }
    return forward(s, x, dt, Bm, Cm, initial_states, reset, y, final_states);
}


#define SSD_SCAN_POINTER_CHECKS \
    REQUIRE_PTR(x);             \
    REQUIRE_PTR(dt);            \
    REQUIRE_PTR(A);             \
    REQUIRE_PTR(Bm);            \
    REQUIRE_PTR(Cm);            \
    REQUIRE_PTR(y);             \
    OPTIONAL_PTR(D);            \
    OPTIONAL_PTR(initial_states); \
    OPTIONAL_PTR(final_states)

int ssd_chunk_scan_reset_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                             const void *Bm, const void *Cm, const float *D, const float *initial_states,
                             const uint8_t *reset, void *y, float *final_states, void *workspace,
                             size_t workspace_bytes, void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    SSD_SCAN_POINTER_CHECKS;
    REQUIRE_PTR(workspace);
    const Workspace w = carve(s);
    if (workspace_bytes < w.total)
        return fail(SSD_ERR_WORKSPACE, "ssd: workspace has %zu bytes, %zu needed", workspace_bytes, w.total);
    return scan_forward(s, dtype, x, dt, A, Bm, Cm, D, initial_states, reset, y, final_states, workspace,
                        (hipStream_t)hip_stream);
}

int ssd_chunk_scan_noalloc_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                               const void *Bm, const void *Cm, const float *D, const float *initial_states,
                               const uint8_t *reset, void *y, float *final_states, void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    const size_t need = scan_scratch_bytes(s, dtype);
    if (need > kStaticScratchBytes)
        return fail(SSD_ERR_WORKSPACE,
                    "ssd: this shape needs %zu bytes of scratch, the library's static scratch array holds %zu; call "
                    "ssd_chunk_scan_fwd with a workspace of ssd_workspace_bytes() instead",
                    need, kStaticScratchBytes);
    SSD_SCAN_POINTER_CHECKS;
    void *scratch = nullptr;
    if (int rc = static_scratch_address(&scratch)) return rc;
    return scan_forward(s, dtype, x, dt, A, Bm, Cm, D, initial_states, reset, y, final_states, scratch,
                        (hipStream_t)hip_stream);
}

int ssd_chunk_scan_bwd_workspace_bytes(const ssd_dims *dims, int dtype, size_t *out_bytes) {
    if (out_bytes == nullptr) return fail(SSD_ERR_INVALID, "ssd: out_bytes must not be NULL");
    ssd::ScanShape s, sT;
    if (int rc = make_bwd_shapes(dims, dtype, &s, &sT)) return rc;
    *out_bytes = carve_bwd(s, sT, dtype == SSD_DTYPE_F32 ? 4 : 2, plan_bwd(s, sT, dtype)).total;
    return SSD_OK;
}

int ssd_chunk_scan_bwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A, const void *Bm,
                       const void *Cm, const float *D, const float *initial_states, const uint8_t *reset, const void *dy,
                       const float *dfinal_states, void *dx, void *ddt, float *dA, void *dB, void *dC, float *dD,
                       float *dinitial_states, void *workspace, size_t workspace_bytes, void *hip_stream) {
    ssd::ScanShape s, sT;
    if (int rc = make_bwd_shapes(dims, dtype, &s, &sT)) return rc;
    REQUIRE_PTR(x);
    REQUIRE_PTR(dt);
    REQUIRE_PTR(A);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(Cm);
    REQUIRE_PTR(dy);
    REQUIRE_PTR(dx);
    REQUIRE_PTR(ddt);
    REQUIRE_PTR(dA);
    REQUIRE_PTR(dB);
    REQUIRE_PTR(dC);
    REQUIRE_PTR(workspace);
    OPTIONAL_PTR(D);
    OPTIONAL_PTR(initial_states);
    OPTIONAL_PTR(dfinal_states);
    OPTIONAL_PTR(dD);
    OPTIONAL_PTR(dinitial_states);
    if (dD != nullptr && D == nullptr) return fail(SSD_ERR_INVALID, "ssd: dD asked for without D");
    const int eb = dtype == SSD_DTYPE_F32 ? 4 : 2;
    const BwdPlan plan = plan_bwd(s, sT, dtype);
    const BwdWorkspace w = carve_bwd(s, sT, eb, plan);
    if (workspace_bytes < w.total)
        return fail(SSD_ERR_WORKSPACE, "ssd: backward workspace has %zu bytes, %zu needed", workspace_bytes, w.total);
    char *base = static_cast<char *>(workspace);
    auto at = [&](size_t off) { return static_cast<void *>(base + off); };
    auto atf = [&](size_t off) { return reinterpret_cast<float *>(base + off); };
    const Workspace sw = sT.H > s.H ? carve(sT) : carve(s);
    float *dtcs = atf(w.scan_off + sw.dtcs_off);  // (unused where the plan has an anchor stride: no staged kernel runs)
    float *states = plan.anchor_stride > 1 ? atf(w.scan_off) : atf(w.scan_off + sw.st_off);
    hipStream_t st = (hipStream_t)hip_stream;
    const int inner = dtype == SSD_DTYPE_F32 ? SSD_DTYPE_F32 : SSD_DTYPE_BF16_Y32;  // the scans write float y
    const int el = dtype == SSD_DTYPE_F32 ? 0 : 1;
    const int rep = s.H / s.G;
    hipError_t e;
#define BWD_LAUNCH(call, what)                      \
    do {                                            \
        e = (call);                                 \
        if (e != hipSuccess) return hip_fail(e, what); \
    } while (0)
    // The reversed sequences are padded in front to whole chunks (Lp rows), so that chunk k of a reversed scan
    // begins where chunk nc - k of the forward ends.
    const int Lp = s.nc * s.Q;
    ssd::ScanShape sR = s, sTR = sT;
    sR.L = Lp;
    sTR.L = Lp;
    float *states2 = atf(w.states2);
    // The staged kernels get their operands gathered: time-reversed copies, and one copy of a group's B or C per head.
    const bool fast_r = plan.fast_r, fast_t = plan.fast_t, sum_on_chip = plan.sum_on_chip, rows_in_scan = plan.rows_in_scan;
    const void *c_heads = Cm, *b_heads = Bm;
    if (!fast_r || !fast_t)
        BWD_LAUNCH(ssd::launch_gather_rows(el, dy, at(w.dy_rev), s.B, s.L, Lp, s.H, s.P, 1, true, st), "gather dy");
    if (!fast_r) {
        BWD_LAUNCH(ssd::launch_gather_rows(el, Cm, at(w.c_rev_g), s.B, s.L, Lp, s.G, s.N, 1, true, st), "gather C");
        BWD_LAUNCH(ssd::launch_gather_rows(el, Bm, at(w.b_rev_g), s.B, s.L, Lp, s.G, s.N, 1, true, st), "gather B");
    }
    if (!fast_t) {
        BWD_LAUNCH(ssd::launch_gather_rows(el, x, at(w.x_rev), s.B, s.L, Lp, s.H, s.P, 1, true, st), "gather x");
        BWD_LAUNCH(ssd::launch_gather_rows(el, Cm, at(w.c_rev_h), s.B, s.L, Lp, s.G, s.N, rep, true, st), "gather C per head");
        c_heads = at(w.c_rev_h);
        if (rep > 1) {
            BWD_LAUNCH(ssd::launch_gather_rows(el, Bm, at(w.b_fwd_h), s.B, s.L, s.L, s.G, s.N, rep, false, st),
                       "gather B per head");
            b_heads = at(w.b_fwd_h);
        }
    }
    const float *init_t = nullptr, *dfin_t = nullptr;
    if (initial_states != nullptr) {
        BWD_LAUNCH(ssd::launch_transpose_state(initial_states, atf(w.init_t), (long long)s.B * s.H, s.P, s.N, st), "transpose");
        init_t = atf(w.init_t);
    }
    if (dfinal_states != nullptr) {
        BWD_LAUNCH(ssd::launch_transpose_state(dfinal_states, atf(w.dfin_t), (long long)s.B * s.H, s.P, s.N, st), "transpose");
        dfin_t = atf(w.dfin_t);
    }
    auto scan = [&](const ssd::ScanShape &shape, bool fast, const void *sx, const void *sb, const void *sc, const float *sinit,
                    int mode, void *sy, float *sfinal, float *sstates, bool keep_states, int x_groups) -> int {
        // a state scanned in parts: dt and A once per part of a head
        const void *sdt = shape.H > s.H ? at(w.dt_parts) : dt;
        const float *sA = shape.H > s.H ? atf(w.a_parts) : A;
        if (fast) {
            ssd::ScanShape f = shape;
            f.mode = mode;
            f.dt_len = s.L;
            f.x_groups = x_groups;
            hipError_t err = ssd::launch_fused_scan(f, inner, sx, sdt, sA, sb, sc, nullptr, sinit, reset, sy, sfinal, st,
                                                     keep_states ? sstates : nullptr);
            return err == hipSuccess ? SSD_OK : hip_fail(err, "one-pass scan launch (backward)");
        }
        return run_staged(shape, inner, sx, sdt, sA, sb, sc, nullptr, sinit, reset, mode, sy, sfinal, dtcs, sstates, st, s.L);
    };
    if (sT.H > s.H) {
        BWD_LAUNCH(ssd::launch_replicate_columns(el, dt, at(w.dt_parts), (long long)s.B * s.L, s.H, sT.H / s.H, st), "dt per part");
        BWD_LAUNCH(ssd::launch_replicate_columns(0, A, at(w.a_parts), 1, s.H, sT.H / s.H, st), "A per part");
    }
    // r = g B: the adjoint recurrence, reversed in time; its last state is g_0
    if (rows_in_scan) {
        ssd::ScanShape f = sR;
        f.mode = 1;
        f.dt_len = s.L;
        BWD_LAUNCH(ssd::launch_adjoint_rows_scan(f, dy, dt, A, Cm, Bm, D, x, dfinal_states, reset, dx, atf(w.gfin), atf(w.e1), st),
                   "adjoint scan with row products");
    } else if (int rc = fast_r ? scan(sR, true, dy, Cm, Bm, dfinal_states, 1, at(w.r_rev), atf(w.gfin), states, false, 0)
                        : scan(sR, false, at(w.dy_rev), at(w.c_rev_g), at(w.b_rev_g), dfinal_states, 1, at(w.r_rev),
                               atf(w.gfin), states, false, 0))
        return rc;
    if (sum_on_chip) {
        // dB = sum over heads of dt (x . g): the adjoint recurrence with the state transposed; dC = sum over heads
        // of dy . h: the forward recurrence with the state transposed.  The one that runs first leaves its tile
        // states (in `states`), the other meets them on the way and leaves the pieces of the anchors.
        ssd::ScanShape fa = sTR, ff = sT;
        fa.mode = 1;
        fa.dt_len = s.L;
        fa.x_groups = ff.x_groups = s.G;
        ssd::ScanAnchors an, keep;
        an.other_tiles = states;
        an.out = reinterpret_cast<double *>(base + w.anchor);
        an.stride = keep.stride = plan.anchor_stride;
        if (ssd::transposed_scan_anchors_in_adjoint(sT)) {
            BWD_LAUNCH(ssd::launch_transposed_scan(ff, false, Bm, dt, A, x, dy, Cm, init_t, reset, dC, atf(w.ffin_t), states,
                                                   atf(w.parts), keep, st),
                       "transposed forward scan");
            an.other_final = atf(w.ffin_t);
            an.other_init = init_t;
            BWD_LAUNCH(ssd::launch_transposed_scan(fa, true, Cm, dt, A, dy, x, nullptr, dfin_t, reset, dB, nullptr, nullptr,
                                                   nullptr, an, st),
                       "transposed adjoint scan");
        } else {
            // (the adjoint scan's tile c starts where forward tile nc - c ends)
            an.phase = keep.phase = s.nc % plan.anchor_stride;
            BWD_LAUNCH(ssd::launch_transposed_scan(fa, true, Cm, dt, A, dy, x, nullptr, dfin_t, reset, dB, atf(w.gfin_t),
                                                   states, nullptr, keep, st),
                       "transposed adjoint scan");
            an.other_final = atf(w.gfin_t);
            an.other_init = dfin_t;
            BWD_LAUNCH(ssd::launch_transposed_scan(ff, false, Bm, dt, A, x, dy, Cm, init_t, reset, dC, nullptr, nullptr,
                                                   atf(w.parts), an, st),
                       "transposed forward scan");
        }
        if (!rows_in_scan)
            BWD_LAUNCH(ssd::launch_bwd_rows_parts(s, fast_r ? 0 : Lp, el, x, dy, dt, D, atf(w.r_rev), atf(w.parts), s.N / 32, dx,
                                                  atf(w.e1), atf(w.dd), atf(w.u), st),
                       "backward rows");
    } else {
    // yB = x . g: the same recurrence with the state transposed; its chunk states stay in `states`
    const int xg = (fast_t && rep > 1) ? s.G : 0;
    if (int rc = fast_t ? scan(sTR, true, Cm, dy, x, dfin_t, 1, at(w.yb_rev), atf(w.gfin_t), states, true, xg)
                        : scan(sTR, false, c_heads, at(w.dy_rev), at(w.x_rev), dfin_t, 1, at(w.yb_rev), atf(w.gfin_t),
                               states, true, 0))
        return rc;
    // yC = dy . h: the forward recurrence with the state transposed; its chunk states go to `states2`
    if (int rc = scan(sT, fast_t, b_heads, x, dy, init_t, 0, at(w.yc), atf(w.ffin_t), states2, true, xg)) return rc;
    if (ssd::bwd_rows_can_sum(s)) {  // dB and dC in the same pass
        BWD_LAUNCH(ssd::launch_bwd_rows(s, fast_r ? 0 : Lp, el, x, dy, dt, Cm, D, atf(w.r_rev), atf(w.yc), dx, atf(w.e1),
                                        atf(w.dd), atf(w.u), st, atf(w.yb_rev), fast_t ? 0 : Lp, dB, dC),
                   "backward rows");
    } else {
        BWD_LAUNCH(ssd::launch_bwd_rows(s, fast_r ? 0 : Lp, el, x, dy, dt, Cm, D, atf(w.r_rev), atf(w.yc), dx, atf(w.e1),
                                        atf(w.dd), atf(w.u), st),
                   "backward rows");
        BWD_LAUNCH(ssd::launch_bwd_group_sums(s, fast_t ? 0 : Lp, el, dt, atf(w.yb_rev), atf(w.yc), dB, dC, st),
                   "backward group sums");
    }
    }
    double *anchor = reinterpret_cast<double *>(base + w.anchor);
    if (!sum_on_chip)
        BWD_LAUNCH(ssd::launch_bwd_anchors(s, el, dt, A, states2, states, atf(w.gfin_t), init_t, atf(w.ffin_t), dfin_t, reset,
                                           anchor, st),
                   "backward anchors");
    double *da_part = reinterpret_cast<double *>(base + w.da_part);
    double *dd_part = da_part + (size_t)s.B * s.nc * s.H;
    BWD_LAUNCH(ssd::launch_bwd_ddt(s, el, dt, A, atf(w.e1), atf(w.u), atf(w.dd), anchor, ddt, da_part, dd_part, st,
                                   rows_in_scan ? atf(w.parts) : nullptr, s.N / 32, reset, sum_on_chip ? s.N / 32 : 0,
                                   plan.anchor_stride),
               "backward ddt");
    BWD_LAUNCH(ssd::launch_bwd_head_sums(s, da_part, dd_part, dA, dD, st), "backward head sums");
    if (dinitial_states != nullptr)
        BWD_LAUNCH(ssd::launch_bwd_dinit(s, el, dt, A, atf(w.gfin), reset, dinitial_states, st), "backward dinit");
#undef BWD_LAUNCH
    return SSD_OK;
}

int ssd_chunk_scan_is_onepass(const ssd_dims *dims, int dtype, int *is_onepass) {
    if (is_onepass == nullptr) return fail(SSD_ERR_INVALID, "ssd: is_onepass must not be NULL");
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    *is_onepass = (takes_one_pass(s, dtype) && ssd::fused_scan_tail_rows(s, dtype) == 0) ? 1 : 0;
    return SSD_OK;
}

int ssd_chunk_scan_segments(const ssd_dims *dims, int dtype, int *segments) {
    if (segments == nullptr) return fail(SSD_ERR_INVALID, "ssd: segments must not be NULL");
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    ssd::fused_scan_plan(s, dtype, segments);
    return SSD_OK;
}

int ssd_chunk_scan_onepass_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                               const void *Bm, const void *Cm, const float *D, const float *initial_states,
                               const uint8_t *reset, void *y, float *final_states, void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(x);
    REQUIRE_PTR(dt);
    REQUIRE_PTR(A);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(Cm);
    REQUIRE_PTR(y);
    OPTIONAL_PTR(D);
    OPTIONAL_PTR(initial_states);
    OPTIONAL_PTR(final_states);
    if (dtype == SSD_DTYPE_F32 ? ssd::fused_scan_f32_waves(s) == 0 : ssd::fused_scan_waves(s, dtype) == 0)
        return fail(SSD_ERR_UNSUPPORTED,
                    "ssd: the one-pass scan needs headdim a multiple of 32, dstate 32, 64 or 128 and "
                    "(nheads/ngroups)*(headdim/32) a multiple of 4 (float32 inputs: dstate 32 or 64, a multiple of 8)");
    hipError_t e = ssd::launch_fused_scan(s, dtype, x, dt, A, Bm, Cm, D, initial_states, reset, y, final_states,
                                          (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "one-pass scan launch");
}

int ssd_step_fwd(const ssd_step_dims *dims, int dtype, float *state, const void *x, const void *dt,
                 const float *A, const void *Bm, const void *Cm, const float *D, void *y, void *hip_stream) {
    if (dims == nullptr) return fail(SSD_ERR_INVALID, "ssd: dims must not be NULL");
    if (int rc = check_dtype(dtype)) return rc;
    if (dims->batch <= 0) return fail(SSD_ERR_INVALID, "ssd: batch must be positive, got %lld", (long long)dims->batch);
    if (int rc = check_state_dims(dims->nheads, dims->headdim, dims->dstate, dims->ngroups)) return rc;
    if (dims->batch * dims->nheads > 0x7fffffff)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: batch*nheads exceeds 2^31-1");
    REQUIRE_PTR(state);
    REQUIRE_PTR(x);
    REQUIRE_PTR(dt);
    REQUIRE_PTR(A);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(Cm);
    REQUIRE_PTR(y);
    OPTIONAL_PTR(D);
    ssd::StepShape s{(int)dims->batch, (int)dims->nheads, (int)dims->headdim, (int)dims->dstate,
                     (int)dims->ngroups};
    hipError_t e = ssd::launch_step(s, dtype, state, x, dt, A, Bm, Cm, D, y, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "step launch");
}

int ssd_steps_fwd(const ssd_step_dims *dims, int64_t nsteps, int dtype, float *state, const uint8_t *reset,
                  const void *x, const void *dt, const float *A, const void *Bm, const void *Cm, const float *D,
                  void *y, void *hip_stream) {
    if (dims == nullptr) return fail(SSD_ERR_INVALID, "ssd: dims must not be NULL");
    if (int rc = check_dtype(dtype)) return rc;
    if (dims->batch <= 0) return fail(SSD_ERR_INVALID, "ssd: batch must be positive, got %lld", (long long)dims->batch);
    if (nsteps <= 0 || nsteps > 0x7fffffff)
        return fail(SSD_ERR_INVALID, "ssd: nsteps must be positive, got %lld", (long long)nsteps);
    if (int rc = check_state_dims(dims->nheads, dims->headdim, dims->dstate, dims->ngroups)) return rc;
    if (dims->batch * dims->nheads > 0x7fffffff)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: batch*nheads exceeds 2^31-1");
    REQUIRE_PTR(state);
    REQUIRE_PTR(x);
    REQUIRE_PTR(dt);
    REQUIRE_PTR(A);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(Cm);
    REQUIRE_PTR(y);
    OPTIONAL_PTR(D);
    ssd::StepShape s{(int)dims->batch, (int)dims->nheads, (int)dims->headdim, (int)dims->dstate,
                     (int)dims->ngroups};
    // A long run of steps is a scan with an initial state, and the one-pass scan does it on the matrix cores: from
    // about ten steps on it is faster than the step-by-step kernel at every batch size (64 steps at batch 4096:
    // 0.25 ms against 0.99 ms).  Each of its waves reads its slice of the initial state before the first tile and
    // writes the final state after the last, so the two may be the same memory.
    constexpr int64_t kStepsAsScanMin = 16;
    if (nsteps >= kStepsAsScanMin && dtype != SSD_DTYPE_F32) {
        const ssd_dims d = {dims->batch, nsteps, dims->nheads, dims->headdim, dims->dstate, dims->ngroups, kBackwardChunk};
        ssd::ScanShape sc;
        // (asked for the bf16-y instance whatever y's type is: the two output types must take the same path, so
        // that the bf16 y stays the float32 y rounded once; one instance exists for float y only)
        if (make_shape(&d, dtype, &sc) == SSD_OK && ssd::fused_scan_waves(sc, SSD_DTYPE_BF16) != 0) {
            hipError_t e = ssd::launch_fused_scan(sc, dtype, x, dt, A, Bm, Cm, D, state, reset, y, state,
                                                  (hipStream_t)hip_stream);
            return e == hipSuccess ? SSD_OK : hip_fail(e, "one-pass scan launch (steps)");
        }
        std::free(ssd_get_and_reset_last_err());  // whatever make_shape had to say: the step kernel decides
    }
    if (!ssd::steps_supported(s))
        return fail(SSD_ERR_UNSUPPORTED, "ssd: the multi-step update keeps the state in registers and needs headdim "
                                         "16, 32 or 64, got %lld", (long long)dims->headdim);
    hipError_t e = ssd::launch_steps(s, (int)nsteps, dtype, state, reset, x, dt, A, Bm, Cm, D, y,
                                     (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "multi-step launch");
}

static int make_block_shape(const ssd_block_dims *d, int dtype, ssd::BlockShape *out) {
    if (d == nullptr) return fail(SSD_ERR_INVALID, "ssd: dims must not be NULL");
    if (int rc = check_dtype(dtype)) return rc;
    if (d->batch <= 0 || d->seqlen <= 0)
        return fail(SSD_ERR_INVALID, "ssd: batch and seqlen must be positive, got %lld %lld", (long long)d->batch,
                    (long long)d->seqlen);
    if (int rc = check_state_dims(d->nheads, d->headdim, d->dstate, d->ngroups)) return rc;
    const int64_t E = 2 * d->nheads * d->headdim + 2 * d->ngroups * d->dstate + d->nheads;
    if (d->batch * d->seqlen > 0x7fffffff || d->zxbcdt_ld > 0x7fffffff ||
        d->batch * d->seqlen * (d->zxbcdt_ld > E ? d->zxbcdt_ld : E) / 8 > 0x7fffffffffLL)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: batch*seqlen exceeds 2^31-1");
    if (E % (dtype == SSD_DTYPE_F32 ? 4 : 8) != 0)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: the %lld channels of a timestep must be a whole number of 16-byte "
                                         "pieces (nheads a multiple of %d)", (long long)E, dtype == SSD_DTYPE_F32 ? 4 : 8);
    const int64_t ld = d->zxbcdt_ld == 0 ? E : d->zxbcdt_ld;
    if (ld < E || ld > 0x7fffffff || ld % (dtype == SSD_DTYPE_F32 ? 4 : 8) != 0)
        return fail(SSD_ERR_INVALID, "ssd: zxbcdt_ld must be 0 or at least the %lld channels of a timestep and a whole "
                                     "number of 16-byte pieces, got %lld", (long long)E, (long long)d->zxbcdt_ld);
    ssd::BlockShape s{(int)d->batch, (int)d->seqlen, (int)d->nheads, (int)d->headdim, (int)d->dstate,
                      (int)d->ngroups, (int)d->d_conv, (int)ld};
    if (!ssd::block_supported(s))
        return fail(SSD_ERR_UNSUPPORTED, "ssd: block stages need d_conv 2..4 (got %lld) and nheads*headdim <= 2048",
                    (long long)d->d_conv);
    *out = s;
    return SSD_OK;
}

int ssd_block_pre_fwd(const ssd_block_dims *dims, int dtype, const void *zxbcdt, const float *conv_w,
                      const float *conv_b, const float *dt_bias, const void *conv_state_in, void *conv_state_out,
                      void *x, void *Bm, void *Cm, void *dt, void *hip_stream) {
    return ssd_block_pre_reset_fwd(dims, dtype, zxbcdt, conv_w, conv_b, dt_bias, conv_state_in, conv_state_out, nullptr, x,
                                   Bm, Cm, dt, hip_stream);
}

int ssd_block_pre_reset_fwd(const ssd_block_dims *dims, int dtype, const void *zxbcdt, const float *conv_w,
                            const float *conv_b, const float *dt_bias, const void *conv_state_in, void *conv_state_out,
                            const uint8_t *reset, void *x, void *Bm, void *Cm, void *dt, void *hip_stream) {
    ssd::BlockShape s;
    if (int rc = make_block_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(zxbcdt);
    REQUIRE_PTR(conv_w);
    REQUIRE_PTR(conv_b);
    REQUIRE_PTR(dt_bias);
    REQUIRE_PTR(x);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(Cm);
    REQUIRE_PTR(dt);
    OPTIONAL_PTR(conv_state_in);
    OPTIONAL_PTR(conv_state_out);
    if (conv_state_in != nullptr && conv_state_in == conv_state_out && s.L > 1)
        return fail(SSD_ERR_INVALID, "ssd: conv_state_in and conv_state_out may alias only for seqlen 1");
    hipError_t e = ssd::launch_block_pre(s, dtype == SSD_DTYPE_F32 ? 0 : 1, zxbcdt, conv_w, conv_b, dt_bias,
                                         conv_state_in, conv_state_out, reset, x, Bm, Cm, dt, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "block pre-scan launch");
}

int ssd_block_proj_fwd(int64_t rows, int64_t in_features, int64_t out_features, int64_t out_ld, int dtype, const void *u,
                       const void *w, void *out, void *hip_stream) {
    if (dtype != SSD_DTYPE_BF16)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: the block projection takes dtype 1 (bfloat16), got %d", dtype);
    if (rows <= 0 || in_features <= 0 || out_features <= 0)
        return fail(SSD_ERR_INVALID, "ssd: projection sizes must be positive, got %lld x %lld -> %lld", (long long)rows,
                    (long long)in_features, (long long)out_features);
    if (in_features > 0x7fffffff || out_features > 0x7fffffff ||
        !ssd::block_proj_supported(rows, (int)in_features, (int)out_features))
        return fail(SSD_ERR_UNSUPPORTED,
                    "ssd: the block projection needs in_features 128 or 256 and out_features a multiple of 8, got "
                    "%lld and %lld",
                    (long long)in_features, (long long)out_features);
    if (out_ld == 0) out_ld = out_features;
    if (out_ld < out_features || out_ld > 0x7fffffff || out_ld % 8 != 0)
        return fail(SSD_ERR_INVALID, "ssd: out_ld must be 0 or at least out_features (%lld) and a multiple of 8, got %lld",
                    (long long)out_features, (long long)out_ld);
    REQUIRE_PTR(u);
    REQUIRE_PTR(w);
    REQUIRE_PTR(out);
    hipError_t e = ssd::launch_block_proj(rows, (int)in_features, (int)out_features, (int)out_ld, u, w, out,
                                          (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "block projection launch");
}

int ssd_block_bwd_workspace_bytes(const ssd_block_dims *dims, int dtype, size_t *out_bytes) {
    if (out_bytes == nullptr) return fail(SSD_ERR_INVALID, "ssd: out_bytes must not be NULL");
    ssd::BlockShape s;
    if (int rc = make_block_shape(dims, dtype, &s)) return rc;
    *out_bytes = align_up(ssd::block_bwd_workspace_bytes(s), 256);
    return SSD_OK;
}

int ssd_block_post_bwd(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                       float eps, const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, void *workspace,
                       size_t workspace_bytes, void *hip_stream) {
    return ssd_block_post_bwd_yn(dims, dtype, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, nullptr, workspace,
                                 workspace_bytes, hip_stream);
}

int ssd_block_post_bwd_yn(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                          float eps, const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, void *yn_out,
                          void *workspace, size_t workspace_bytes, void *hip_stream) {
    ssd::BlockShape s;
    if (int rc = make_block_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(y);
    REQUIRE_PTR(zxbcdt);
    REQUIRE_PTR(norm_w);
    REQUIRE_PTR(dout);
    REQUIRE_PTR(dy);
    REQUIRE_PTR(dzxbcdt);
    REQUIRE_PTR(dnorm_w);
    REQUIRE_PTR(workspace);
    if (!(eps > 0.f)) return fail(SSD_ERR_INVALID, "ssd: eps must be positive");
    const size_t need = ssd::block_bwd_workspace_bytes(s);
    if (workspace_bytes < need)
        return fail(SSD_ERR_WORKSPACE, "ssd: block backward workspace has %zu bytes, %zu needed", workspace_bytes, need);
    OPTIONAL_PTR(yn_out);
    hipError_t e = ssd::launch_block_post_bwd(s, dtype, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, workspace,
                                              (hipStream_t)hip_stream, yn_out);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "block post-scan backward launch");
}

int ssd_block_pre_bwd(const ssd_block_dims *dims, int dtype, const void *zxbcdt, const float *conv_w, const float *conv_b,
                      const float *dt_bias, const void *conv_state_in, const uint8_t *reset, const void *dx, const void *dB,
                      const void *dC, const void *ddt, const void *dconv_state_out, void *dzxbcdt, float *dconv_w,
                      float *dconv_b, float *ddt_bias, void *dconv_state_in, void *workspace, size_t workspace_bytes,
                      void *hip_stream) {
    ssd::BlockShape s;
    if (int rc = make_block_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(zxbcdt);
    REQUIRE_PTR(conv_w);
    REQUIRE_PTR(conv_b);
    REQUIRE_PTR(dt_bias);
    REQUIRE_PTR(dx);
    REQUIRE_PTR(dB);
    REQUIRE_PTR(dC);
    REQUIRE_PTR(ddt);
    REQUIRE_PTR(dzxbcdt);
    REQUIRE_PTR(dconv_w);
    REQUIRE_PTR(dconv_b);
    REQUIRE_PTR(ddt_bias);
    REQUIRE_PTR(workspace);
    OPTIONAL_PTR(conv_state_in);
    OPTIONAL_PTR(dconv_state_out);
    OPTIONAL_PTR(dconv_state_in);
    const size_t need = ssd::block_bwd_workspace_bytes(s);
    if (workspace_bytes < need)
        return fail(SSD_ERR_WORKSPACE, "ssd: block backward workspace has %zu bytes, %zu needed", workspace_bytes, need);
    hipError_t e = ssd::launch_block_pre_bwd(s, dtype == SSD_DTYPE_F32 ? 0 : 1, zxbcdt, conv_w, conv_b, dt_bias, conv_state_in,
                                             reset, dx, dB, dC, ddt, dconv_state_out, dzxbcdt, dconv_w, dconv_b, ddt_bias,
                                             dconv_state_in, workspace, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "block pre-scan backward launch");
}

int ssd_block_post_fwd(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt,
                       const float *norm_w, float eps, void *out, void *hip_stream) {
    ssd::BlockShape s;
    if (int rc = make_block_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(y);
    REQUIRE_PTR(zxbcdt);
    REQUIRE_PTR(norm_w);
    REQUIRE_PTR(out);
    if (!(eps > 0.f)) return fail(SSD_ERR_INVALID, "ssd: eps must be positive");
    hipError_t e = ssd::launch_block_post(s, dtype, y, zxbcdt, norm_w, eps, out, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "block post-scan launch");
}

int ssd_block_post_proj_fwd(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                            float eps, const void *w, int64_t out_features, int64_t out_ld, void *out, void *hip_stream) {
    ssd::BlockShape s;
    if (int rc = make_block_shape(dims, dtype, &s)) return rc;
    if (dtype != SSD_DTYPE_BF16)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: the fused post-scan + out-projection takes dtype 1 (bfloat16), got %d", dtype);
    if (out_features <= 0 || out_features > 0x7fffffff)
        return fail(SSD_ERR_INVALID, "ssd: out_features must be positive, got %lld", (long long)out_features);
    if (!ssd::block_post_proj_supported(s, (int)out_features))
        return fail(SSD_ERR_UNSUPPORTED,
                    "ssd: the fused post-scan + out-projection needs nheads*headdim 128 or 256 and out_features a multiple "
                    "of 8 up to 256, got %d and %lld", s.H * s.P, (long long)out_features);
    if (out_ld == 0) out_ld = out_features;
    if (out_ld < out_features || out_ld > 0x7ffff || out_ld % 8 != 0)
        return fail(SSD_ERR_INVALID, "ssd: out_ld must be 0 or at least out_features (%lld), a multiple of 8 and below 524288, got %lld",
                    (long long)out_features, (long long)out_ld);
    REQUIRE_PTR(y);
    REQUIRE_PTR(zxbcdt);
    REQUIRE_PTR(norm_w);
    REQUIRE_PTR(w);
    REQUIRE_PTR(out);
    if (!(eps > 0.f)) return fail(SSD_ERR_INVALID, "ssd: eps must be positive");
    hipError_t e = ssd::launch_block_post_proj(s, y, zxbcdt, norm_w, eps, w, (int)out_features, (int)out_ld, out,
                                               (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "block post-scan + out-projection launch");
}

int ssd_block_step_fwd(const ssd_block_dims *dims, int dtype, int64_t d_model, const void *u, const void *w_in,
                       const float *conv_w, const float *conv_b, const float *dt_bias, const float *A, const float *D,
                       const float *norm_w, float eps, const void *w_out, void *conv_state, float *ssm_state, void *out,
                       void *hip_stream) {
    ssd::BlockShape s;
    if (int rc = make_block_shape(dims, dtype, &s)) return rc;
    if (dtype != SSD_DTYPE_F32 && dtype != SSD_DTYPE_BF16)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: the fused block step takes dtype 0 (float32) or 1 (bfloat16), got %d", dtype);
    if (s.L != 1) return fail(SSD_ERR_INVALID, "ssd: the fused block step advances one timestep, got seqlen %d", s.L);
    if (d_model <= 0 || d_model > 0x7fffffff || !ssd::block_step_supported(s, (int)d_model))
        return fail(SSD_ERR_UNSUPPORTED,
                    "ssd: the fused block step needs d_model and nheads*headdim of 128 or 256 and dstate a multiple of 16, "
                    "got d_model %lld, nheads*headdim %d, dstate %d", (long long)d_model, s.H * s.P, s.N);
    REQUIRE_PTR(u);
    REQUIRE_PTR(w_in);
    REQUIRE_PTR(conv_w);
    REQUIRE_PTR(conv_b);
    REQUIRE_PTR(dt_bias);
    REQUIRE_PTR(A);
    REQUIRE_PTR(norm_w);
    REQUIRE_PTR(w_out);
    REQUIRE_PTR(conv_state);
    REQUIRE_PTR(ssm_state);
    REQUIRE_PTR(out);
    OPTIONAL_PTR(D);
    if (!(eps > 0.f)) return fail(SSD_ERR_INVALID, "ssd: eps must be positive");
    hipError_t e = ssd::launch_block_step(s, dtype == SSD_DTYPE_F32 ? 0 : 1, (int)d_model, u, w_in, conv_w, conv_b, dt_bias,
                                          A, D, norm_w, eps, w_out, conv_state, ssm_state, out, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "fused block step launch");
}

}  // extern "C"
