// C ABI of libssd_hip: argument validation, error slot, workspace carving, stage sequencing.
// Conventions follow the reference's own extern "C" shim (thread-local malloc'd error string,
// vendor/torch-sys-0.25.0/libtch/torch_api.h:18-24,33 and torch_api.cpp:32,84-88) and its op
// wrappers' validate-then-call shape (trading_bots/src/torch/fa4.rs:145-191).
#include "../../include/ssd_hip.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "ssd_launch.h"

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
    return ssd::fused_scan_waves(s, dtype) == 8 && (int64_t)s.B * s.H * (s.P / 32) / 8 >= kOnePassMinWorkgroups;
}

int hip_fail(hipError_t e, const char *what) {
    return fail(SSD_ERR_RUNTIME, "ssd: %s failed: %s", what, hipGetErrorString(e));
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

int ssd_chunk_scan_reset_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                             const void *Bm, const void *Cm, const float *D, const float *initial_states,
                             const uint8_t *reset, void *y, float *final_states, void *workspace,
                             size_t workspace_bytes, void *hip_stream) {
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    REQUIRE_PTR(x);
    REQUIRE_PTR(dt);
    REQUIRE_PTR(A);
    REQUIRE_PTR(Bm);
    REQUIRE_PTR(Cm);
    REQUIRE_PTR(y);
    REQUIRE_PTR(workspace);
    OPTIONAL_PTR(D);
    OPTIONAL_PTR(initial_states);
    OPTIONAL_PTR(final_states);
    const Workspace w = carve(s);
    if (workspace_bytes < w.total)
        return fail(SSD_ERR_WORKSPACE, "ssd: workspace has %zu bytes, %zu needed", workspace_bytes, w.total);
    char *base = static_cast<char *>(workspace);
    float *dtcs = reinterpret_cast<float *>(base + w.dtcs_off);
    float *states = reinterpret_cast<float *>(base + w.st_off);
    hipStream_t st = (hipStream_t)hip_stream;
    hipError_t e;
    if (takes_one_pass(s, dtype)) {
        e = ssd::launch_fused_scan(s, dtype, x, dt, A, Bm, Cm, D, initial_states, reset, y, final_states, st);
        return e == hipSuccess ? SSD_OK : hip_fail(e, "one-pass scan launch");
    }
    e = ssd::launch_chunk_cumsum(s, dtype, dt, A, reset, dtcs, st);
    if (e != hipSuccess) return hip_fail(e, "chunk_cumsum launch");
    if ((int64_t)s.B * s.H >= kFusedStatePassingMinSequences) {
        // enough (b,h) sequences to fill the chip: stages 2 and 3 in one pass, states carried on chip
        e = ssd::launch_chunk_state_scan(s, dtype, x, Bm, dtcs, initial_states, states, final_states, st);
        if (e != hipSuccess) return hip_fail(e, "chunk_state_passing launch");
    } else {
        e = ssd::launch_chunk_state(s, dtype, x, Bm, dtcs, states, st);
        if (e != hipSuccess) return hip_fail(e, "chunk_state launch");
        e = ssd::launch_state_passing(s, states, dtcs, initial_states, states, final_states, st);  // in place
        if (e != hipSuccess) return hip_fail(e, "state_passing launch");
    }
    e = ssd::launch_chunk_scan(s, dtype, x, Bm, Cm, dtcs, states, D, y, st);
    if (e != hipSuccess) return hip_fail(e, "chunk_scan launch");
    return SSD_OK;
}

int ssd_chunk_scan_is_onepass(const ssd_dims *dims, int dtype, int *is_onepass) {
    if (is_onepass == nullptr) return fail(SSD_ERR_INVALID, "ssd: is_onepass must not be NULL");
    ssd::ScanShape s;
    if (int rc = make_shape(dims, dtype, &s)) return rc;
    *is_onepass = takes_one_pass(s, dtype) ? 1 : 0;
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
    if (ssd::fused_scan_waves(s, dtype) == 0)
        return fail(SSD_ERR_UNSUPPORTED,
                    "ssd: the one-pass scan needs bf16 inputs, headdim a multiple of 32, dstate 32 or 64 and "
                    "(nheads/ngroups)*(headdim/32) a multiple of 4");
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
    if (d->batch * d->seqlen > 0x7fffffff || d->batch * d->seqlen * E / 8 > 0x7fffffffffLL)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: batch*seqlen exceeds 2^31-1");
    if (E % (dtype == SSD_DTYPE_F32 ? 4 : 8) != 0)
        return fail(SSD_ERR_UNSUPPORTED, "ssd: the %lld channels of a timestep must be a whole number of 16-byte "
                                         "pieces (nheads a multiple of %d)", (long long)E, dtype == SSD_DTYPE_F32 ? 4 : 8);
    ssd::BlockShape s{(int)d->batch, (int)d->seqlen, (int)d->nheads, (int)d->headdim, (int)d->dstate,
                      (int)d->ngroups, (int)d->d_conv};
    if (!ssd::block_supported(s))
        return fail(SSD_ERR_UNSUPPORTED, "ssd: block stages need d_conv 2..4 (got %lld) and nheads*headdim <= 2048",
                    (long long)d->d_conv);
    *out = s;
    return SSD_OK;
}

int ssd_block_pre_fwd(const ssd_block_dims *dims, int dtype, const void *zxbcdt, const float *conv_w,
                      const float *conv_b, const float *dt_bias, const void *conv_state_in, void *conv_state_out,
                      void *x, void *Bm, void *Cm, void *dt, void *hip_stream) {
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
                                         conv_state_in, conv_state_out, x, Bm, Cm, dt, (hipStream_t)hip_stream);
    return e == hipSuccess ? SSD_OK : hip_fail(e, "block pre-scan launch");
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

}  // extern "C"
