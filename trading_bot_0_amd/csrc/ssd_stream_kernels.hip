// Mamba-2 SSD forward for gfx950 (MI355X, CDNA4): the three streaming kernels.
// Stage 1 (chunk_cumsum) is a DPP wavefront scan; stage 3 (state_passing) and stage 5 (the
// single-timestep update) are pure HBM streams.  Stages 2 and 4 (MFMA tiles) live in
// ssd_chunk_state.hip and ssd_chunk_scan.hip.
#include "ssd_device.h"

namespace ssd {

// ------------------------------------------------------------------------------------------
// Stage 1: chunk_cumsum.  One workgroup per (b,c): the [Q,H] tile of dt is read coalesced,
// transposed through LDS, and every head row gets a wavefront inclusive scan of dt*A.
//
// Output "dtcs" [B,H,nc,4,Q] float32: rows 0/1 = alpha (the cumulative sum times log2 e) as
// an unevaluated pair hi + lo, row 2 = dt, row 3 = the stage-2 weight
// exp2(alpha[Q-1] - alpha[l]) * dt[l] (decay from step l to the end of the chunk).  The scan runs in float64 and is split into two
// floats because the later stages only ever use DIFFERENCES alpha[l] - alpha[s]: with one
// float, a large |alpha| (hundreds after a strongly decaying step) leaves an absolute error
// of ulp(|alpha|) in a difference that may itself be small, i.e. a relative error of
// 1e-5..1e-3 in the decay factor.  (hi_l - hi_s) + (lo_l - lo_s) keeps the difference good to
// its own ulp.
// ------------------------------------------------------------------------------------------
template <typename T, int EPL>  // EPL = elements per lane = max(Q/64, 1)
__global__ __launch_bounds__(256) void chunk_cumsum_kernel(const T *__restrict__ dt,
                                                           const float *__restrict__ A,
                                                           const unsigned char *__restrict__ reset,
                                                           float *__restrict__ dtcs, ScanShape s, int mode,
                                                           int dt_len) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *tile = reinterpret_cast<float *>(smem);  // [H][Q+1]
    const int ldt = s.Q + 1;
    float *drop = tile + s.H * ldt;                 // [Q]: kResetDrop where the state restarts, else 0
    const int b = blockIdx.x / s.nc, c = blockIdx.x % s.nc;
    const int t0 = c * s.Q;
    for (int idx = threadIdx.x; idx < s.Q * s.H; idx += blockDim.x) {
        const int l = idx / s.H, h = idx % s.H;
        const int t = t0 + l;
        // mode 1 (the time-reversed adjoint recurrence): step t decays by the dt of step L - t of a dt tensor
        // of dt_len <= L rows; steps that fall outside it (step 0, and the L - dt_len leading steps that pad
        // the reversed sequence to whole chunks) do not decay
        float v;
        if (mode == 0) v = (t < s.L) ? (float)dt[((size_t)b * s.L + t) * s.H + h] : 0.f;
        else v = (t < s.L && s.L - t >= 1 && s.L - t < dt_len) ? (float)dt[((size_t)b * dt_len + (s.L - t)) * s.H + h] : 0.f;
        tile[h * ldt + l] = v;
    }
    for (int l = threadIdx.x; l < s.Q; l += blockDim.x)
    {
        // in mode 1 the restart before step L - t of the forward sequence cuts the adjoint at reversed step t
        const int t = t0 + l, src = mode == 0 ? t : s.L - t;
        const bool in = mode == 0 ? t < s.L : (t < s.L && src >= 1 && src < dt_len);
        drop[l] = (reset != nullptr && in && reset[(size_t)b * (mode == 0 ? s.L : dt_len) + src] != 0) ? (float)kResetDrop : 0.f;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    constexpr double kLog2e = 1.4426950408889634;
    for (int h = wave; h < s.H; h += nwaves) {
        const double a = (double)A[h];
        float dtv[EPL];
        double cs[EPL];
        double run = 0.0;
        const int l0 = lane * EPL;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            dtv[e] = (l0 + e < s.Q) ? tile[h * ldt + l0 + e] : 0.f;
            run += (double)dtv[e] * a - (double)((l0 + e < s.Q) ? drop[l0 + e] : 0.f);
            cs[e] = run;
        }
        const double incl = wave_inclusive_scan(run);
        const double excl = incl - run;
        // chunk total = the last lane's inclusive sum (lanes past Q carry zeros)
        const double total = __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(incl), 63),
                                              __builtin_amdgcn_readlane(__double2loint(incl), 63));
        if (l0 < s.Q) {
            float *row = dtcs + ((((size_t)b * s.H + h) * s.nc + c) * 4) * s.Q + l0;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const double cum = cs[e] + excl;
                const double al = cum * kLog2e;
                const float hi = (float)al;
                row[e] = hi;
                row[s.Q + e] = (float)(al - (double)hi);
                // the input weight: dt, or in mode 1 one for every step of the sequence (padding steps stay no-ops)
                const float wv = mode == 0 ? dtv[e] : ((t0 + l0 + e < s.L) ? 1.f : 0.f);
                row[2 * s.Q + e] = wv;
                row[3 * s.Q + e] = exp2_hw(fminf((float)((total - cum) * kLog2e), 0.f)) * wv;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Stage 3: state_passing.  One lane per float4 of the [P,N] state of one (b,h); the chunk
// loop is the only sequential axis.  All chunk loads of a batch of chunks are issued before
// the dependent multiply-adds so the recurrence does not serialise memory latency.
// prev may alias states: each lane reads its element of chunk c before overwriting it.
// ------------------------------------------------------------------------------------------
constexpr int kPassUnroll = 8;

__global__ __launch_bounds__(256) void state_passing_kernel(const float *states, const float *__restrict__ dtcs,
                                                            const float *init, float *prev,
                                                            float *final_states, ScanShape s,
                                                            long long total) {
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const int pn4 = s.P * s.N / 4;
    const int bh = (int)(gid / pn4), idx = (int)(gid % pn4);
    const int b = bh / s.H, h = bh % s.H;
    const size_t chunk_stride = (size_t)s.H * pn4;  // in float4
    const float4 *src = reinterpret_cast<const float4 *>(states) + ((size_t)b * s.nc * s.H + h) * pn4 + idx;
    float4 *dst = reinterpret_cast<float4 *>(prev) + ((size_t)b * s.nc * s.H + h) * pn4 + idx;
    const float *a_end = dtcs + ((size_t)bh * s.nc) * 4 * s.Q + (s.Q - 1);  // alpha_hi at the chunk end
    const size_t a_stride = (size_t)4 * s.Q;
    const bool fresh = s.fresh != nullptr && s.fresh[(size_t)b * s.L] != 0;  // restarts before its first step
    float4 st = init && !fresh ? reinterpret_cast<const float4 *>(init)[(size_t)bh * pn4 + idx] : make_float4(0, 0, 0, 0);
    int c = 0;
    for (; c + kPassUnroll <= s.nc; c += kPassUnroll) {
        float4 sv[kPassUnroll];
        float dec[kPassUnroll];
#pragma unroll
        for (int i = 0; i < kPassUnroll; ++i) {
            sv[i] = src[(size_t)(c + i) * chunk_stride];
            dec[i] = exp2_hw(a_end[(size_t)(c + i) * a_stride]);
        }
#pragma unroll
        for (int i = 0; i < kPassUnroll; ++i) {
            dst[(size_t)(c + i) * chunk_stride] = st;
            st.x = dec[i] * st.x + sv[i].x;
            st.y = dec[i] * st.y + sv[i].y;
            st.z = dec[i] * st.z + sv[i].z;
            st.w = dec[i] * st.w + sv[i].w;
        }
    }
    for (; c < s.nc; ++c) {
        const float4 sv = src[(size_t)c * chunk_stride];
        const float dec = exp2_hw(a_end[(size_t)c * a_stride]);
        dst[(size_t)c * chunk_stride] = st;
        st.x = dec * st.x + sv.x;
        st.y = dec * st.y + sv.y;
        st.z = dec * st.z + sv.z;
        st.w = dec * st.w + sv.w;
    }
    if (final_states) reinterpret_cast<float4 *>(final_states)[(size_t)bh * pn4 + idx] = st;
}

// four consecutive elements as floats, one load
__device__ inline void load4(const float *p, float (&o)[4]) {
    const float4 v = *reinterpret_cast<const float4 *>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ inline void load4(const __bf16 *p, float (&o)[4]) {
    const uint2 v = *reinterpret_cast<const uint2 *>(p);
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
}

// ------------------------------------------------------------------------------------------
// Stage 5: single-timestep update, in place.  One wave per (b,h); NL = N/4 lanes cover one
// state row with a float4 each, 64/NL rows per pass.  The row dot-product with C is reduced
// across the NL lanes with xor-shuffles.  TO is the element type of y.
// ------------------------------------------------------------------------------------------
template <typename T, typename TO, int NL>
__global__ __launch_bounds__(256) void step_kernel(float *__restrict__ state, const T *__restrict__ x,
                                                   const T *__restrict__ dt, const float *__restrict__ A,
                                                   const T *__restrict__ Bm, const T *__restrict__ Cm,
                                                   const float *__restrict__ D, TO *__restrict__ y, StepShape s) {
    constexpr int N = NL * 4;
    constexpr int RPP = 64 / NL;  // rows per pass
    // passes whose loads are issued together: a whole [32, 64] state; never more than NL, so that lane u of a
    // row's group can keep pass u's result
    constexpr int UN = NL < 8 ? NL : 8;
    const int lane = threadIdx.x & 63;
    // the wave's (b, h), in scalar registers (the launcher keeps B * H below 2^31)
    const int bh = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)));
    if (bh >= s.B * s.H) return;
    const int b = bh / s.H, h = bh - b * s.H;
    const int g = h / (s.H / s.G);
    const int nl = lane % NL, rl = lane / NL;
    float4 *st = reinterpret_cast<float4 *>(state) + (size_t)bh * s.P * NL;
    const T *xr = x + (size_t)bh * s.P;
    TO *yr = y + (size_t)bh * s.P;
    // Every load of a block of rows is issued before the first result is needed, none of them under a condition (a
    // conditional load is a branch, and the compiler waits for all earlier loads at every one): rows past the state
    // are read as its last row and never stored.  The block's rows of x are one load: lane (rl, nl < UN) takes row
    // p0 + nl * RPP + rl (the lane that stores that row's y), and every pass fetches its row's value from that lane.
    float4 hv[UN];
    float xq;
    auto load_block = [&](int p0) {
        const bool whole = p0 + RPP * UN <= s.P;  // uniform
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int p = p0 + u * RPP + rl;
            hv[u] = st[(size_t)(whole ? p : min(p, s.P - 1)) * NL + nl];
        }
        xq = (float)xr[min(p0 + nl * RPP + rl, s.P - 1)];
    };
    // the step's scalars and this lane's four columns of B and C are requested first and used after the first block
    // of the state has been requested, so that the state's loads do not wait for them
    const T dt_raw = dt[bh];
    const float a_h = A[h];
    const float dh = D ? D[h] : 0.f;
    float bv[4], cv[4];
    load4(Bm + ((size_t)b * s.G + g) * N + nl * 4, bv);
    load4(Cm + ((size_t)b * s.G + g) * N + nl * 4, cv);
    load_block(0);
    const float dtv = (float)dt_raw;
    const float decay = expf(dtv * a_h);
#pragma unroll
    for (int i = 0; i < 4; ++i) bv[i] *= dtv;
    for (int p0 = 0; p0 < s.P; p0 += RPP * UN) {
        if (p0 != 0) load_block(p0);
        const bool whole = p0 + RPP * UN <= s.P;
        float xv[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) xv[u] = group_lane<NL>(xq, u);
        float keep = 0.f;  // lane u of a row's group: y of the row of pass u
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int p = p0 + u * RPP + rl;
            float4 v = hv[u];
            v.x = decay * v.x + xv[u] * bv[0];
            v.y = decay * v.y + xv[u] * bv[1];
            v.z = decay * v.z + xv[u] * bv[2];
            v.w = decay * v.w + xv[u] * bv[3];
            if (whole || p < s.P) st[(size_t)p * NL + nl] = v;
            const float part = group_sum<NL>(v.x * cv[0] + v.y * cv[1] + v.z * cv[2] + v.w * cv[3]);
            if (nl == u) keep = part + dh * xv[u];
        }
        const int pq = p0 + nl * RPP + rl;
        if (nl < UN && pq < s.P) yr[pq] = (TO)keep;
    }
}

// ------------------------------------------------------------------------------------------
// T consecutive single-timestep updates in one launch, with per-row resets.  One wave per (b,h)
// keeps its [P,N] state in registers for all T steps (PASSES float4 per lane), so the state is
// read and written once per launch instead of once per step; the next step's x, dt, B, C are
// requested before the current step's arithmetic.  reset[b,t] != 0 zeroes batch row b before
// step t.  Inputs and y have the layout of the scan's tensors: [B,T,...].
// ------------------------------------------------------------------------------------------
template <typename T, typename TO, int NL, int PASSES>
__global__ __launch_bounds__(256) void steps_kernel(float *__restrict__ state, const unsigned char *__restrict__ reset,
                                                    const T *__restrict__ x, const T *__restrict__ dt,
                                                    const float *__restrict__ A, const T *__restrict__ Bm,
                                                    const T *__restrict__ Cm, const float *__restrict__ D,
                                                    TO *__restrict__ y, StepShape s, int nsteps) {
    constexpr int N = NL * 4;
    constexpr int RPP = 64 / NL;  // rows per pass
    const int lane = threadIdx.x & 63;
    const long long bh = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (bh >= (long long)s.B * s.H) return;
    const int b = (int)(bh / s.H), h = (int)(bh % s.H);
    const int g = h / (s.H / s.G);
    const int nl = lane % NL, rl = lane / NL;
    const float a_h = A[h];
    const float dh = D ? D[h] : 0.f;
    float4 *sp = reinterpret_cast<float4 *>(state) + (size_t)bh * s.P * NL;
    float4 hv[PASSES];
#pragma unroll
    for (int u = 0; u < PASSES; ++u) hv[u] = sp[(size_t)(u * RPP + rl) * NL + nl];

    struct StepIn {
        float dtv, bv[4], cv[4], xv[PASSES];
        bool clear;
    };
    auto fetch = [&](int t, StepIn &in) {
        const size_t bt = (size_t)b * nsteps + t;
        in.dtv = (float)dt[bt * s.H + h];
        in.clear = reset != nullptr && reset[bt] != 0;
        const T *bp = Bm + (bt * s.G + g) * N + nl * 4, *cp = Cm + (bt * s.G + g) * N + nl * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            in.bv[i] = (float)bp[i];
            in.cv[i] = (float)cp[i];
        }
        const T *xp = x + (bt * s.H + h) * s.P + rl;
#pragma unroll
        for (int u = 0; u < PASSES; ++u) in.xv[u] = (float)xp[u * RPP];
    };
    StepIn cur, nxt;
    fetch(0, cur);
    for (int t = 0; t < nsteps; ++t) {
        if (t + 1 < nsteps) fetch(t + 1, nxt);
        const float decay = expf(cur.dtv * a_h);
        if (cur.clear) {  // a reset row restarts from zero, whatever the state held (uniform per wave)
#pragma unroll
            for (int u = 0; u < PASSES; ++u) hv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        TO *yp = y + (((size_t)b * nsteps + t) * s.H + h) * s.P + rl;
#pragma unroll
        for (int u = 0; u < PASSES; ++u) {
            const float xd = cur.xv[u] * cur.dtv;
            float4 v = hv[u];
            v.x = decay * v.x + xd * cur.bv[0];
            v.y = decay * v.y + xd * cur.bv[1];
            v.z = decay * v.z + xd * cur.bv[2];
            v.w = decay * v.w + xd * cur.bv[3];
            hv[u] = v;
            float part = v.x * cur.cv[0] + v.y * cur.cv[1] + v.z * cur.cv[2] + v.w * cur.cv[3];
            part = group_sum<NL>(part);
            if (nl == 0) yp[u * RPP] = (TO)(part + dh * cur.xv[u]);
        }
        if (t + 1 < nsteps) cur = nxt;
    }
#pragma unroll
    for (int u = 0; u < PASSES; ++u) sp[(size_t)(u * RPP + rl) * NL + nl] = hv[u];
}

// ------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------
template <typename T>
static hipError_t cumsum_dispatch(const ScanShape &s, const void *dt, const float *A, const unsigned char *reset,
                                  float *dtcs, hipStream_t st, int mode, int dt_len) {
    const dim3 grid(s.B * s.nc), block(256);
    const size_t lds = chunk_cumsum_lds_bytes(s);
    const T *d = static_cast<const T *>(dt);
    hipError_t e;
    if (s.Q <= 64) {
        if ((e = allow_lds(chunk_cumsum_kernel<T, 1>, lds)) != hipSuccess) return e;
        chunk_cumsum_kernel<T, 1><<<grid, block, lds, st>>>(d, A, reset, dtcs, s, mode, dt_len);
    } else if (s.Q == 128) {
        if ((e = allow_lds(chunk_cumsum_kernel<T, 2>, lds)) != hipSuccess) return e;
        chunk_cumsum_kernel<T, 2><<<grid, block, lds, st>>>(d, A, reset, dtcs, s, mode, dt_len);
    } else {
        if ((e = allow_lds(chunk_cumsum_kernel<T, 4>, lds)) != hipSuccess) return e;
        chunk_cumsum_kernel<T, 4><<<grid, block, lds, st>>>(d, A, reset, dtcs, s, mode, dt_len);
    }
    return hipGetLastError();
}

hipError_t launch_chunk_cumsum(const ScanShape &s, int dtype, const void *dt, const float *A,
                               const unsigned char *reset, float *dtcs, hipStream_t st, int mode, int dt_len) {
    if (dt_len <= 0) dt_len = s.L;
    return dtype ? cumsum_dispatch<__bf16>(s, dt, A, reset, dtcs, st, mode, dt_len)
                 : cumsum_dispatch<float>(s, dt, A, reset, dtcs, st, mode, dt_len);
}

hipError_t launch_state_passing(const ScanShape &s, const float *states, const float *dtcs, const float *init,
                                float *prev, float *final_states, hipStream_t st) {
    const long long total = (long long)s.B * s.H * (s.P * s.N / 4);
    const unsigned blocks = (unsigned)((total + 255) / 256);
    state_passing_kernel<<<dim3(blocks), dim3(256), 0, st>>>(states, dtcs, init, prev, final_states, s, total);
    return hipGetLastError();
}

template <typename T, typename TO>
static hipError_t step_dispatch(const StepShape &s, float *state, const void *x, const void *dt,
                                const float *A, const void *Bm, const void *Cm, const float *D, void *y,
                                hipStream_t st) {
    const long long pairs = (long long)s.B * s.H;
    if (pairs > 0x7fffffffLL) return hipErrorInvalidValue;  // the kernel counts (b, h) pairs in an int
    const dim3 grid((unsigned)((pairs + 3) / 4)), block(256);
    const T *xx = static_cast<const T *>(x), *dd = static_cast<const T *>(dt);
    const T *bb = static_cast<const T *>(Bm), *cc = static_cast<const T *>(Cm);
    TO *yy = static_cast<TO *>(y);
    switch (s.N) {
        case 16: step_kernel<T, TO, 4><<<grid, block, 0, st>>>(state, xx, dd, A, bb, cc, D, yy, s); break;
        case 32: step_kernel<T, TO, 8><<<grid, block, 0, st>>>(state, xx, dd, A, bb, cc, D, yy, s); break;
        case 64: step_kernel<T, TO, 16><<<grid, block, 0, st>>>(state, xx, dd, A, bb, cc, D, yy, s); break;
        case 128: step_kernel<T, TO, 32><<<grid, block, 0, st>>>(state, xx, dd, A, bb, cc, D, yy, s); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_step(const StepShape &s, int dtype, float *state, const void *x, const void *dt,
                       const float *A, const void *Bm, const void *Cm, const float *D, void *y,
                       hipStream_t st) {
    switch (dtype) {
        case 0: return step_dispatch<float, float>(s, state, x, dt, A, Bm, Cm, D, y, st);
        case 1: return step_dispatch<__bf16, __bf16>(s, state, x, dt, A, Bm, Cm, D, y, st);
        default: return step_dispatch<__bf16, float>(s, state, x, dt, A, Bm, Cm, D, y, st);
    }
}

template <typename T, typename TO, int NL>
static hipError_t steps_dispatch_p(const StepShape &s, int nsteps, float *state, const unsigned char *reset,
                                   const T *x, const T *dt, const float *A, const T *Bm, const T *Cm,
                                   const float *D, TO *y, hipStream_t st) {
    const long long pairs = (long long)s.B * s.H;
    const dim3 grid((unsigned)((pairs + 3) / 4)), block(256);
    constexpr int RPP = 64 / NL;
    switch (s.P) {
        case 16: steps_kernel<T, TO, NL, 16 / RPP><<<grid, block, 0, st>>>(state, reset, x, dt, A, Bm, Cm, D, y, s, nsteps); break;
        case 32: steps_kernel<T, TO, NL, 32 / RPP><<<grid, block, 0, st>>>(state, reset, x, dt, A, Bm, Cm, D, y, s, nsteps); break;
        case 64: steps_kernel<T, TO, NL, 64 / RPP><<<grid, block, 0, st>>>(state, reset, x, dt, A, Bm, Cm, D, y, s, nsteps); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <typename T, typename TO>
static hipError_t steps_dispatch(const StepShape &s, int nsteps, float *state, const unsigned char *reset,
                                 const void *x, const void *dt, const float *A, const void *Bm, const void *Cm,
                                 const float *D, void *y, hipStream_t st) {
    const T *xx = static_cast<const T *>(x), *dd = static_cast<const T *>(dt);
    const T *bb = static_cast<const T *>(Bm), *cc = static_cast<const T *>(Cm);
    TO *yy = static_cast<TO *>(y);
    switch (s.N) {
        case 16: return steps_dispatch_p<T, TO, 4>(s, nsteps, state, reset, xx, dd, A, bb, cc, D, yy, st);
        case 32: return steps_dispatch_p<T, TO, 8>(s, nsteps, state, reset, xx, dd, A, bb, cc, D, yy, st);
        case 64: return steps_dispatch_p<T, TO, 16>(s, nsteps, state, reset, xx, dd, A, bb, cc, D, yy, st);
        case 128: return steps_dispatch_p<T, TO, 32>(s, nsteps, state, reset, xx, dd, A, bb, cc, D, yy, st);
        default: return hipErrorInvalidValue;
    }
}

bool steps_supported(const StepShape &s) { return s.P == 16 || s.P == 32 || s.P == 64; }

hipError_t launch_steps(const StepShape &s, int nsteps, int dtype, float *state, const unsigned char *reset,
                        const void *x, const void *dt, const float *A, const void *Bm, const void *Cm,
                        const float *D, void *y, hipStream_t st) {
    switch (dtype) {
        case 0: return steps_dispatch<float, float>(s, nsteps, state, reset, x, dt, A, Bm, Cm, D, y, st);
        case 1: return steps_dispatch<__bf16, __bf16>(s, nsteps, state, reset, x, dt, A, Bm, Cm, D, y, st);
        default: return steps_dispatch<__bf16, float>(s, nsteps, state, reset, x, dt, A, Bm, Cm, D, y, st);
    }
}

}  // namespace ssd
