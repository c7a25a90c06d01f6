// The two memory-bound stages of a Mamba-2 block around the SSD scan (gfx950):
//   pre   causal depthwise conv1d (width d_conv) + bias + SiLU over the x, B, C channels of the
//         in-projection's output, split into the tensors the scan takes, and dt = softplus(dt_raw + dt_bias)
//   post  gated RMSNorm: out = rmsnorm(y * silu(z)) * weight
// The projections on either side are plain GEMMs and stay with the caller's BLAS.
//
// Input layout (per timestep, E = 2*H*P + 2*G*N + H channels): [ z | x | B | C | dt_raw ], rows s.ld elements
// apart (ld >= E: a padded row keeps every row's 128-byte lines whole).
#include "ssd_block_common.h"

namespace ssd {

// One thread per (run of kPreSteps timesteps, 8 channels of x | B | C): the filter taps of its channels are
// loaded once and the d_conv-1 previous input rows slide through registers, so every input row is read once
// per run.  The dt channels are done by the threads after those, one (timestep, 8 heads) each, so that no
// wave mixes the two code paths.  History
// before t = 0 comes from state_in [B, d_conv-1, C] (the last d_conv-1 input rows of the previous call) or is
// zero; state_out receives the last d_conv-1 input rows.  reset [B, L] bytes or NULL: a non-zero reset[b,t] cuts
// the filter's history before timestep t (an episode boundary: the rows before t count as zeros from t on, in the
// outputs and in state_out), which is what zeroing the conv state between two calls does at a window boundary.
constexpr int kPreSteps = 16;

template <typename T, int DCONV>
__global__ __launch_bounds__(256) void block_pre_kernel(const T *__restrict__ zxbcdt, const float *__restrict__ conv_w,
                                                        const float *__restrict__ conv_b, const float *__restrict__ dt_bias,
                                                        const T *state_in, T *state_out,
                                                        const unsigned char *__restrict__ reset,
                                                        T *__restrict__ x, T *__restrict__ Bm, T *__restrict__ Cm,
                                                        T *__restrict__ dt, BlockShape s) {
    const int DI = s.H * s.P, GN = s.G * s.N, C = DI + 2 * GN;
    const int CP = C / 8, HP8 = (s.H + 7) / 8;
    const int runs = (s.L + kPreSteps - 1) / kPreSteps;
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long conv_total = (long long)s.B * runs * CP;
    if (gid >= conv_total) {
        // the threads after the conv threads: dt = softplus(dt_raw + dt_bias), one (timestep, 8 heads) each
        const long long d = gid - conv_total;
        if (d >= (long long)s.B * s.L * HP8) return;
        const int h0 = (int)(d % HP8) * 8;
        const long long bt = d / HP8;
        const T *src = zxbcdt + (size_t)bt * s.ld + 2 * DI + 2 * GN;
        if (s.H % 8 == 0) {  // eight heads are one aligned 16-byte (bf16) piece on both sides
            const Pack8<T> v = Pack8<T>::load(src + h0);
            const float4 b0 = *reinterpret_cast<const float4 *>(dt_bias + h0), b1 = *reinterpret_cast<const float4 *>(dt_bias + h0 + 4);
            const float bias[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
            float o[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = softplus(v.get(i) + bias[i]);
            Pack8<T>::store(dt + (size_t)bt * s.H + h0, o);
            return;
        }
        for (int h = h0; h < min(h0 + 8, s.H); ++h) dt[(size_t)bt * s.H + h] = (T)softplus((float)src[h] + dt_bias[h]);
        return;
    }
    const int piece = (int)(gid % CP);
    const long long br = gid / CP;
    const int t0 = (int)(br % runs) * kPreSteps, b = (int)(br / runs);
    const int t1 = min(t0 + kPreSteps, s.L);
    const T *row0 = zxbcdt + ((size_t)b * s.L) * s.ld;  // this batch row's first timestep
    const int c0 = piece * 8;  // channel within [x | B | C]
    // Every load of the thread is issued before the first is used and none is under a condition (a conditional load
    // is a branch, and the compiler waits for all earlier loads -- and stores -- at every one): rows outside the
    // sequence read a row inside it and are replaced by zeros or never stored.
    // the run's input rows
    Pack8<T> in[kPreSteps];
#pragma unroll
    for (int j = 0; j < kPreSteps; ++j) in[j] = Pack8<T>::load(row0 + (size_t)min(t0 + j, s.L - 1) * s.ld + DI + c0);
    // the d_conv-1 rows before the run: rows of this call, of state_in, or zeros
    Pack8<T> hist[DCONV - 1];
#pragma unroll
    for (int k = 0; k < DCONV - 1; ++k) {
        const int ts = t0 - (DCONV - 1) + k;
        const T *own = row0 + (size_t)max(ts, 0) * s.ld + DI + c0;
        const T *old = state_in != nullptr ? state_in + ((size_t)b * (DCONV - 1) + max(DCONV - 1 + ts, 0)) * C + c0 : own;
        hist[k] = Pack8<T>::load(ts >= 0 ? own : old);
    }
    // restart flags of the d_conv-2 steps before the run and of its own steps (bit j: step t0 - (DCONV-2) + j)
    const unsigned char *rs = reset ? reset + (size_t)b * s.L : nullptr;
    unsigned flags = 0;
    if (rs != nullptr) {
        unsigned char rv[kPreSteps + DCONV - 2];
#pragma unroll
        for (int j = 0; j < kPreSteps + DCONV - 2; ++j) rv[j] = rs[min(max(t0 - (DCONV - 2) + j, 0), s.L - 1)];
#pragma unroll
        for (int j = 0; j < kPreSteps + DCONV - 2; ++j) {
            const int ts = t0 - (DCONV - 2) + j;
            flags |= (ts >= 0 && ts < s.L && rv[j] != 0) ? (1u << j) : 0u;
        }
    }
    float w[8][DCONV], bias[8];
    {   // the taps of 8 consecutive channels are 8*DCONV consecutive floats
        float wf[8 * DCONV];
#pragma unroll
        for (int q = 0; q < 2 * DCONV; ++q) {
            const float4 v = *reinterpret_cast<const float4 *>(conv_w + (size_t)c0 * DCONV + 4 * q);
            wf[4 * q] = v.x; wf[4 * q + 1] = v.y; wf[4 * q + 2] = v.z; wf[4 * q + 3] = v.w;
        }
        const float4 b0 = *reinterpret_cast<const float4 *>(conv_b + c0), b1 = *reinterpret_cast<const float4 *>(conv_b + c0 + 4);
        bias[0] = b0.x; bias[1] = b0.y; bias[2] = b0.z; bias[3] = b0.w;
        bias[4] = b1.x; bias[5] = b1.y; bias[6] = b1.z; bias[7] = b1.w;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int k = 0; k < DCONV; ++k) w[i][k] = wf[i * DCONV + k];
        }
    }
    // win[k] = input row t - (DCONV-1) + k for the current t; the last slot is filled per timestep
    float win[DCONV][8];
#pragma unroll
    for (int k = 0; k < DCONV - 1; ++k) {
        const int ts = t0 - (DCONV - 1) + k;
        const bool have = ts >= 0 || state_in != nullptr;
#pragma unroll
        for (int i = 0; i < 8; ++i) win[k][i] = have ? hist[k].get(i) : 0.f;
    }
    {
        // a restart at one of the d_conv-2 timesteps before this run cuts the window rows before it
        bool cut = false;
#pragma unroll
        for (int k = DCONV - 2; k >= 1; --k) {  // window row k is timestep t0 - (DCONV-1) + k: flag bit k - 1
            cut = cut || ((flags >> (k - 1)) & 1u) != 0;
            if (cut) {
#pragma unroll
                for (int i = 0; i < 8; ++i) win[k - 1][i] = 0.f;
            }
        }
    }
    T *dst;
    int dst_stride;
    if (c0 < DI) {
        dst = x + ((size_t)b * s.L) * DI + c0;
        dst_stride = DI;
    } else if (c0 < DI + GN) {
        dst = Bm + ((size_t)b * s.L) * GN + (c0 - DI);
        dst_stride = GN;
    } else {
        dst = Cm + ((size_t)b * s.L) * GN + (c0 - DI - GN);
        dst_stride = GN;
    }
#pragma unroll
    for (int j = 0; j < kPreSteps; ++j) {
        const int t = t0 + j;
        if (t >= t1) break;
        const Pack8<T> v = in[j];
        if ((flags >> (j + DCONV - 2)) & 1u) {
#pragma unroll
            for (int k = 0; k < DCONV - 1; ++k) {
#pragma unroll
                for (int i = 0; i < 8; ++i) win[k][i] = 0.f;
            }
        }
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            win[DCONV - 1][i] = v.get(i);
            float a = bias[i];
#pragma unroll
            for (int k = 0; k < DCONV; ++k) a += w[i][k] * win[k][i];
            acc[i] = silu(a);
        }
        Pack8<T>::store(dst + (size_t)t * dst_stride, acc);
#pragma unroll
        for (int k = 0; k < DCONV - 1; ++k) {
#pragma unroll
            for (int i = 0; i < 8; ++i) win[k][i] = win[k + 1][i];
        }
    }
    // Streaming state: the d_conv-1 input rows before timestep L.  After the run that ends the sequence the window
    // registers hold exactly those rows -- rows of this call, or, where the call brought fewer than d_conv-1 new
    // rows, the tail of state_in, which was loaded before anything was stored: state_in and state_out may be the
    // same memory whenever one thread both reads and writes a channel piece's state (seqlen <= kPreSteps).
    if (state_out != nullptr && t1 == s.L) {
#pragma unroll
        for (int k = 0; k < DCONV - 1; ++k) Pack8<T>::store(state_out + ((size_t)b * (DCONV - 1) + k) * C + c0, win[k]);
    }
}

// LPR lanes per (b, t) row, 64 / LPR rows per wave: out = rmsnorm(y * silu(z)) * weight over the H*P channels.
// LPR is the smallest of 16, 32, 64 whose lanes cover the row with at most 4 pieces of 8 channels each, so that
// narrow rows (256 channels are 32 pieces) leave no lane idle; PPL is the number of pieces a lane holds.  All of a
// lane's loads are issued before the first is used and none is under a condition -- a conditional load is a branch,
// and the compiler waits for every earlier load at each one: a piece past the row's end reads the row's last piece
// and counts as zeros, a row past the tensor reads row 0 and is not stored.
template <typename T, typename TY, int LPR, int PPL>
__global__ __launch_bounds__(256) void block_post_kernel(const TY *__restrict__ y, const T *__restrict__ zxbcdt,
                                                         const float *__restrict__ norm_w, float eps,
                                                         T *__restrict__ out, BlockShape s) {
    const int DI = s.H * s.P;
    const int lane = threadIdx.x & (LPR - 1);
    const long long row = ((long long)blockIdx.x * blockDim.x + threadIdx.x) / LPR;
    const bool live = row < (long long)s.B * s.L;  // (whole waves stay for the lane exchanges)
    const TY *yr = y + (size_t)(live ? row : 0) * DI;
    const T *zr = zxbcdt + (size_t)(live ? row : 0) * s.ld;
    Pack8<TY> yv[PPL];
    Pack8<T> zv[PPL];
    typedef float f4 __attribute__((ext_vector_type(4)));
    f4 wa[PPL], wb[PPL];
#pragma unroll
    for (int u = 0; u < PPL; ++u) {
        const int c0 = min((u * LPR + lane) * 8, DI - 8);
        yv[u] = Pack8<TY>::load(yr + c0);
        zv[u] = Pack8<T>::load(zr + c0);
    }
#pragma unroll
    for (int u = 0; u < PPL; ++u) {
        const int c0 = min((u * LPR + lane) * 8, DI - 8);
        wa[u] = *reinterpret_cast<const f4 *>(norm_w + c0);
        wb[u] = *reinterpret_cast<const f4 *>(norm_w + c0 + 4);
    }
    // (named as inputs of one statement here, the weights cannot be requested later than this: left alone, the
    // compiler moves their loads behind the arithmetic on y and z, a second trip to memory)
    if constexpr (PPL == 1) asm volatile("" ::"v"(wa[0]), "v"(wb[0]));
    if constexpr (PPL == 2) asm volatile("" ::"v"(wa[0]), "v"(wb[0]), "v"(wa[1]), "v"(wb[1]));
    if constexpr (PPL == 3) asm volatile("" ::"v"(wa[0]), "v"(wb[0]), "v"(wa[1]), "v"(wb[1]), "v"(wa[2]), "v"(wb[2]));
    if constexpr (PPL == 4)
        asm volatile("" ::"v"(wa[0]), "v"(wb[0]), "v"(wa[1]), "v"(wb[1]), "v"(wa[2]), "v"(wb[2]), "v"(wa[3]), "v"(wb[3]));
    float v[PPL][8];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < PPL; ++u) {
        // (a factor, not a select: a select would put every element's exponential under a branch of its own)
        const float in = (u * LPR + lane) * 8 < DI ? 1.f : 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[u][i] = in * yv[u].get(i) * silu(zv[u].get(i));
            ss += v[u][i] * v[u][i];
        }
    }
    ss = group_sum<LPR>(ss);
    const float scale = rsqrtf(ss / (float)DI + eps);
#pragma unroll
    for (int u = 0; u < PPL; ++u) {
        const int c0 = (u * LPR + lane) * 8;
        const float w[8] = {wa[u].x, wa[u].y, wa[u].z, wa[u].w, wb[u].x, wb[u].y, wb[u].z, wb[u].w};
        float o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = v[u][i] * scale * w[i];
        if (c0 < DI && live) Pack8<T>::store(out + (size_t)row * DI + c0, o);
    }
}

bool block_supported(const BlockShape &s) {
    return (s.d_conv >= 2 && s.d_conv <= 4) && (s.H * s.P) % 8 == 0 && (s.G * s.N) % 8 == 0 && s.H * s.P <= 2048;
}

template <typename T>
static hipError_t pre_dispatch(const BlockShape &s, const void *zxbcdt, const float *conv_w, const float *conv_b,
                               const float *dt_bias, const void *state_in, void *state_out,
                               const unsigned char *reset, void *x, void *Bm, void *Cm, void *dt, hipStream_t st) {
    const long long total = (long long)s.B * ((s.L + kPreSteps - 1) / kPreSteps) * ((s.H * s.P + 2 * s.G * s.N) / 8) +
                            (long long)s.B * s.L * ((s.H + 7) / 8);
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    const T *in = static_cast<const T *>(zxbcdt), *si = static_cast<const T *>(state_in);
    T *so = static_cast<T *>(state_out), *xx = static_cast<T *>(x), *bb = static_cast<T *>(Bm), *cc = static_cast<T *>(Cm),
      *dd = static_cast<T *>(dt);
    switch (s.d_conv) {
        case 2: block_pre_kernel<T, 2><<<grid, block, 0, st>>>(in, conv_w, conv_b, dt_bias, si, so, reset, xx, bb, cc, dd, s); break;
        case 3: block_pre_kernel<T, 3><<<grid, block, 0, st>>>(in, conv_w, conv_b, dt_bias, si, so, reset, xx, bb, cc, dd, s); break;
        case 4: block_pre_kernel<T, 4><<<grid, block, 0, st>>>(in, conv_w, conv_b, dt_bias, si, so, reset, xx, bb, cc, dd, s); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_block_pre(const BlockShape &s, int dtype, const void *zxbcdt, const float *conv_w,
                            const float *conv_b, const float *dt_bias, const void *state_in, void *state_out,
                            const unsigned char *reset, void *x, void *Bm, void *Cm, void *dt, hipStream_t st) {
    return dtype ? pre_dispatch<__bf16>(s, zxbcdt, conv_w, conv_b, dt_bias, state_in, state_out, reset, x, Bm, Cm, dt, st)
                 : pre_dispatch<float>(s, zxbcdt, conv_w, conv_b, dt_bias, state_in, state_out, reset, x, Bm, Cm, dt, st);
}

template <typename T, typename TY>
static hipError_t post_dispatch(const BlockShape &s, const void *y, const void *zxbcdt, const float *norm_w, float eps,
                                void *out, hipStream_t st) {
    const long long rows = (long long)s.B * s.L;
    const int pieces = s.H * s.P / 8;
    const TY *yy = static_cast<const TY *>(y);
    const T *zz = static_cast<const T *>(zxbcdt);
    T *oo = static_cast<T *>(out);
    // the fewest lanes per row that keep a lane's pieces within four, and the pieces a lane then holds
    const int lpr = pieces <= 16 * 4 ? 16 : pieces <= 32 * 4 ? 32 : 64;
    const int ppl = (pieces + lpr - 1) / lpr;
    const dim3 grid((unsigned)((rows * lpr + 255) / 256)), block(256);
#define SSD_POST_CASE(LPRv, PPLv)                                                                        \
    if (lpr == LPRv && ppl == PPLv) {                                                                    \
        block_post_kernel<T, TY, LPRv, PPLv><<<grid, block, 0, st>>>(yy, zz, norm_w, eps, oo, s);         \
        return hipGetLastError();                                                                        \
    }
    SSD_POST_CASE(16, 1) SSD_POST_CASE(16, 2) SSD_POST_CASE(16, 3) SSD_POST_CASE(16, 4)
    SSD_POST_CASE(32, 3) SSD_POST_CASE(32, 4)
    SSD_POST_CASE(64, 3) SSD_POST_CASE(64, 4)
#undef SSD_POST_CASE
    return hipErrorInvalidValue;
}

hipError_t launch_block_post(const BlockShape &s, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                             float eps, void *out, hipStream_t st) {
    switch (dtype) {
        case 0: return post_dispatch<float, float>(s, y, zxbcdt, norm_w, eps, out, st);
        case 1: return post_dispatch<__bf16, __bf16>(s, y, zxbcdt, norm_w, eps, out, st);
        default: return post_dispatch<__bf16, float>(s, y, zxbcdt, norm_w, eps, out, st);  // the scan's float32 y
    }
}

}  // namespace ssd
