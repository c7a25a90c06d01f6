// Backward pass of the two memory-bound stages of a Mamba-2 block around the SSD scan (gfx950):
//   post_bwd  gradients of out = rmsnorm(y * silu(z)) * w: dy, dz (into the z channels of dzxbcdt), dw
//   pre_bwd   gradients of the causal depthwise conv + SiLU over x | B | C and of dt = softplus(dt_raw + bias):
//             the x | B | C | dt channels of dzxbcdt, dconv_w, dconv_b, ddt_bias, and the gradient of the conv state
// Between them sits ssd_chunk_scan_bwd; the projections on either side are two plain GEMMs each (the caller's BLAS).
//
// Parameter gradients are sums over batch and time.  Every workgroup leaves its partial sums in the workspace and a
// second small kernel adds the partials in a fixed order, so results do not depend on timing (no float atomics).
#include <algorithm>

#include "ssd_block_common.h"

namespace ssd {

namespace {

constexpr int kBwdSteps = 16;    // timesteps per thread of the conv backward (its forward's run length)
constexpr int kPiecesPerBlock = 16;  // channel pieces (of 8) per workgroup of the conv backward
constexpr int kRunsPerBlock = 16;
constexpr int kPostBlocks = 1024;    // workgroups of post_bwd (each walks rows with a grid stride)

// ---- post ----------------------------------------------------------------------------------------------------
// LPR lanes per (b, t) row as in the forward; v = y silu(z), r = (mean v^2 + eps)^-1/2, g = dout w:
//   dv = r g - r^3 v mean(g v);  dy = dv silu(z);  dz = dv y silu'(z);  dw += dout v r
template <typename T, typename TY, int LPR>
__global__ __launch_bounds__(256) void block_post_bwd_kernel(const TY *__restrict__ y, const T *__restrict__ zxbcdt,
                                                             const float *__restrict__ norm_w, float eps,
                                                             const T *__restrict__ dout, T *__restrict__ dy,
                                                             T *__restrict__ dzxbcdt, float *__restrict__ dw_part,
                                                             BlockShape s) {
    const int DI = s.H * s.P;
    const int lane = threadIdx.x & (LPR - 1);
    constexpr int MAXP = 4;
    constexpr int RPB = 256 / LPR;  // rows per workgroup and pass
    const long long rows = (long long)s.B * s.L;
    float wv[MAXP][8], dwacc[MAXP][8];
#pragma unroll
    for (int u = 0; u < MAXP; ++u) {
        const int c0 = (u * LPR + lane) * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            wv[u][i] = c0 < DI ? norm_w[c0 + i] : 0.f;
            dwacc[u][i] = 0.f;
        }
    }
    const float inv_di = 1.f / (float)DI;
    for (long long row0 = (long long)blockIdx.x * RPB; row0 < rows; row0 += (long long)gridDim.x * RPB) {
        const long long row = row0 + threadIdx.x / LPR;
        const bool live = row < rows;  // (whole waves stay for the lane exchanges)
        const size_t r_ = live ? (size_t)row : 0;
        float yy[MAXP][8], zz[MAXP][8], dd[MAXP][8];
        float ss = 0.f, gv = 0.f;
#pragma unroll
        for (int u = 0; u < MAXP; ++u) {
            const int c0 = (u * LPR + lane) * 8;
            if (c0 < DI) {
                const Pack8<TY> yv = Pack8<TY>::load(y + r_ * DI + c0);
                const Pack8<T> zv = Pack8<T>::load(zxbcdt + r_ * s.ld + c0);
                const Pack8<T> dv = Pack8<T>::load(dout + r_ * DI + c0);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    yy[u][i] = yv.get(i);
                    zz[u][i] = zv.get(i);
                    dd[u][i] = dv.get(i);
                    const float v = yy[u][i] * silu(zz[u][i]);
                    ss += v * v;
                    gv += dd[u][i] * wv[u][i] * v;
                }
            }
        }
#pragma unroll
        for (int m = LPR / 2; m >= 1; m >>= 1) {
            ss += __shfl_xor(ss, m, 64);
            gv += __shfl_xor(gv, m, 64);
        }
        const float r = rsqrtf(ss * inv_di + eps);
        const float k3 = r * r * r * gv * inv_di;
#pragma unroll
        for (int u = 0; u < MAXP; ++u) {
            const int c0 = (u * LPR + lane) * 8;
            if (c0 < DI && live) {
                float oy[8], oz[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float sz = silu(zz[u][i]);
                    const float v = yy[u][i] * sz;
                    const float dvv = r * dd[u][i] * wv[u][i] - k3 * v;
                    oy[i] = dvv * sz;
                    oz[i] = dvv * yy[u][i] * dsilu(zz[u][i]);
                    dwacc[u][i] += dd[u][i] * v * r;
                }
                Pack8<T>::store(dy + (size_t)row * DI + c0, oy);
                Pack8<T>::store(dzxbcdt + (size_t)row * s.ld + c0, oz);
            }
        }
    }
    // the workgroup's partial of dw: the RPB row slots of every channel, added in slot order
    __shared__ float red[256 * 8];
#pragma unroll
    for (int u = 0; u < MAXP; ++u) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i) red[threadIdx.x * 8 + i] = dwacc[u][i];
        __syncthreads();
        if (threadIdx.x < LPR) {
            const int c0 = (u * LPR + threadIdx.x) * 8;
            if (c0 < DI) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float acc = 0.f;
                    for (int q = 0; q < RPB; ++q) acc += red[(q * LPR + threadIdx.x) * 8 + i];
                    dw_part[(size_t)blockIdx.x * DI + c0 + i] = acc;
                }
            }
        }
    }
}

// out[c] = sum over parts of part[p][c], in order (columns = channels)
__global__ __launch_bounds__(256) void column_sums_kernel(const float *__restrict__ part, int nparts, int cols,
                                                          float *__restrict__ out) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    float acc = 0.f;
    for (int p = 0; p < nparts; ++p) acc += part[(size_t)p * cols + c];
    out[c] = acc;
}

// ---- pre -----------------------------------------------------------------------------------------------------
// One thread per (run of kBwdSteps timesteps, 8 channels of x | B | C).  pre[t] = b + sum_k w[k] in[t-(K-1)+k]
// (taps before the latest restart at or before t cut), out = silu(pre); with dpre[t] = dout[t] silu'(pre[t]):
//   din[s]  = sum_{j=0..K-1} w[K-1-j] dpre[s+j]      over the j whose output s+j exists and lies before any restart
//                                                     after s
//   dw[k]  += dpre[t] in[t-(K-1)+k] (live taps),  db += dpre[t]
// The thread recomputes pre over its run and K-1 timesteps beyond it.  The run that starts at t = 0 also leaves the
// gradient of the conv state (the inputs before t = 0); a gradient on the returned conv state joins din of the last
// K-1 timesteps.
template <typename T, int K>
__global__ __launch_bounds__(256) void block_pre_bwd_kernel(const T *__restrict__ zxbcdt, const float *__restrict__ conv_w,
                                                            const float *__restrict__ conv_b, const T *__restrict__ state_in,
                                                            const unsigned char *__restrict__ reset, const T *__restrict__ dx,
                                                            const T *__restrict__ dB, const T *__restrict__ dC,
                                                            const T *__restrict__ dstate_out, T *__restrict__ dzxbcdt,
                                                            T *__restrict__ dstate_in, float *__restrict__ part, BlockShape s) {
    const int DI = s.H * s.P, GN = s.G * s.N, C = DI + 2 * GN;
    const int CP = C / 8;
    const int runs = (s.L + kBwdSteps - 1) / kBwdSteps;
    const int pl = threadIdx.x % kPiecesPerBlock, rl = threadIdx.x / kPiecesPerBlock;
    const int piece = blockIdx.x * kPiecesPerBlock + pl;
    const long long br = (long long)blockIdx.y * kRunsPerBlock + rl;
    const bool active = piece < CP && br < (long long)s.B * runs;
    float dwacc[8][K], dbacc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        dbacc[i] = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k) dwacc[i][k] = 0.f;
    }
    if (active) {
        const int t0 = (int)(br % runs) * kBwdSteps, b = (int)(br / runs);
        const int t1 = min(t0 + kBwdSteps, s.L);
        const int c0 = piece * 8;
        const T *row0 = zxbcdt + ((size_t)b * s.L) * s.ld + DI + c0;
        const unsigned char *rs = reset ? reset + (size_t)b * s.L : nullptr;
        float w[8][K], bias[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            bias[i] = conv_b[c0 + i];
#pragma unroll
            for (int k = 0; k < K; ++k) w[i][k] = conv_w[(size_t)(c0 + i) * K + k];
        }
        // where the gradient of the scan's input for these channels comes from
        const T *gsrc;
        int gstride;
        if (c0 < DI) {
            gsrc = dx + ((size_t)b * s.L) * DI + c0;
            gstride = DI;
        } else if (c0 < DI + GN) {
            gsrc = dB + ((size_t)b * s.L) * GN + (c0 - DI);
            gstride = GN;
        } else {
            gsrc = dC + ((size_t)b * s.L) * GN + (c0 - DI - GN);
            gstride = GN;
        }
        // input row of timestep ts (history before 0 from the conv state, zero without one)
        auto in_row = [&](int ts, float (&v)[8]) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = 0.f;
            if (ts >= 0) {
                const Pack8<T> p = Pack8<T>::load(row0 + (size_t)ts * s.ld);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = p.get(i);
            } else if (state_in != nullptr) {
                const Pack8<T> p = Pack8<T>::load(state_in + ((size_t)b * (K - 1) + (K - 1 + ts)) * C + c0);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = p.get(i);
            }
        };
        // dpre of the timesteps t0 .. t0 + kBwdSteps + K - 2 (zero past the sequence), from a window of inputs that slides
        constexpr int NT = kBwdSteps + K - 1;
        float dpre[NT][8];
        float win[K][8];
        // `depth` = how many of the window's older rows are still live: a restart at t makes it zero for t itself
        int depth = K - 1;
#pragma unroll
        for (int k = 0; k < K - 1; ++k) in_row(t0 - (K - 1) + k, win[k]);
        if (rs != nullptr) {
            // restarts at the K-2 timesteps before the run cut the rows before them
            depth = K - 1;
            for (int back = 1; back <= K - 2; ++back) {
                const int ts = t0 - back;
                if (ts >= 0 && rs[ts] != 0) {
                    depth = back;
                    break;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int t = t0 + j;
            const bool exists = t < s.L;
            if (exists) in_row(t, win[K - 1]);
            if (exists && rs != nullptr && rs[t] != 0) depth = 0;
            float gin[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) gin[i] = 0.f;
            if (exists) {
                const Pack8<T> p = Pack8<T>::load(gsrc + (size_t)t * gstride);
#pragma unroll
                for (int i = 0; i < 8; ++i) gin[i] = p.get(i);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float a = bias[i];
#pragma unroll
                for (int k = 0; k < K; ++k) a += (K - 1 - k <= depth) ? w[i][k] * win[k][i] : 0.f;
                dpre[j][i] = exists ? gin[i] * dsilu(a) : 0.f;
            }
            if (exists && t < t1) {  // this thread's own timesteps: the parameter gradients
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    dbacc[i] += dpre[j][i];
#pragma unroll
                    for (int k = 0; k < K; ++k) dwacc[i][k] += (K - 1 - k <= depth) ? dpre[j][i] * win[k][i] : 0.f;
                }
            }
#pragma unroll
            for (int k = 0; k < K - 1; ++k) {
#pragma unroll
                for (int i = 0; i < 8; ++i) win[k][i] = win[k + 1][i];
            }
            if (depth < K - 1) ++depth;
        }
        // din[s] for the run's timesteps: outputs s .. s+K-1 while no restart lies after s
        T *drow = dzxbcdt + ((size_t)b * s.L) * s.ld + DI + c0;
#pragma unroll
        for (int j = 0; j < kBwdSteps; ++j) {
            const int sidx = t0 + j;
            if (sidx >= t1) break;
            float o[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = 0.f;
            bool open = true;
#pragma unroll
            for (int q = 0; q < K; ++q) {
                const int t = sidx + q;
                if (q > 0 && open && t < s.L && rs != nullptr && rs[t] != 0) open = false;
                if (open && t < s.L) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) o[i] += w[i][K - 1 - q] * dpre[j + q][i];
                }
            }
            // a gradient on the conv state the forward returned: that state is the last K-1 input rows, those before
            // the window's last restart zeroed
            if (dstate_out != nullptr && sidx >= s.L - (K - 1)) {
                bool kept = true;
                for (int t = sidx + 1; t < s.L; ++t) kept = kept && !(rs != nullptr && rs[t] != 0);
                if (kept) {
                    const Pack8<T> p = Pack8<T>::load(dstate_out + ((size_t)b * (K - 1) + (sidx - (s.L - (K - 1)))) * C + c0);
#pragma unroll
                    for (int i = 0; i < 8; ++i) o[i] += p.get(i);
                }
            }
            Pack8<T>::store(drow + (size_t)sidx * s.ld, o);
        }
        // the gradient of the conv state: inputs at s = -(K-1) .. -1 reach outputs 0 .. s+K-1, up to the first restart
        if (t0 == 0 && dstate_in != nullptr) {
#pragma unroll
            for (int jrow = 0; jrow < K - 1; ++jrow) {
                const int sidx = jrow - (K - 1);
                float o[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = 0.f;
                bool open = true;
#pragma unroll
                for (int t = 0; t < K - 1; ++t) {
                    if (open && t < s.L && rs != nullptr && rs[t] != 0) open = false;
                    const int k = sidx - t + (K - 1);
                    if (open && t < s.L && k >= 0) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) o[i] += w[i][k] * dpre[t][i];
                    }
                }
                // rows of the old state that are still part of the new one (fewer than K-1 new timesteps)
                if (dstate_out != nullptr && sidx >= s.L - (K - 1)) {
                    bool kept = true;
                    for (int t = 0; t < s.L; ++t) kept = kept && !(rs != nullptr && rs[t] != 0);
                    if (kept) {
                        const Pack8<T> p = Pack8<T>::load(dstate_out + ((size_t)b * (K - 1) + (sidx - (s.L - (K - 1)))) * C + c0);
#pragma unroll
                        for (int i = 0; i < 8; ++i) o[i] += p.get(i);
                    }
                }
                Pack8<T>::store(dstate_in + ((size_t)b * (K - 1) + jrow) * C + c0, o);
            }
        }
    }
    // the workgroup's partial sums: per channel piece, its kRunsPerBlock threads added in order
    __shared__ float red[256 * (K + 1)];
    const int cols = C * (K + 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        __syncthreads();
#pragma unroll
        for (int k = 0; k < K; ++k) red[threadIdx.x * (K + 1) + k] = dwacc[i][k];
        red[threadIdx.x * (K + 1) + K] = dbacc[i];
        __syncthreads();
        if (rl == 0 && piece < CP) {
            const int c = piece * 8 + i;
#pragma unroll
            for (int k = 0; k <= K; ++k) {
                float acc = 0.f;
                for (int q = 0; q < kRunsPerBlock; ++q) acc += red[(q * kPiecesPerBlock + pl) * (K + 1) + k];
                part[(size_t)blockIdx.y * cols + (size_t)c * (K + 1) + k] = acc;
            }
        }
    }
}

// ddt_raw = ddt sigmoid(dt_raw + dt_bias) into the dt channels of dzxbcdt; per workgroup the sums over its rows
template <typename T>
__global__ __launch_bounds__(256) void block_dt_bwd_kernel(const T *__restrict__ zxbcdt, const float *__restrict__ dt_bias,
                                                           const T *__restrict__ ddt, T *__restrict__ dzxbcdt,
                                                           float *__restrict__ part, BlockShape s) {
    const int DI = s.H * s.P, GN = s.G * s.N, off = 2 * DI + 2 * GN;
    const long long rows = (long long)s.B * s.L;
    __shared__ float red[256];
    for (int h0 = 0; h0 < s.H; h0 += 256) {
        // thread = (row slot, head): heads fastest so that a row's heads are adjacent
        const int hpt = min(s.H - h0, 256);          // heads handled in this pass
        const int slots = 256 / hpt;                 // rows per pass
        const int h = h0 + threadIdx.x % hpt, slot = threadIdx.x / hpt;
        float acc = 0.f;
        if (slot < slots) {
            const float bias = dt_bias[h];
            for (long long row = (long long)blockIdx.x * slots + slot; row < rows; row += (long long)gridDim.x * slots) {
                const float raw = (float)zxbcdt[(size_t)row * s.ld + off + h] + bias;
                const float g = (float)ddt[(size_t)row * s.H + h] * sigmoidf(raw);
                dzxbcdt[(size_t)row * s.ld + off + h] = (T)g;
                acc += g;
            }
        }
        __syncthreads();
        red[threadIdx.x] = acc;
        __syncthreads();
        if (threadIdx.x < hpt) {
            float sum = 0.f;
            for (int q = 0; q < slots; ++q) sum += red[q * hpt + threadIdx.x];
            part[(size_t)blockIdx.x * s.H + h0 + threadIdx.x] = sum;
        }
    }
}

constexpr int kDtBlocks = 512;

// [C][K+1] sums -> dconv_w [C][K], dconv_b [C]
__global__ __launch_bounds__(256) void split_conv_sums_kernel(const float *__restrict__ sums, int C, int K,
                                                              float *__restrict__ dw, float *__restrict__ db) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    for (int k = 0; k < K; ++k) dw[(size_t)c * K + k] = sums[(size_t)c * (K + 1) + k];
    db[c] = sums[(size_t)c * (K + 1) + K];
}

}  // namespace

// workspace: the partial sums of post_bwd, or those of pre_bwd (conv, their column sums, dt)
size_t block_bwd_workspace_bytes(const BlockShape &s) {
    const size_t DI = (size_t)s.H * s.P, C = DI + 2 * (size_t)s.G * s.N;
    const size_t runs = (s.L + kBwdSteps - 1) / kBwdSteps;
    const size_t run_blocks = ((size_t)s.B * runs + kRunsPerBlock - 1) / kRunsPerBlock;
    const size_t post = (size_t)kPostBlocks * DI;
    const size_t pre = (run_blocks + 1) * C * (s.d_conv + 1) + (size_t)kDtBlocks * s.H;
    return sizeof(float) * (post > pre ? post : pre);  // the two stages run one after the other and share it
}

template <typename T, typename TY>
static hipError_t post_bwd_dispatch(const BlockShape &s, const void *y, const void *zxbcdt, const float *norm_w, float eps,
                                    const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, float *part, hipStream_t st) {
    const int DI = s.H * s.P, pieces = DI / 8;
    const long long rows = (long long)s.B * s.L;
    const TY *yy = static_cast<const TY *>(y);
    const T *zz = static_cast<const T *>(zxbcdt), *dd = static_cast<const T *>(dout);
    T *oy = static_cast<T *>(dy), *oz = static_cast<T *>(dzxbcdt);
    int blocks;
    if (pieces <= 16 * 4) {
        blocks = (int)std::min<long long>(kPostBlocks, (rows + 15) / 16);
        block_post_bwd_kernel<T, TY, 16><<<dim3(blocks), dim3(256), 0, st>>>(yy, zz, norm_w, eps, dd, oy, oz, part, s);
    } else if (pieces <= 32 * 4) {
        blocks = (int)std::min<long long>(kPostBlocks, (rows + 7) / 8);
        block_post_bwd_kernel<T, TY, 32><<<dim3(blocks), dim3(256), 0, st>>>(yy, zz, norm_w, eps, dd, oy, oz, part, s);
    } else {
        blocks = (int)std::min<long long>(kPostBlocks, (rows + 3) / 4);
        block_post_bwd_kernel<T, TY, 64><<<dim3(blocks), dim3(256), 0, st>>>(yy, zz, norm_w, eps, dd, oy, oz, part, s);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    column_sums_kernel<<<dim3((DI + 255) / 256), dim3(256), 0, st>>>(part, blocks, DI, dnorm_w);
    return hipGetLastError();
}

hipError_t launch_block_post_bwd(const BlockShape &s, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                                 float eps, const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, void *workspace,
                                 hipStream_t st) {
    float *part = static_cast<float *>(workspace);
    switch (dtype) {
        case 0: return post_bwd_dispatch<float, float>(s, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, part, st);
        case 1: return post_bwd_dispatch<__bf16, __bf16>(s, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, part, st);
        default: return post_bwd_dispatch<__bf16, float>(s, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, part, st);
    }
}

template <typename T>
static hipError_t pre_bwd_dispatch(const BlockShape &s, const void *zxbcdt, const float *conv_w, const float *conv_b,
                                   const float *dt_bias, const void *state_in, const unsigned char *reset, const void *dx,
                                   const void *dB, const void *dC, const void *ddt, const void *dstate_out, void *dzxbcdt,
                                   float *dconv_w, float *dconv_b, float *ddt_bias, void *dstate_in, float *part,
                                   hipStream_t st) {
    const int DI = s.H * s.P, C = DI + 2 * s.G * s.N, CP = C / 8, K = s.d_conv;
    const long long runs = (s.L + kBwdSteps - 1) / kBwdSteps;
    const long long run_blocks = ((long long)s.B * runs + kRunsPerBlock - 1) / kRunsPerBlock;
    if (run_blocks > 65535LL * 32768LL) return hipErrorInvalidValue;
    const dim3 grid((CP + kPiecesPerBlock - 1) / kPiecesPerBlock, (unsigned)run_blocks);
    const T *in = static_cast<const T *>(zxbcdt), *si = static_cast<const T *>(state_in);
    const T *gx = static_cast<const T *>(dx), *gb = static_cast<const T *>(dB), *gc = static_cast<const T *>(dC);
    const T *gso = static_cast<const T *>(dstate_out);
    T *out = static_cast<T *>(dzxbcdt), *gsi = static_cast<T *>(dstate_in);
    switch (K) {
        case 2: block_pre_bwd_kernel<T, 2><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, gsi, part, s); break;
        case 3: block_pre_bwd_kernel<T, 3><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, gsi, part, s); break;
        case 4: block_pre_bwd_kernel<T, 4><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, gsi, part, s); break;
        default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    // the partials hold, per run block, [C][K+1] = (dw[0..K-1], db): sum the columns, then split them
    const int cols = C * (K + 1);
    float *sums = part + (size_t)run_blocks * cols;  // (behind the partials: cols floats)
    column_sums_kernel<<<dim3((cols + 255) / 256), dim3(256), 0, st>>>(part, (int)run_blocks, cols, sums);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    float *dt_part = sums + cols;
    const long long rows = (long long)s.B * s.L;
    const int dt_blocks = (int)std::min<long long>(kDtBlocks, rows);
    block_dt_bwd_kernel<T><<<dim3(dt_blocks), dim3(256), 0, st>>>(in, dt_bias, static_cast<const T *>(ddt), out, dt_part, s);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    column_sums_kernel<<<dim3((s.H + 255) / 256), dim3(256), 0, st>>>(dt_part, dt_blocks, s.H, ddt_bias);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    split_conv_sums_kernel<<<dim3((C + 255) / 256), dim3(256), 0, st>>>(sums, C, K, dconv_w, dconv_b);
    return hipGetLastError();
}

hipError_t launch_block_pre_bwd(const BlockShape &s, int dtype, const void *zxbcdt, const float *conv_w, const float *conv_b,
                                const float *dt_bias, const void *state_in, const unsigned char *reset, const void *dx,
                                const void *dB, const void *dC, const void *ddt, const void *dstate_out, void *dzxbcdt,
                                float *dconv_w, float *dconv_b, float *ddt_bias, void *dstate_in, void *workspace,
                                hipStream_t st) {
    // the post partials occupy the front of the workspace (the two stages of one backward pass share it: post runs
    // first and has added its partials up before pre starts on the same stream)
    float *part = static_cast<float *>(workspace);
    return dtype ? pre_bwd_dispatch<__bf16>(s, zxbcdt, conv_w, conv_b, dt_bias, state_in, reset, dx, dB, dC, ddt, dstate_out,
                                            dzxbcdt, dconv_w, dconv_b, ddt_bias, dstate_in, part, st)
                 : pre_bwd_dispatch<float>(s, zxbcdt, conv_w, conv_b, dt_bias, state_in, reset, dx, dB, dC, ddt, dstate_out,
                                           dzxbcdt, dconv_w, dconv_b, ddt_bias, dstate_in, part, st);
}

}  // namespace ssd
