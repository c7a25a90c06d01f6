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

constexpr int kBwdSteps = 32;    // timesteps per thread of the conv backward
constexpr int kBwdCh = 4;            // channels per thread of the conv backward (eight would take 290 registers)
constexpr int kPiecesPerBlock = 32;  // channel pieces (of kBwdCh) per workgroup of the conv backward
constexpr int kRunsPerBlock = 8;

template <typename T> struct PackCh;  // kBwdCh = four consecutive channels
template <> struct PackCh<__bf16> {
    uint2 u;
    __device__ inline float get(int i) const {
        const unsigned w = (&u.x)[i >> 1];
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    static __device__ inline PackCh load(const __bf16 *p) { return PackCh{*reinterpret_cast<const uint2 *>(p)}; }
    static __device__ inline void store(__bf16 *p, const float (&v)[4]) {
        *reinterpret_cast<uint2 *>(p) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
    }
};
template <> struct PackCh<float> {
    float4 a;
    __device__ inline float get(int i) const { return (&a.x)[i]; }
    static __device__ inline PackCh load(const float *p) { return PackCh{*reinterpret_cast<const float4 *>(p)}; }
    static __device__ inline void store(float *p, const float (&v)[4]) {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
constexpr int kPostBlocks = 1024;    // workgroups of post_bwd (each walks rows with a grid stride)

// ---- post ----------------------------------------------------------------------------------------------------
// LPR lanes per (b, t) row as in the forward, PPL pieces of 8 channels per lane; v = y silu(z),
// r = (mean v^2 + eps)^-1/2, g = dout w:
//   dv = r g - r^3 v mean(g v);  dy = dv silu(z);  dz = dv y silu'(z);  dw += dout v r
// No load is under a condition (a piece past the row's end reads the row's last piece and counts as zeros, a row past
// the tensor reads the last row and is not stored), and a lane's next row is requested before this row's arithmetic
// and stores: behind a conditional load the compiler waits for every earlier load and store.
// EXACT: the lanes' pieces cover the row exactly.  Whole passes of the workgroup's rows then store without a
// condition, so that the compiler can count the stores between a row's loads and their use instead of waiting for
// all of them (the last, partial pass of the tensor runs the guarded code).
template <typename T, typename TY, int LPR, int PPL, bool EXACT>
__global__ __launch_bounds__(256) void block_post_bwd_kernel(const TY *__restrict__ y, const T *__restrict__ zxbcdt,
                                                             const float *__restrict__ norm_w, float eps,
                                                             const T *__restrict__ dout, T *__restrict__ dy,
                                                             T *__restrict__ dzxbcdt, float *__restrict__ dw_part,
                                                             T *__restrict__ yn, BlockShape s) {
    const int DI = s.H * s.P;
    const int lane = threadIdx.x & (LPR - 1);
    constexpr int MAXP = PPL;
    constexpr int RPB = 256 / LPR;  // rows per workgroup and pass
    const long long rows = (long long)s.B * s.L;
    float wv[MAXP][8], dwacc[MAXP][8], in[MAXP];
    int cc[MAXP];  // the piece this lane reads for slot u (the row's last piece where the slot lies past the row)
#pragma unroll
    for (int u = 0; u < MAXP; ++u) {
        const int c0 = (u * LPR + lane) * 8;
        in[u] = c0 < DI ? 1.f : 0.f;
        cc[u] = min(c0, DI - 8);
        const float4 wa = *reinterpret_cast<const float4 *>(norm_w + cc[u]), wb = *reinterpret_cast<const float4 *>(norm_w + cc[u] + 4);
        const float wq[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            wv[u][i] = in[u] * wq[i];
            dwacc[u][i] = 0.f;
        }
    }
    struct RowIn {
        Pack8<TY> y[MAXP];
        Pack8<T> z[MAXP], d[MAXP];
    };
    auto fetch = [&](long long row) {
        RowIn o;
        const size_t r_ = (size_t)min(row, rows - 1);
#pragma unroll
        for (int u = 0; u < MAXP; ++u) {
            o.y[u] = Pack8<TY>::load(y + r_ * DI + cc[u]);
            o.z[u] = Pack8<T>::load(zxbcdt + r_ * s.ld + cc[u]);
            o.d[u] = Pack8<T>::load(dout + r_ * DI + cc[u]);
        }
        return o;
    };
    const float inv_di = 1.f / (float)DI;
    const float di = (float)DI;
    const long long stride = (long long)gridDim.x * RPB;
    RowIn cur = fetch((long long)blockIdx.x * RPB + threadIdx.x / LPR);
    auto pass = [&](long long row0, auto whole_tag) {
        constexpr bool WHOLE = decltype(whole_tag)::value;  // every row of the pass exists
        const long long row = row0 + threadIdx.x / LPR;
        const bool live = WHOLE || row < rows;  // (whole waves stay for the lane exchanges)
        float yy[MAXP][8], zz[MAXP][8], dd[MAXP][8];
#pragma unroll
        for (int u = 0; u < MAXP; ++u) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                yy[u][i] = EXACT ? cur.y[u].get(i) : in[u] * cur.y[u].get(i);
                zz[u][i] = cur.z[u].get(i);
                dd[u][i] = cur.d[u].get(i);
                // (the unpacked values exist from here on: left alone, the compiler unpacks where they are used, keeps
                // the packed registers alive until then and moves the next row's loads behind the arithmetic)
                asm volatile("" : "+v"(yy[u][i]), "+v"(zz[u][i]), "+v"(dd[u][i]));
            }
        }
        cur = fetch(row + stride);  // (after the values have been taken out: the loads go into the same registers)
        __builtin_amdgcn_sched_barrier(0);  // (and are not moved behind the arithmetic)
        float ss = 0.f, gv = 0.f;
#pragma unroll
        for (int u = 0; u < MAXP; ++u) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float v = yy[u][i] * silu(zz[u][i]);  // (zero in a slot past the row: y counts as zero there)
                ss += v * v;
                gv += dd[u][i] * wv[u][i] * v;
            }
        }
        ss = group_sum<LPR>(ss);
        gv = group_sum<LPR>(gv);
        const float r = rsqrtf(ss / di + eps);  // (the forward's expression: yn below is its output bit for bit)
        const float k3 = r * r * r * gv * inv_di;
#pragma unroll
        for (int u = 0; u < MAXP; ++u) {
            const int c0 = (u * LPR + lane) * 8;
            if ((EXACT || c0 < DI) && live) {
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
                if (yn != nullptr) {  // (uniform) the normalised row, for a forward that did not keep it
                    float on[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) on[i] = yy[u][i] * silu(zz[u][i]) * r * wv[u][i];
                    Pack8<T>::store(yn + (size_t)row * DI + c0, on);
                }
            }
        }
    };
    // (the first pass stands outside the loop: entered from code with no stores in flight, the loop's first wait would
    // be counted for that case and wait for the stores of the pass before on every later round)
    long long row0 = (long long)blockIdx.x * RPB;
    if (row0 + RPB <= rows) {
        pass(row0, std::true_type{});
        for (row0 += stride; row0 + RPB <= rows; row0 += stride) pass(row0, std::true_type{});
    }
    if (row0 < rows) pass(row0, std::false_type{});
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

// out[c] = sum over parts of part[p][c] (columns = channels), in a fixed order: a workgroup is 64 columns x 4 slices
// of its share of the parts (blockIdx.y of gridDim.y shares); a slice adds every fourth part of the share in order,
// the four slices are added in order, and the shares' sums [gridDim.y][cols] go through the same kernel once more.
constexpr int kSumShares = 32;
__global__ __launch_bounds__(256) void column_sums_kernel(const float *__restrict__ part, int nparts, int cols,
                                                          float *__restrict__ out) {
    __shared__ float sm[4][64];
    const int cl = threadIdx.x & 63, q = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + cl;
    const int per = (nparts + gridDim.y - 1) / gridDim.y;
    const int p0 = blockIdx.y * per, p1 = min(nparts, p0 + per);
    float acc = 0.f;
    if (c < cols) {
#pragma unroll 4
        for (int p = p0 + q; p < p1; p += 4) acc += part[(size_t)p * cols + c];
    }
    sm[q][cl] = acc;
    __syncthreads();
    if (q == 0 && c < cols) out[(size_t)blockIdx.y * cols + c] = ((sm[0][cl] + sm[1][cl]) + sm[2][cl]) + sm[3][cl];
}

// sums of nparts rows of `cols` floats into out[cols]; tmp holds kSumShares * cols floats
static hipError_t launch_column_sums(const float *part, int nparts, int cols, float *tmp, float *out, hipStream_t st) {
    const dim3 blocks((cols + 63) / 64, nparts >= 4 * kSumShares ? kSumShares : 1);
    if (blocks.y == 1) {
        column_sums_kernel<<<blocks, dim3(256), 0, st>>>(part, nparts, cols, out);
        return hipGetLastError();
    }
    column_sums_kernel<<<blocks, dim3(256), 0, st>>>(part, nparts, cols, tmp);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    column_sums_kernel<<<dim3(blocks.x, 1), dim3(256), 0, st>>>(tmp, kSumShares, cols, out);
    return hipGetLastError();
}

// ---- pre -----------------------------------------------------------------------------------------------------
// One thread per (run of kBwdSteps timesteps, kBwdCh channels of x | B | C).  pre[t] = b + sum_k w[k] in[t-(K-1)+k]
// (taps before the latest restart at or before t cut: the window's older rows are zeroed at a restart, as in the
// forward), out = silu(pre); with dpre[t] = dout[t] silu'(pre[t]):
//   din[s]  = sum_{q=0..K-1} w[K-1-q] dpre[s+q]      over the q whose output s+q exists and lies before any restart
//                                                     after s
//   dw[k]  += dpre[t] in[t-(K-1)+k],  db += dpre[t]
// The thread walks its run and K-1 timesteps beyond it once, with the last K input rows and the last K dpre rows in
// two rings of registers (the loop is unrolled by K, so ring positions are compile-time): dpre[t] is formed at step t
// and din[t-(K-1)] leaves at the same step.  A gradient on the returned conv state joins din of the last K-1
// timesteps; the gradient of the incoming conv state is block_pre_bwd_state_kernel's.
// Every load is unconditional (rows outside the sequence read a row inside it and count as zeros) and a step's rows
// are requested K steps before they are used, into the ring slot the step K before has just emptied: a conditional
// load is a branch at which the compiler waits for every earlier load and store, which made each step wait for the
// store of the step before.  RS: the call has a reset mask.
template <typename T, int K, bool RS>
__global__ __launch_bounds__(256) void block_pre_bwd_kernel(const T *__restrict__ zxbcdt, const float *__restrict__ conv_w,
                                                            const float *__restrict__ conv_b, const T *__restrict__ state_in,
                                                            const unsigned char *__restrict__ reset, const T *__restrict__ dx,
                                                            const T *__restrict__ dB, const T *__restrict__ dC,
                                                            const T *__restrict__ dstate_out, T *__restrict__ dzxbcdt,
                                                            float *__restrict__ part, BlockShape s) {
    const int DI = s.H * s.P, GN = s.G * s.N, C = DI + 2 * GN;
    const int CP = C / kBwdCh;
    const int runs = (s.L + kBwdSteps - 1) / kBwdSteps;
    const int pl = threadIdx.x % kPiecesPerBlock, rl = threadIdx.x / kPiecesPerBlock;
    // one linear grid, piece blocks fastest (the grid's second dimension stops at 65 535 run blocks)
    const unsigned piece_blocks = (CP + kPiecesPerBlock - 1) / kPiecesPerBlock;
    const unsigned run_block = blockIdx.x / piece_blocks;
    const int piece = (blockIdx.x % piece_blocks) * kPiecesPerBlock + pl;
    const long long br = (long long)run_block * kRunsPerBlock + rl;
    const bool active = piece < CP && br < (long long)s.B * runs;
    float dwacc[kBwdCh][K], dbacc[kBwdCh];
#pragma unroll
    for (int i = 0; i < kBwdCh; ++i) {
        dbacc[i] = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k) dwacc[i][k] = 0.f;
    }
    if (active) {
        const int t0 = (int)(br % runs) * kBwdSteps, b = (int)(br / runs);
        const int t1 = min(t0 + kBwdSteps, s.L);
        const int c0 = piece * kBwdCh;
        const T *row0 = zxbcdt + ((size_t)b * s.L) * s.ld + DI + c0;
        const unsigned char *rs = RS ? reset + (size_t)b * s.L : nullptr;
        static_assert(kBwdCh == 4, "a thread's taps are K float4, its biases one");
        float w[kBwdCh][K], bias[kBwdCh];
        {
            float wf[kBwdCh * K];
#pragma unroll
            for (int q = 0; q < K; ++q) {
                const float4 v = *reinterpret_cast<const float4 *>(conv_w + (size_t)c0 * K + 4 * q);
                wf[4 * q] = v.x; wf[4 * q + 1] = v.y; wf[4 * q + 2] = v.z; wf[4 * q + 3] = v.w;
            }
            const float4 bq = *reinterpret_cast<const float4 *>(conv_b + c0);
            bias[0] = bq.x; bias[1] = bq.y; bias[2] = bq.z; bias[3] = bq.w;
#pragma unroll
            for (int i = 0; i < kBwdCh; ++i) {
#pragma unroll
                for (int k = 0; k < K; ++k) w[i][k] = wf[i * K + k];
            }
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
        // what step j (timestep t0 + j) reads: its input row, its gradient row, its restart flag
        struct StepIn {
            PackCh<T> p, g;
            unsigned char r;
        };
        auto fetch = [&](int j) {
            StepIn o;
            const int tc = min(t0 + j, s.L - 1);
            o.p = PackCh<T>::load(row0 + (size_t)tc * s.ld);
            o.g = PackCh<T>::load(gsrc + (size_t)tc * gstride);
            o.r = RS ? rs[tc] : (unsigned char)0;
            return o;
        };
        // the K-1 input rows before the run (history before 0 from the conv state, zero without one) and the restart
        // flags of the K-2 timesteps before it
        PackCh<T> hist[K - 1];
#pragma unroll
        for (int m = 1; m <= K - 1; ++m) {
            const int ts = t0 - m;
            const T *own = row0 + (size_t)max(ts, 0) * s.ld;
            const T *old = state_in != nullptr ? state_in + ((size_t)b * (K - 1) + max(K - 1 + ts, 0)) * C + c0 : own;
            hist[m - 1] = PackCh<T>::load(ts >= 0 ? own : old);
        }
        unsigned char rb[K > 2 ? K - 2 : 1] = {};
        if constexpr (RS) {
#pragma unroll
            for (int back = 1; back <= K - 2; ++back) rb[back - 1] = rs[max(t0 - back, 0)];
        }
        StepIn cur[K];
#pragma unroll
        for (int u = 0; u < K; ++u) cur[u] = fetch(u);
        // rings: step j (timestep t0 + j) uses position j % K; position of step j - m is (j - m) mod K
        float win[K][kBwdCh], dq[K][kBwdCh];
        bool fl[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            fl[k] = false;
#pragma unroll
            for (int i = 0; i < kBwdCh; ++i) dq[k][i] = 0.f;
        }
#pragma unroll
        for (int m = 1; m <= K - 1; ++m) {
            const bool have = t0 - m >= 0 || state_in != nullptr;
#pragma unroll
            for (int i = 0; i < kBwdCh; ++i) win[K - m][i] = have ? hist[m - 1].get(i) : 0.f;
        }
        if constexpr (RS) {
            // a restart at one of the K-2 timesteps before the run cuts the rows before it
#pragma unroll
            for (int back = 1; back <= K - 2; ++back) {
                if (t0 - back >= 0 && rb[back - 1] != 0) {
#pragma unroll
                    for (int m = back + 1; m <= K - 1; ++m) {
#pragma unroll
                        for (int i = 0; i < kBwdCh; ++i) win[K - m][i] = 0.f;
                    }
                }
            }
        }
        T *drow = dzxbcdt + ((size_t)b * s.L) * s.ld + DI + c0;
        constexpr int NT = kBwdSteps + K - 1;
#pragma unroll 1
        for (int jb = 0; jb < NT; jb += K) {
#pragma unroll
            for (int u = 0; u < K; ++u) {  // ring position of this step: u
                const int t = t0 + jb + u;
                const bool exists = t < s.L && jb + u < NT;
                const bool r = RS && exists && cur[u].r != 0;
                if (r) {  // the rows before a restart do not reach it
#pragma unroll
                    for (int m = 1; m <= K - 1; ++m) {
#pragma unroll
                        for (int i = 0; i < kBwdCh; ++i) win[(u + K - m) % K][i] = 0.f;
                    }
                }
                float gin[kBwdCh];
#pragma unroll
                for (int i = 0; i < kBwdCh; ++i) {
                    win[u][i] = exists ? cur[u].p.get(i) : 0.f;
                    gin[i] = exists ? cur[u].g.get(i) : 0.f;
                }
                // (after the slot's values have been taken out, so that the load can go into the same registers: a
                // copy at the loop's end would have to wait for it)
                cur[u] = fetch(jb + u + K);
                const bool own = exists && t < t1;  // this thread's own timesteps: the parameter gradients
#pragma unroll
                for (int i = 0; i < kBwdCh; ++i) {
                    float a = bias[i];
#pragma unroll
                    for (int k = 0; k < K; ++k) a += w[i][k] * win[(u + k + 1) % K][i];
                    const float d = gin[i] * dsilu(a);  // (gin is zero past the sequence)
                    dq[u][i] = d;
                    const float dm = own ? d : 0.f;
                    dbacc[i] += dm;
#pragma unroll
                    for (int k = 0; k < K; ++k) dwacc[i][k] += dm * win[(u + k + 1) % K][i];
                }
                fl[u] = r;
                // din of timestep sidx = t - (K-1): outputs sidx .. t while no restart lies after sidx
                const int sidx = t - (K - 1);
                if (jb + u >= K - 1 && sidx < t1) {
                    float o[kBwdCh];
#pragma unroll
                    for (int i = 0; i < kBwdCh; ++i) o[i] = w[i][K - 1] * dq[(u + 1) % K][i];
                    bool open = true;
#pragma unroll
                    for (int q = 1; q < K; ++q) {
                        open = open && !fl[(u + 1 + q) % K];
                        if (open) {
#pragma unroll
                            for (int i = 0; i < kBwdCh; ++i) o[i] += w[i][K - 1 - q] * dq[(u + 1 + q) % K][i];
                        }
                    }
                    // a gradient on the conv state the forward returned: that state is the last K-1 input rows,
                    // those before the window's last restart zeroed
                    if (dstate_out != nullptr && sidx >= s.L - (K - 1)) {
                        bool kept = true;
                        for (int tt = sidx + 1; tt < s.L; ++tt) kept = kept && !(RS && rs[tt] != 0);
                        if (kept) {
                            const PackCh<T> p = PackCh<T>::load(dstate_out + ((size_t)b * (K - 1) + (sidx - (s.L - (K - 1)))) * C + c0);
#pragma unroll
                            for (int i = 0; i < kBwdCh; ++i) o[i] += p.get(i);
                        }
                    }
                    PackCh<T>::store(drow + (size_t)sidx * s.ld, o);
                }
            }
        }
    }
    // the workgroup's partial sums: per channel piece, its kRunsPerBlock threads added in order
    __shared__ float red[256 * (K + 1)];
    const int cols = C * (K + 1);
#pragma unroll
    for (int i = 0; i < kBwdCh; ++i) {
        __syncthreads();
#pragma unroll
        for (int k = 0; k < K; ++k) red[threadIdx.x * (K + 1) + k] = dwacc[i][k];
        red[threadIdx.x * (K + 1) + K] = dbacc[i];
        __syncthreads();
        if (rl == 0 && piece < CP) {
            const int c = piece * kBwdCh + i;
#pragma unroll
            for (int k = 0; k <= K; ++k) {
                float acc = 0.f;
                for (int q = 0; q < kRunsPerBlock; ++q) acc += red[(q * kPiecesPerBlock + pl) * (K + 1) + k];
                part[(size_t)run_block * cols + (size_t)c * (K + 1) + k] = acc;
            }
        }
    }
}

// The gradient of the incoming conv state: one thread per (batch row, 8 channels).  The inputs at s = -(K-1) .. -1
// reach outputs 0 .. s+K-1, up to the first restart; the thread recomputes dpre of those K-1 outputs.
template <typename T, int K>
__global__ __launch_bounds__(256) void block_pre_bwd_state_kernel(const T *__restrict__ zxbcdt, const float *__restrict__ conv_w,
                                                                  const float *__restrict__ conv_b, const T *__restrict__ state_in,
                                                                  const unsigned char *__restrict__ reset, const T *__restrict__ dx,
                                                                  const T *__restrict__ dB, const T *__restrict__ dC,
                                                                  const T *__restrict__ dstate_out, T *__restrict__ dstate_in,
                                                                  BlockShape s) {
    const int DI = s.H * s.P, GN = s.G * s.N, C = DI + 2 * GN, CP = C / 8;
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (long long)s.B * CP) return;
    const int piece = (int)(gid % CP), b = (int)(gid / CP), c0 = piece * 8;
    const T *row0 = zxbcdt + ((size_t)b * s.L) * s.ld + DI + c0;
    const unsigned char *rs = reset ? reset + (size_t)b * s.L : nullptr;
    float w[8][K], bias[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        bias[i] = conv_b[c0 + i];
#pragma unroll
        for (int k = 0; k < K; ++k) w[i][k] = conv_w[(size_t)(c0 + i) * K + k];
    }
    const T *gsrc = c0 < DI ? dx + ((size_t)b * s.L) * DI + c0
                            : c0 < DI + GN ? dB + ((size_t)b * s.L) * GN + (c0 - DI) : dC + ((size_t)b * s.L) * GN + (c0 - DI - GN);
    const int gstride = c0 < DI ? DI : GN;
    // dpre of outputs 0 .. K-2; `open` = no restart at 0 .. t (a restart at t cuts the state off output t as well)
    float acc[K - 1][8];
#pragma unroll
    for (int jr = 0; jr < K - 1; ++jr) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[jr][i] = 0.f;
    }
    bool open = true;
#pragma unroll
    for (int t = 0; t < K - 1; ++t) {
        if (t < s.L) {
            if (rs != nullptr && rs[t] != 0) open = false;
            if (open) {  // no restart so far: the window is the state's rows and inputs 0 .. t, none zeroed
                float a[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) a[i] = bias[i];
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    const int ts = t - (K - 1) + k;
                    if (ts >= 0) {
                        const Pack8<T> p = Pack8<T>::load(row0 + (size_t)ts * s.ld);
#pragma unroll
                        for (int i = 0; i < 8; ++i) a[i] += w[i][k] * p.get(i);
                    } else if (state_in != nullptr) {
                        const Pack8<T> p = Pack8<T>::load(state_in + ((size_t)b * (K - 1) + (K - 1 + ts)) * C + c0);
#pragma unroll
                        for (int i = 0; i < 8; ++i) a[i] += w[i][k] * p.get(i);
                    }
                }
                const Pack8<T> g = Pack8<T>::load(gsrc + (size_t)t * gstride);
#pragma unroll
                for (int jr = 0; jr < K - 1; ++jr) {
                    const int k = jr - t;  // tap of input s = jr - (K-1) in output t
                    if (k >= 0) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) acc[jr][i] += w[i][k] * (g.get(i) * dsilu(a[i]));
                    }
                }
            }
        }
    }
#pragma unroll
    for (int jr = 0; jr < K - 1; ++jr) {
        const int sidx = jr - (K - 1);
        // rows of the old state that are still part of the new one (fewer than K-1 new timesteps)
        if (dstate_out != nullptr && sidx >= s.L - (K - 1)) {
            bool kept = true;
            for (int t = 0; t < s.L; ++t) kept = kept && !(rs != nullptr && rs[t] != 0);
            if (kept) {
                const Pack8<T> p = Pack8<T>::load(dstate_out + ((size_t)b * (K - 1) + (sidx - (s.L - (K - 1)))) * C + c0);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[jr][i] += p.get(i);
            }
        }
        Pack8<T>::store(dstate_in + ((size_t)b * (K - 1) + jr) * C + c0, acc[jr]);
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
            // four rows per round, their loads requested together and without a condition (a row past the tensor
            // reads the last row and is not stored): one trip to memory per round instead of one per row
            constexpr int kRound = 4;
            const long long stride = (long long)gridDim.x * slots;
            for (long long row0 = (long long)blockIdx.x * slots + slot; row0 < rows; row0 += kRound * stride) {
                T raw_q[kRound], ddt_q[kRound];
#pragma unroll
                for (int u = 0; u < kRound; ++u) {
                    const size_t row = (size_t)min(row0 + u * stride, rows - 1);
                    raw_q[u] = zxbcdt[row * s.ld + off + h];
                    ddt_q[u] = ddt[row * s.H + h];
                }
#pragma unroll
                for (int u = 0; u < kRound; ++u) {
                    const long long row = row0 + u * stride;
                    const float g = (float)ddt_q[u] * sigmoidf((float)raw_q[u] + bias);
                    if (row < rows) {
                        dzxbcdt[(size_t)row * s.ld + off + h] = (T)g;
                        acc += g;
                    }
                }
            }
        }
        __syncthreads();
        red[threadIdx.x] = acc;
        __syncthreads();
        if ((int)threadIdx.x < hpt) {
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
    const size_t post = (size_t)(kPostBlocks + kSumShares) * DI;
    const size_t pre = (run_blocks + 1 + kSumShares) * C * (s.d_conv + 1) + (size_t)(kDtBlocks + kSumShares) * s.H;
    return sizeof(float) * (post > pre ? post : pre);  // the two stages run one after the other and share it
}

template <typename T, typename TY>
static hipError_t post_bwd_dispatch(const BlockShape &s, const void *y, const void *zxbcdt, const float *norm_w, float eps,
                                    const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, float *part, void *yn,
                                    hipStream_t st) {
    const int DI = s.H * s.P, pieces = DI / 8;
    const long long rows = (long long)s.B * s.L;
    const TY *yy = static_cast<const TY *>(y);
    const T *zz = static_cast<const T *>(zxbcdt), *dd = static_cast<const T *>(dout);
    T *oy = static_cast<T *>(dy), *oz = static_cast<T *>(dzxbcdt), *on = static_cast<T *>(yn);
    // lanes per row and pieces per lane as in the forward
    const int lpr = pieces <= 16 * 4 ? 16 : pieces <= 32 * 4 ? 32 : 64;
    const int ppl = (pieces + lpr - 1) / lpr;
    const int blocks = (int)std::min<long long>(kPostBlocks, (rows + 256 / lpr - 1) / (256 / lpr));
    bool launched = false;
#define SSD_POST_BWD_CASE(LPRv, PPLv)                                                                                       \
    if (lpr == LPRv && ppl == PPLv) {                                                                                       \
        if (pieces == LPRv * PPLv)                                                                                          \
            block_post_bwd_kernel<T, TY, LPRv, PPLv, true><<<dim3(blocks), dim3(256), 0, st>>>(yy, zz, norm_w, eps, dd, oy, oz, part, on, s); \
        else                                                                                                                \
            block_post_bwd_kernel<T, TY, LPRv, PPLv, false><<<dim3(blocks), dim3(256), 0, st>>>(yy, zz, norm_w, eps, dd, oy, oz, part, on, s); \
        launched = true;                                                                                                    \
    }
    SSD_POST_BWD_CASE(16, 1) SSD_POST_BWD_CASE(16, 2) SSD_POST_BWD_CASE(16, 3) SSD_POST_BWD_CASE(16, 4)
    SSD_POST_BWD_CASE(32, 3) SSD_POST_BWD_CASE(32, 4)
    SSD_POST_BWD_CASE(64, 3) SSD_POST_BWD_CASE(64, 4)
#undef SSD_POST_BWD_CASE
    if (!launched) return hipErrorInvalidValue;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_column_sums(part, blocks, DI, part + (size_t)kPostBlocks * DI, dnorm_w, st);
}

hipError_t launch_block_post_bwd(const BlockShape &s, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                                 float eps, const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, void *workspace,
                                 hipStream_t st, void *yn) {
    float *part = static_cast<float *>(workspace);
    switch (dtype) {
        case 0: return post_bwd_dispatch<float, float>(s, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, part, yn, st);
        case 1: return post_bwd_dispatch<__bf16, __bf16>(s, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, part, yn, st);
        default: return post_bwd_dispatch<__bf16, float>(s, y, zxbcdt, norm_w, eps, dout, dy, dzxbcdt, dnorm_w, part, yn, st);
    }
}

template <typename T>
static hipError_t pre_bwd_dispatch(const BlockShape &s, const void *zxbcdt, const float *conv_w, const float *conv_b,
                                   const float *dt_bias, const void *state_in, const unsigned char *reset, const void *dx,
                                   const void *dB, const void *dC, const void *ddt, const void *dstate_out, void *dzxbcdt,
                                   float *dconv_w, float *dconv_b, float *ddt_bias, void *dstate_in, float *part,
                                   hipStream_t st) {
    const int DI = s.H * s.P, C = DI + 2 * s.G * s.N, CP = C / kBwdCh, K = s.d_conv;
    const long long runs = (s.L + kBwdSteps - 1) / kBwdSteps;
    const long long run_blocks = ((long long)s.B * runs + kRunsPerBlock - 1) / kRunsPerBlock;
    const long long piece_blocks = (CP + kPiecesPerBlock - 1) / kPiecesPerBlock;
    if (run_blocks * piece_blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(run_blocks * piece_blocks));
    const T *in = static_cast<const T *>(zxbcdt), *si = static_cast<const T *>(state_in);
    const T *gx = static_cast<const T *>(dx), *gb = static_cast<const T *>(dB), *gc = static_cast<const T *>(dC);
    const T *gso = static_cast<const T *>(dstate_out);
    T *out = static_cast<T *>(dzxbcdt), *gsi = static_cast<T *>(dstate_in);
    const dim3 sgrid((unsigned)(((long long)s.B * (C / 8) + 255) / 256));
    switch (K) {
        case 2:
            if (reset != nullptr)
                block_pre_bwd_kernel<T, 2, true><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, part, s);
            else
                block_pre_bwd_kernel<T, 2, false><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, part, s);
            if (gsi) block_pre_bwd_state_kernel<T, 2><<<sgrid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, gsi, s);
            break;
        case 3:
            if (reset != nullptr)
                block_pre_bwd_kernel<T, 3, true><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, part, s);
            else
                block_pre_bwd_kernel<T, 3, false><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, part, s);
            if (gsi) block_pre_bwd_state_kernel<T, 3><<<sgrid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, gsi, s);
            break;
        case 4:
            if (reset != nullptr)
                block_pre_bwd_kernel<T, 4, true><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, part, s);
            else
                block_pre_bwd_kernel<T, 4, false><<<grid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, out, part, s);
            if (gsi) block_pre_bwd_state_kernel<T, 4><<<sgrid, dim3(256), 0, st>>>(in, conv_w, conv_b, si, reset, gx, gb, gc, gso, gsi, s);
            break;
        default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    // the partials hold, per run block, [C][K+1] = (dw[0..K-1], db): sum the columns, then split them
    const int cols = C * (K + 1);
    float *sums = part + (size_t)run_blocks * cols;  // (behind the partials: cols floats, then the shares' sums)
    float *tmp = sums + cols;
    if ((e = launch_column_sums(part, (int)run_blocks, cols, tmp, sums, st)) != hipSuccess) return e;
    float *dt_part = tmp + (size_t)kSumShares * cols;
    const long long rows = (long long)s.B * s.L;
    const int dt_blocks = (int)std::min<long long>(kDtBlocks, rows);
    block_dt_bwd_kernel<T><<<dim3(dt_blocks), dim3(256), 0, st>>>(in, dt_bias, static_cast<const T *>(ddt), out, dt_part, s);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    if ((e = launch_column_sums(dt_part, dt_blocks, s.H, dt_part + (size_t)kDtBlocks * s.H, ddt_bias, st)) != hipSuccess) return e;
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
