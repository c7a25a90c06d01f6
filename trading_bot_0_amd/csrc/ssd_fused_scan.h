// The whole SSD forward in one pass over the inputs (gfx950, bf16 inputs).
//
// A wave owns one "unit": 32 head-dim columns of one head of one batch row, for the whole
// sequence.  It walks the chunks in order and keeps the running state H^T [N x 32] of its unit
// in MFMA accumulators, so neither per-chunk states nor the cumulative-decay rows ever go to
// HBM: x, dt, B, C are read once and y (plus the final state) is written once.  The WAVES
// waves of a workgroup are consecutive units of one (batch, group); they share the chunk's B
// and C tiles in LDS and load them, and their own x tiles, together, in full-row pieces.
//
// Per chunk a wave does, for its unit,
//   scan     alpha[l] = log2(e) * cumsum(dt*A) in float64 across the wave (DPP), split hi + lo;
//            decay tables in its private LDS rows (see below)
//   phase 1  for each block of 32 output columns l (lb = 0 .. Q/32-1), yT[p,l] =
//              E[l] * ( exp2(alpha[32 lb]) * (H . C^T)                     state readout
//                       + sum_{s-blocks sb <= lb} xT . (B.C^T o F_lb) )    intra-chunk
//            with E[l] = exp2(alpha[l] - alpha[32 lb]) and F_lb[s] = exp2(alpha[32 lb] - alpha[s]) dt[s];
//            + D x in the epilogue.  The state is the A operand straight from its accumulator
//            registers (hi + lo bf16), in the register order of the accumulator, which fixes the
//            K order in which C and B are read (n0..n0+3, n0+8..n0+11 per lane).
//   phase 2  H^T <- exp2(alpha[Q-1]) H^T + B^T . (w o x),  w[l] = exp2(alpha[Q-1] - alpha[l]) dt[l];
//            x is weighted in registers after the transposing LDS read.
//
// Decay factors are separable through the first row of the column block, so a score element
// costs one multiply.  That also holds on the diagonal block (with the causal mask) as long as
// the block's total log2-decay stays below 120: then neither factor leaves the float range and
// E[l] F[s] is exp2(alpha[l]-alpha[s]) dt[s] to rounding.  A block that decays more takes the
// exact path: one exp2 of the hi/lo difference per element.  The choice is uniform per wave.
//
// Everything this kernel manufactures in fp32 and feeds to an MFMA (masked decayed scores, the
// state, weighted x) goes in as a hi + lo pair of bf16; x, B and C enter exactly as given.
//
// LDS tiles are row-major with their 8-byte pieces XOR-swizzled (ChunkTile) so that all three
// read patterns used here are free of bank conflicts: the transposing read (4 rows x 64 bytes
// per 32 lanes), 8 bytes of each of 32 consecutive rows, and the staging writes.
#pragma once
#include "ssd_device.h"

namespace ssd {

template <int COLS> struct ChunkTile {  // bf16 [rows][COLS], COLS = 32 or 64
    static_assert(COLS == 32 || COLS == 64, "tile rows are 64 or 128 bytes");
    // XOR mask on the index of an 8-byte piece within its row.  32 consecutive rows map a fixed logical
    // piece to 32 different bank pairs, and 4 consecutive rows (first one a multiple of 4) keep their
    // 64-byte halves in different quarters of the banks.
    static __device__ inline int f(int row) {
        if constexpr (COLS == 32) {
            return (row >> 2) & 7;
        } else {
            const int v = (row >> 1) & 15;
            return ((v & 1) << 3) | (v >> 1);
        }
    }
    static __device__ inline int off(int row, int col) {
        return row * COLS + ((((col >> 2) ^ f(row)) << 2) | (col & 3));
    }
    // 8 consecutive elements of a row (col a multiple of 8), as they come from a 16-byte global load
    static __device__ inline void put16(__bf16 *tile, int row, int col, const uint4 &v) {
        *reinterpret_cast<uint2 *>(tile + off(row, col)) = make_uint2(v.x, v.y);
        *reinterpret_cast<uint2 *>(tile + off(row, col + 4)) = make_uint2(v.z, v.w);
    }
    static __device__ inline bf16x4 row4(const __bf16 *tile, int row, int col) {
        return *reinterpret_cast<const bf16x4 *>(tile + off(row, col));
    }
    // this lane's 4 elements tile[k0 + 0..3][c0 + lane%32] (k0 a multiple of 4 that already includes
    // the lane half's K offset): K-consecutive data for operand row/column c0 + lane%32
    static __device__ inline bf16x4 tr4(const __bf16 *tile, int k0, int c0, int lane) {
        const int q = lane >> 4, a = (lane >> 2) & 3, b = lane & 3;
        const __bf16 *src = tile + off(k0 + a, c0 + 16 * (q & 1) + 4 * b);
        const bf16x4_gcc v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((SSD_LDS_AS bf16x4_gcc *)(src));
        return __builtin_bit_cast(bf16x4, v);
    }
    static __device__ inline Frag<__bf16> frag(const __bf16 *tile, int k0, int gap, int c0, int lane) {
        Frag<__bf16> fr;
        const bf16x4 lo = tr4(tile, k0, c0, lane), hi = tr4(tile, k0 + gap, c0, lane);
        fr.v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return fr;
    }
    // elements col0..col0+3 and col0+8..col0+11 of one row: the K order of an accumulator reused as operand
    static __device__ inline Frag<__bf16> split_frag(const __bf16 *tile, int row, int col0) {
        Frag<__bf16> fr;
        const bf16x4 lo = row4(tile, row, col0), hi = row4(tile, row, col0 + 8);
        fr.v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return fr;
    }
};

__device__ inline float readlane_f(float v, int src_lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}

constexpr float kFastDiagSpan = 120.f;  // log2-decay across a diagonal block up to which E*F is safe

// Dynamic LDS of one workgroup: B and C tiles, one x tile per wave, (5 + Q/32) float rows and 16 block
// scalars per wave.
constexpr size_t fused_scan_lds_bytes(int N, int Q, int waves) {
    return (size_t)2 * Q * N * 2 + (size_t)waves * ((size_t)Q * 32 * 2 + (size_t)(5 + Q / 32) * Q * 4 + 64);
}

template <typename TO, int NK, int QB, int WAVES, bool EARLY>  // N = 16*NK, Q = 32*QB
__global__ __launch_bounds__(64 * WAVES, WAVES == 8 ? 1 : 2) void fused_scan_kernel(
    const __bf16 *__restrict__ x, const __bf16 *__restrict__ dt, const float *__restrict__ A,
    const __bf16 *__restrict__ Bm, const __bf16 *__restrict__ Cm, const float *__restrict__ D,
    const float *init, TO *__restrict__ y, float *final_states, ScanShape s) {
    using T = __bf16;
    constexpr int N = 16 * NK, NB = NK / 2, Q = 32 * QB, nthr = 64 * WAVES;
    constexpr int EPL = Q >= 64 ? Q / 64 : 1;  // chunk positions per lane in the scan
    constexpr int BSL = Q * N / 8;             // 16-byte pieces of a B (or C) tile
    constexpr int UBC = (BSL + nthr - 1) / nthr;
    constexpr int XPR = WAVES * 4;             // 16-byte pieces of one timestep's x for the workgroup
    constexpr int UX = Q * XPR / nthr;         // = Q / 16
    using XT = ChunkTile<32>;
    using BT = ChunkTile<N>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T *Bs = reinterpret_cast<T *>(smem);  // [Q][N]
    T *Cs = Bs + Q * N;                   // [Q][N]
    T *xs_all = Cs + Q * N;               // [WAVES][Q][32]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, half = lane >> 5;
    T *xs = xs_all + wave * (Q * 32);
    float *wf = reinterpret_cast<float *>(xs_all + WAVES * Q * 32) + wave * ((5 + QB) * Q + 16);
    float *ah_s = wf, *alo_s = wf + Q, *dt_s = wf + 2 * Q, *w_s = wf + 3 * Q, *E_s = wf + 4 * Q, *F_s = wf + 5 * Q;
    float *blk_s = wf + (5 + QB) * Q;  // [0..QB): exp2(alpha[32 lb]); [8..8+QB): log2-decay across block lb

    // ---- which units this workgroup owns ----
    const int PBn = s.P / 32, HG = s.H / s.G;
    const int UW = (HG * PBn) / WAVES;  // workgroups per (batch, group)
    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int b = logical / (s.G * UW);
    const int g = (logical / UW) % s.G;
    const int unit0 = (logical % UW) * WAVES;
    const int unit = unit0 + wave;
    const int h = g * HG + unit / PBn, pb = unit % PBn;
    const int xcol0 = g * HG * s.P + unit0 * 32;  // first element of the workgroup's slice of an x row
    const int HP = s.H * s.P;
    const T *xb = x + (size_t)b * s.L * HP + xcol0;
    const T *Bb = Bm + ((size_t)b * s.L * s.G + g) * N;
    const T *Cb = Cm + ((size_t)b * s.L * s.G + g) * N;
    const T *dtb = dt + (size_t)b * s.L * s.H + h;
    TO *yb = y + (size_t)b * s.L * HP + h * s.P + pb * 32;
    const float dh = D ? D[h] : 0.f;
    const double a_h = (double)A[h];

    // ---- registers holding the next chunk's inputs ----
    // A thread's pieces sit at fixed 32-bit element offsets from the chunk's first row.
    const int bc_row0 = tid / (N / 8), bc_off0 = bc_row0 * s.G * N + (tid % (N / 8)) * 8;
    const int bc_step = (nthr / (N / 8)) * s.G * N, bc_rstep = nthr / (N / 8);
    const int x_row0 = tid / XPR, x_off0 = x_row0 * HP + (tid % XPR) * 8, x_step = (nthr / XPR) * HP;
    const int dt_off0 = lane * EPL * s.H;
    uint4 bq[UBC], cq[UBC], xq[UX];
    unsigned short dq[EPL];
    auto prefetch = [&](int c) {
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        const T *bp = Bb + (size_t)t0 * s.G * N, *cp = Cb + (size_t)t0 * s.G * N;
        const T *xp = xb + (size_t)t0 * HP, *dp = dtb + (size_t)t0 * s.H;
        // (a conditional expression over *ptr and a zero constant would become a load through a selected
        // pointer, with the constant in scratch memory)
        auto ld16 = [](const T *ptr, bool ok) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ok) v = *reinterpret_cast<const uint4 *>(ptr);
            return v;
        };
        if (rows == Q) {
#pragma unroll
            for (int u = 0; u < UBC; ++u) {
                const bool ok = BSL % nthr == 0 || tid + u * nthr < BSL;
                bq[u] = ld16(bp + bc_off0 + u * bc_step, ok);
                cq[u] = ld16(cp + bc_off0 + u * bc_step, ok);
            }
#pragma unroll
            for (int u = 0; u < UX; ++u) xq[u] = *reinterpret_cast<const uint4 *>(xp + x_off0 + u * x_step);
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                dq[e] = (Q >= 64 || lane < Q) ? __builtin_bit_cast(unsigned short, dp[dt_off0 + e * s.H]) : (unsigned short)0;
        } else {  // ragged last chunk: rows past the sequence read as zero (dt = 0 makes them no-ops)
#pragma unroll
            for (int u = 0; u < UBC; ++u) {
                const bool ok = (BSL % nthr == 0 || tid + u * nthr < BSL) && bc_row0 + u * bc_rstep < rows;
                bq[u] = ld16(bp + bc_off0 + u * bc_step, ok);
                cq[u] = ld16(cp + bc_off0 + u * bc_step, ok);
            }
#pragma unroll
            for (int u = 0; u < UX; ++u)
                xq[u] = ld16(xp + x_off0 + u * x_step, x_row0 + u * (nthr / XPR) < rows);
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                dq[e] = (lane * EPL + e < rows) ? __builtin_bit_cast(unsigned short, dp[dt_off0 + e * s.H]) : (unsigned short)0;
        }
    };

    // ---- running state of this unit: st[nb][v] = H[p = r, n = 32 nb + 8 (v/4) + 4 half + v%4] ----
    f32x16 st[NB];
    {
        const float *ib = init ? init + (((size_t)b * s.H + h) * s.P + pb * 32 + r) * N + 4 * half : nullptr;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const float4 v = ib ? *reinterpret_cast<const float4 *>(ib + 32 * nb + 8 * gq) : make_float4(0, 0, 0, 0);
                st[nb][4 * gq + 0] = v.x;
                st[nb][4 * gq + 1] = v.y;
                st[nb][4 * gq + 2] = v.z;
                st[nb][4 * gq + 3] = v.w;
            }
        }
    }

    prefetch(0);
    for (int c = 0; c < s.nc; ++c) {
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        block_sync_lds();  // every wave is done reading the previous chunk's tiles
        // ---- registers -> LDS tiles ----
#pragma unroll
        for (int u = 0; u < UBC; ++u) {
            const int idx = tid + u * nthr;
            if (BSL % nthr == 0 || idx < BSL) {
                const int row = idx / (N / 8), ch = idx % (N / 8);
                BT::put16(Bs, row, ch * 8, bq[u]);
                BT::put16(Cs, row, ch * 8, cq[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            const int idx = tid + u * nthr;
            const int row = idx / XPR, piece = idx % XPR;
            XT::put16(xs_all + (piece / 4) * (Q * 32), row, (piece % 4) * 8, xq[u]);
        }
        // ---- scan of dt*A over the chunk and the decay tables of this unit ----
        float a_end;       // exp2(alpha[Q-1]): the chunk's total decay
        {
            constexpr double kLog2e = 1.4426950408889634;
            float dtv[EPL], hi[EPL], lo[EPL];
            double cs[EPL], run = 0.0;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                dtv[e] = (float)__builtin_bit_cast(__bf16, dq[e]);
                run += (double)dtv[e] * a_h;
                cs[e] = run;
            }
            const double excl = wave_inclusive_scan(run) - run;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const double al = (cs[e] + excl) * kLog2e;
                hi[e] = (float)al;
                lo[e] = (float)(al - (double)hi[e]);
            }
            float refh[QB], refl[QB], endh[QB], endl[QB];  // alpha at the first / last row of each block
#pragma unroll
            for (int lb = 0; lb < QB; ++lb) {
                refh[lb] = readlane_f(hi[0], (32 * lb) / EPL);
                refl[lb] = readlane_f(lo[0], (32 * lb) / EPL);
                endh[lb] = readlane_f(hi[EPL - 1], (32 * lb + 31) / EPL);
                endl[lb] = readlane_f(lo[EPL - 1], (32 * lb + 31) / EPL);
                if (lane == 0) {
                    blk_s[lb] = exp2_hw(refh[lb] + refl[lb]);
                    blk_s[8 + lb] = fmaxf(alpha_diff(refh[lb], refl[lb], endh[lb], endl[lb]), 0.f);
                }
            }
            a_end = exp2_hw(endh[QB - 1] + endl[QB - 1]);
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int l = lane * EPL + e;
                if (Q >= 64 || l < Q) {
                    const int blk = l >> 5;
                    ah_s[l] = hi[e];
                    alo_s[l] = lo[e];
                    dt_s[l] = dtv[e];
                    w_s[l] = exp2_hw(fminf(alpha_diff(endh[QB - 1], endl[QB - 1], hi[e], lo[e]), 0.f)) * dtv[e];
                    float rh = refh[0], rl = refl[0];
#pragma unroll
                    for (int lb = 1; lb < QB; ++lb) {
                        rh = (blk >= lb) ? refh[lb] : rh;
                        rl = (blk >= lb) ? refl[lb] : rl;
                    }
                    E_s[l] = exp2_hw(fminf(alpha_diff(hi[e], lo[e], rh, rl), 0.f));
#pragma unroll
                    for (int lb = 0; lb < QB; ++lb)
                        if (lb >= blk)
                            F_s[lb * Q + l] = exp2_hw(fminf(alpha_diff(refh[lb], refl[lb], hi[e], lo[e]), 126.f)) * dtv[e];
                }
            }
        }
        if (EARLY && c + 1 < s.nc) prefetch(c + 1);
        block_sync_lds();  // tiles and tables are visible

        // ---- phase 1: outputs of this chunk from the state entering it ----
        {
            Frag<T> Hhi[NK], Hlo[NK];
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    T vh, vl;
                    Split<T>::split(st[kk / 2][8 * (kk % 2) + i], vh, vl);
                    Hhi[kk].v[i] = vh;
                    Hlo[kk].v[i] = vl;
                }
            }
#pragma unroll 1
            for (int lb = 0; lb < QB; ++lb) {
                const int l = lb * 32 + r;
                // non-negative floats order like their bit patterns: a scalar compare
                const bool fast = __builtin_amdgcn_readfirstlane(__float_as_int(blk_s[8 + lb])) <= __float_as_int(kFastDiagSpan);
                Frag<T> Cf[NK];
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) Cf[kk] = BT::split_frag(Cs, l, 16 * kk + 4 * half);
                f32x16 acc = {0};
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) {
                    acc = mma32(Hhi[kk], Cf[kk], acc);
                    acc = mma32(Hlo[kk], Cf[kk], acc);
                }
                acc = acc * blk_s[lb];
                const float *F_row = F_s + lb * Q;
                auto scores = [&](int sb) {
                    f32x16 sc = {0};
#pragma unroll
                    for (int kk = 0; kk < NK; ++kk)
                        sc = mma32(BT::split_frag(Bs, sb * 32 + r, 16 * kk + 4 * half), Cf[kk], sc);
                    return sc;
                };
                auto accumulate = [&](int sb, const Frag<T>(&mh)[2], const Frag<T>(&ml)[2]) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        // K order of mh[j]: rows s = 32 sb + 16 j + 4 half + {0..3} and the same + 8
                        const Frag<T> xf = XT::frag(xs, sb * 32 + 16 * j + 4 * half, 8, 0, lane);
                        acc = mma32(xf, mh[j], acc);
                        acc = mma32(xf, ml[j], acc);
                    }
                };
#pragma unroll 1
                for (int sb = 0; sb < lb; ++sb) {
                    const f32x16 sc = scores(sb);
                    Frag<T> mh[2], ml[2];
#pragma unroll
                    for (int vg = 0; vg < 4; ++vg) {
                        const float4 f4 = *reinterpret_cast<const float4 *>(F_row + sb * 32 + 8 * vg + 4 * half);
                        const float fv[4] = {f4.x, f4.y, f4.z, f4.w};
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int v = vg * 4 + i;
                            T vh, vl;
                            Split<T>::split(sc[v] * fv[i], vh, vl);
                            mh[v / 8].v[v % 8] = vh;
                            ml[v / 8].v[v % 8] = vl;
                        }
                    }
                    accumulate(sb, mh, ml);
                }
                {   // diagonal block
                    const f32x16 sc = scores(lb);
                    const float El = E_s[l];
                    Frag<T> mh[2], ml[2];
                    if (fast) {
#pragma unroll
                        for (int vg = 0; vg < 4; ++vg) {
                            const float4 f4 = *reinterpret_cast<const float4 *>(F_row + lb * 32 + 8 * vg + 4 * half);
                            const float fv[4] = {f4.x, f4.y, f4.z, f4.w};
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                const int v = vg * 4 + i;
                                const float wv = (8 * vg + 4 * half + i <= r) ? sc[v] * fv[i] : 0.f;
                                T vh, vl;
                                Split<T>::split(wv, vh, vl);
                                mh[v / 8].v[v % 8] = vh;
                                ml[v / 8].v[v % 8] = vl;
                            }
                        }
                        accumulate(lb, mh, ml);
                        acc = acc * El;
                    } else {
                        acc = acc * El;
                        const float al_hi = ah_s[l], al_lo = alo_s[l];
#pragma unroll
                        for (int vg = 0; vg < 4; ++vg) {
                            const int s0 = lb * 32 + 8 * vg + 4 * half;
                            const float4 ah4 = *reinterpret_cast<const float4 *>(ah_s + s0);
                            const float4 al4 = *reinterpret_cast<const float4 *>(alo_s + s0);
                            const float4 dt4 = *reinterpret_cast<const float4 *>(dt_s + s0);
                            const float ahv[4] = {ah4.x, ah4.y, ah4.z, ah4.w};
                            const float alv[4] = {al4.x, al4.y, al4.z, al4.w};
                            const float dtv4[4] = {dt4.x, dt4.y, dt4.z, dt4.w};
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                const int v = vg * 4 + i;
                                // masked entries get exp2(-inf) = 0: a select on the exponent
                                const float arg = fminf(alpha_diff(al_hi, al_lo, ahv[i], alv[i]), 0.f);
                                const float wv = exp2_hw((s0 + i <= l) ? arg : -INFINITY) * dtv4[i] * sc[v];
                                T vh, vl;
                                Split<T>::split(wv, vh, vl);
                                mh[v / 8].v[v % 8] = vh;
                                ml[v / 8].v[v % 8] = vl;
                            }
                        }
                        accumulate(lb, mh, ml);
                    }
                }
                // epilogue: y[t, h, p] = yT[p, l] + D[h] * x[t, h, p]
                float o[16];
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const bf16x4 x4 = XT::row4(xs, l, 8 * vg + 4 * half);
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[vg * 4 + i] = acc[vg * 4 + i] + dh * (float)x4[i];
                }
                store_column<TO>(yb + (size_t)(t0 + l) * HP, o, half, 32, l < rows);
            }
        }

        // ---- phase 2: the state leaving this chunk ----
        if (!EARLY && c + 1 < s.nc) prefetch(c + 1);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) st[nb] = st[nb] * a_end;
#pragma unroll 2
        for (int ks = 0; ks < Q; ks += 16) {
            const int k0 = ks + 8 * half;
            const Frag<T> xr = XT::frag(xs, k0, 4, 0, lane);  // x[l = k0..k0+7, p = r]
            const float4 wa = *reinterpret_cast<const float4 *>(w_s + k0);
            const float4 wb = *reinterpret_cast<const float4 *>(w_s + k0 + 4);
            const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
            Frag<T> xh, xl;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                T vh, vl;
                Split<T>::split(wv[i] * (float)xr.v[i], vh, vl);
                xh.v[i] = vh;
                xl.v[i] = vl;
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const Frag<T> bf = BT::frag(Bs, k0, 4, nb * 32, lane);  // B[l = k0..k0+7, n = 32 nb + r]
                st[nb] = mma32(bf, xh, st[nb]);
                st[nb] = mma32(bf, xl, st[nb]);
            }
        }
    }

    if (final_states) {
        float *fb = final_states + (((size_t)b * s.H + h) * s.P + pb * 32 + r) * N + 4 * half;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq)
                *reinterpret_cast<float4 *>(fb + 32 * nb + 8 * gq) =
                    make_float4(st[nb][4 * gq], st[nb][4 * gq + 1], st[nb][4 * gq + 2], st[nb][4 * gq + 3]);
        }
    }
}

// ------------------------------------------------------------------------------------------
// Launchers (one translation unit per output type instantiates fused_dispatch)
// ------------------------------------------------------------------------------------------
template <typename TO, int NK, int QB, int WAVES>
static hipError_t fused_launch(const ScanShape &s, const void *x, const void *dt, const float *A, const void *Bm,
                               const void *Cm, const float *D, const float *init, void *y, float *final_states,
                               hipStream_t st) {
    constexpr bool EARLY = false;
    const size_t lds = fused_scan_lds_bytes(16 * NK, 32 * QB, WAVES);
    hipError_t e = allow_lds(fused_scan_kernel<TO, NK, QB, WAVES, EARLY>, lds);
    if (e != hipSuccess) return e;
    const int units = (s.H / s.G) * (s.P / 32);
    const int grid = s.B * s.G * (units / WAVES);
    fused_scan_kernel<TO, NK, QB, WAVES, EARLY><<<dim3(grid), dim3(64 * WAVES), lds, st>>>(
        static_cast<const __bf16 *>(x), static_cast<const __bf16 *>(dt), A, static_cast<const __bf16 *>(Bm),
        static_cast<const __bf16 *>(Cm), D, init, static_cast<TO *>(y), final_states, s);
    return hipGetLastError();
}

template <typename TO, int NK, int QB>
static hipError_t fused_dispatch_w(const ScanShape &s, int waves, const void *x, const void *dt, const float *A,
                                   const void *Bm, const void *Cm, const float *D, const float *init, void *y,
                                   float *final_states, hipStream_t st) {
    return waves == 8 ? fused_launch<TO, NK, QB, 8>(s, x, dt, A, Bm, Cm, D, init, y, final_states, st)
                      : fused_launch<TO, NK, QB, 4>(s, x, dt, A, Bm, Cm, D, init, y, final_states, st);
}

template <typename TO>
hipError_t fused_dispatch(const ScanShape &s, int waves, const void *x, const void *dt, const float *A,
                          const void *Bm, const void *Cm, const float *D, const float *init, void *y,
                          float *final_states, hipStream_t st) {
#define SSD_FUSED_CASE(NKv, QBv) \
    if (s.N == 16 * NKv && s.Q == 32 * QBv) \
        return fused_dispatch_w<TO, NKv, QBv>(s, waves, x, dt, A, Bm, Cm, D, init, y, final_states, st);
    SSD_FUSED_CASE(2, 2)
    SSD_FUSED_CASE(2, 4)
    SSD_FUSED_CASE(4, 2)
    SSD_FUSED_CASE(4, 4)
#undef SSD_FUSED_CASE
    return hipErrorInvalidValue;
}

}  // namespace ssd
