// Mamba-2 SSD forward for gfx950 (MI355X, CDNA4): the four chunk-scan stages and the
// single-timestep streaming update.  Written for 64-wide wavefronts: stages 2 and 4 are
// 32x32 MFMA tiles with fp32 accumulation staged through LDS, stage 1 is a DPP wave scan,
// stages 3 and 5 are pure HBM streams.
//
// Notation: b batch, c chunk, l/s position inside a chunk (0..Q-1), h head, g group,
// p head-dim index, n state index, t = c*Q + l absolute timestep.
// alpha[l] = log2(e) * sum_{i<=l} dt[i]*A is the per-chunk cumulative log2-decay, so every
// decay factor is one v_exp_f32:  exp(sum_{s<i<=l} dt_i A) = exp2(alpha[l] - alpha[s]).
//
// MFMA operand convention used throughout (v_mfma_f32_32x32x16_bf16 and, in float mode,
// eight v_mfma_f32_32x32x2_f32): a lane with r = lane%32 and half = lane/32 supplies, for the
// A operand, 8 K-consecutive elements of row r starting at k = 8*half; for the B operand the
// same for column r.  Accumulator register v of that lane is element
// (row 8*(v/4) + 4*half + v%4, column r).
#include <type_traits>

#include "ssd_launch.h"

namespace ssd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <typename T> constexpr bool is_bf16 = std::is_same<T, __bf16>::value;

// ------------------------------------------------------------------------------------------
// Fragments and 16-byte vectors
// ------------------------------------------------------------------------------------------
template <typename T> struct Frag;
template <> struct Frag<__bf16> {
    bf16x8 v;
};
template <> struct Frag<float> {
    float v[8];
};

__device__ inline f32x16 mma32(const Frag<__bf16> &a, const Frag<__bf16> &b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}
// Float mode: K index 8*half + i is fed to MFMA number i as its k = half; the K order is a
// permutation of the bf16 one, which a sum does not see.
__device__ inline f32x16 mma32(const Frag<float> &a, const Frag<float> &b, f32x16 c) {
#pragma unroll
    for (int i = 0; i < 8; ++i) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i], b.v[i], c, 0, 0, 0);
    return c;
}

template <typename T> struct Vec16;  // one 16-byte global/LDS transaction
template <> struct Vec16<__bf16> {
    static constexpr int N = 8;
    union {
        uint4 u;
        __bf16 e[8];
    };
};
template <> struct Vec16<float> {
    static constexpr int N = 4;
    union {
        uint4 u;
        float e[4];
    };
};

template <typename T> __device__ inline Vec16<T> load_vec16(const T *p) {
    Vec16<T> r;
    r.u = *reinterpret_cast<const uint4 *>(p);
    return r;
}
template <typename T> __device__ inline Vec16<T> zero_vec16() {
    Vec16<T> r;
    r.u = make_uint4(0, 0, 0, 0);
    return r;
}
template <typename T> __device__ inline Frag<T> zero_frag() {
    Frag<T> f;
#pragma unroll
    for (int i = 0; i < 8; ++i) f.v[i] = (T)0.f;
    return f;
}

// 8 consecutive elements starting at p (16-byte aligned).
__device__ inline Frag<__bf16> load_frag(const __bf16 *p) {
    Frag<__bf16> f;
    f.v = *reinterpret_cast<const bf16x8 *>(p);
    return f;
}
__device__ inline Frag<float> load_frag(const float *p) {
    Frag<float> f;
    const float4 a = *reinterpret_cast<const float4 *>(p);
    const float4 b = *reinterpret_cast<const float4 *>(p + 4);
    f.v[0] = a.x; f.v[1] = a.y; f.v[2] = a.z; f.v[3] = a.w;
    f.v[4] = b.x; f.v[5] = b.y; f.v[6] = b.z; f.v[7] = b.w;
    return f;
}
// Elements p[0..3] and p[8..11]: the K order in which an accumulator tile, reused directly as
// a B operand, presents its rows (see chunk_scan_kernel).  Float mode only; bf16 uses LDS
// transpose reads.
__device__ inline Frag<float> load_frag_split(const float *p) {
    Frag<float> f;
    const float4 a = *reinterpret_cast<const float4 *>(p);
    const float4 b = *reinterpret_cast<const float4 *>(p + 8);
    f.v[0] = a.x; f.v[1] = a.y; f.v[2] = a.z; f.v[3] = a.w;
    f.v[4] = b.x; f.v[5] = b.y; f.v[6] = b.z; f.v[7] = b.w;
    return f;
}

template <typename T> __device__ inline void store4(T *p, float a, float b, float c, float d);
template <> __device__ inline void store4<float>(float *p, float a, float b, float c, float d) {
    *reinterpret_cast<float4 *>(p) = make_float4(a, b, c, d);
}
template <> __device__ inline void store4<__bf16>(__bf16 *p, float a, float b, float c, float d) {
    bf16x4 v;
    v[0] = (__bf16)a; v[1] = (__bf16)b; v[2] = (__bf16)c; v[3] = (__bf16)d;
    *reinterpret_cast<bf16x4 *>(p) = v;
}

template <typename T> constexpr int lds_pad() { return 16 / (int)sizeof(T); }

// exp2 as the single hardware instruction (v_exp_f32, ~1 ulp); arguments here are <= 0 and
// results below 2^-126 flush to zero, which is the wanted limit of a vanished decay.
__device__ inline float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }
// alpha difference from hi/lo pairs: good to the rounding of the difference itself
__device__ inline float alpha_diff(float hi_a, float lo_a, float hi_b, float lo_b) {
    return (hi_a - hi_b) + (lo_a - lo_b);
}

// hi/lo split of an fp32 value into two bf16 (relative error 2^-17 instead of 2^-9); in float
// mode there is nothing to split.
template <typename T> struct Split;
template <> struct Split<__bf16> {
    static constexpr int PARTS = 2;
    static __device__ inline void split(float v, __bf16 &hi, __bf16 &lo) {
        hi = (__bf16)v;
        lo = (__bf16)(v - (float)hi);
    }
};
template <> struct Split<float> {
    static constexpr int PARTS = 1;
    static __device__ inline void split(float v, float &hi, float &lo) {
        hi = v;
        lo = 0.f;
    }
};

// ------------------------------------------------------------------------------------------
// Row-major bf16 tiles in LDS read through the gfx950 transpose load.
//
// x and B arrive with the MFMA K axis (time) as their slow axis, but an MFMA lane needs K
// consecutive for its row/column.  ds_read_b64_tr_b16 does that transposition inside the LDS
// read: within each block of 16 lanes, lane 4a+b supplies the address of 4 consecutive
// 16-bit elements of tile row (k0+a), columns c0+4b..c0+4b+3, and lane i receives the 4
// elements tile[k0+0..3][c0+i] (measured on the device; one such read is half of an 8-deep
// MFMA operand).  Tiles are therefore stored exactly as they come from memory, with 16-byte
// vector writes, instead of being scattered element by element.
//
// COLS (elements per row) is 32, 64 or 128, i.e. 1, 2 or 4 granules of 64 bytes.  A transpose
// read touches 4 consecutive rows x 64 bytes per 32 lanes; the granule index is XOR-swizzled
// with the row so those four pieces fall into the four quarters of the 64 banks.
// ------------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_gcc;
#define SSD_LDS_AS __attribute__((address_space(3)))

template <int COLS> struct RowMajorTile {
    static constexpr int GR = COLS / 32;
    static __device__ inline int swz(int row) { return GR == 1 ? 0 : (GR == 2 ? ((row >> 1) & 1) : (row & 3)); }
    // element offset of (row, col); col..col+7 stay inside one granule when col % 8 == 0
    static __device__ inline int off(int row, int col) {
        return row * COLS + ((((col >> 5) ^ swz(row)) << 5) | (col & 31));
    }
    // this lane's 4 elements tile[k0 + 0..3][c0 + lane%16 + 16*((lane/16)%2)] -- with k0 already
    // including the lane half's K offset, that is K-consecutive data for operand row c0 + lane%32
    static __device__ inline bf16x4 tr4(const __bf16 *tile, int k0, int c0, int lane) {
        const int q = lane >> 4, a = (lane >> 2) & 3, b = lane & 3;
        const __bf16 *src = tile + off(k0 + a, c0 + 16 * (q & 1) + 4 * b);
        const bf16x4_gcc v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((SSD_LDS_AS bf16x4_gcc *)(src));
        return __builtin_bit_cast(bf16x4, v);
    }
    // operand fragment: rows k0..k0+3 then k0+gap..k0+gap+3 (gap 4 = 8 consecutive K values)
    static __device__ inline Frag<__bf16> frag(const __bf16 *tile, int k0, int gap, int c0, int lane) {
        Frag<__bf16> f;
        const bf16x4 lo = tr4(tile, k0, c0, lane), hi = tr4(tile, k0 + gap, c0, lane);
        f.v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return f;
    }
};

// Workgroups are dealt round-robin to the 8 XCDs, each with a private L2.  Re-number them so
// that consecutive logical ids (the heads of one (b,c) tile, which share B and C and sit in
// the same cache lines of x) land on the same XCD at nearly the same time.
__device__ inline int xcd_remap(int bid, int total) {
    return (total % 8 == 0) ? (bid % 8) * (total / 8) + bid / 8 : bid;
}

// ------------------------------------------------------------------------------------------
// Stage 1: chunk_cumsum.  One workgroup per (b,c): the [Q,H] tile of dt is read coalesced,
// transposed through LDS, and every head row gets a wavefront inclusive scan of dt*A.
//
// Output "dtcs" [B,H,nc,3,Q] float32: rows 0/1 = alpha (the cumulative sum times log2 e) as
// an unevaluated pair hi + lo, row 2 = dt.  The scan runs in float64 and is split into two
// floats because the later stages only ever use DIFFERENCES alpha[l] - alpha[s]: with one
// float, a large |alpha| (hundreds after a strongly decaying step) leaves an absolute error
// of ulp(|alpha|) in a difference that may itself be small, i.e. a relative error of
// 1e-5..1e-3 in the decay factor.  (hi_l - hi_s) + (lo_l - lo_s) keeps the difference good to
// its own ulp.
// ------------------------------------------------------------------------------------------
template <int CTRL, int ROWMASK> __device__ inline double dpp_move(double v) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROWMASK, 0xf, false);
    hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROWMASK, 0xf, false);
    return __hiloint2double(hi, lo);  // lanes the row mask disables, or with no source lane, get +0.0
}
// Inclusive sum across the 64 lanes with DPP data movement: shifts inside rows of 16, then the
// row totals are broadcast into the following rows (row_bcast:15 / row_bcast:31).
__device__ inline double wave_inclusive_scan(double v) {
    v += dpp_move<0x111, 0xf>(v);  // row_shr:1
    v += dpp_move<0x112, 0xf>(v);  // row_shr:2
    v += dpp_move<0x114, 0xf>(v);  // row_shr:4
    v += dpp_move<0x118, 0xf>(v);  // row_shr:8
    v += dpp_move<0x142, 0xa>(v);  // row_bcast:15 -> rows 1,3
    v += dpp_move<0x143, 0xc>(v);  // row_bcast:31 -> rows 2,3
    return v;
}

template <typename T, int EPL>  // EPL = elements per lane = max(Q/64, 1)
__global__ __launch_bounds__(256) void chunk_cumsum_kernel(const T *__restrict__ dt,
                                                           const float *__restrict__ A,
                                                           float *__restrict__ dtcs, ScanShape s) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *tile = reinterpret_cast<float *>(smem);  // [H][Q+1]
    const int ldt = s.Q + 1;
    const int b = blockIdx.x / s.nc, c = blockIdx.x % s.nc;
    const int t0 = c * s.Q;
    for (int idx = threadIdx.x; idx < s.Q * s.H; idx += blockDim.x) {
        const int l = idx / s.H, h = idx % s.H;
        const int t = t0 + l;
        const float v = (t < s.L) ? (float)dt[((size_t)b * s.L + t) * s.H + h] : 0.f;
        tile[h * ldt + l] = v;
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
            run += (double)dtv[e] * a;
            cs[e] = run;
        }
        const double excl = wave_inclusive_scan(run) - run;
        if (l0 < s.Q) {
            float *row = dtcs + ((((size_t)b * s.H + h) * s.nc + c) * 3) * s.Q + l0;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const double al = (cs[e] + excl) * kLog2e;
                const float hi = (float)al;
                row[e] = hi;
                row[s.Q + e] = (float)(al - (double)hi);
                row[2 * s.Q + e] = dtv[e];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Stage 2: chunk_state.  One workgroup per (b,c,h); one wave per 32x32 tile of S[p,n].
//   S = (w o x)^T [P x Q] . B [Q x N],   w[l] = exp2(alpha[Q-1] - alpha[l]) * dt[l]
// The decay weight goes onto the x side (the smaller tile) in fp32; in bf16 mode the weighted
// x is kept as a hi + lo pair of bf16 (two MFMAs per K step) so that the result carries the
// inputs' precision rather than one extra bf16 rounding.  B enters exactly as given.
// Both operands have K = l as their slow axis in memory: bf16 tiles are stored row-major and
// transposed by the LDS transpose read; float tiles are transposed on their way into LDS.
// All global loads of a workgroup are issued before the first LDS write.
// ------------------------------------------------------------------------------------------
template <typename T, int PB, int NB>  // PB = ceil(P/32), NB = ceil(N/32)
__global__ __launch_bounds__(512) void chunk_state_kernel(const T *__restrict__ x,
                                                          const T *__restrict__ Bm,
                                                          const float *__restrict__ dtcs,
                                                          float *__restrict__ states, ScanShape s) {
    constexpr int VEC = Vec16<T>::N;
    constexpr int PARTS = Split<T>::PARTS;
    constexpr int Ppad = PB * 32, Npad = NB * 32;
    constexpr int UX = 4, UB = 8;  // 16-byte loads in flight per thread (one batch covers the usual tiles)
    using XT = RowMajorTile<Ppad>;
    using BT = RowMajorTile<Npad>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int ldq = s.Q + lds_pad<T>();  // float mode: transposed tiles [p or n][ldq]
    float *w_s = reinterpret_cast<float *>(smem);  // [Q]
    T *xs = reinterpret_cast<T *>(w_s + s.Q);      // bf16: [PARTS][Q][Ppad] row-major; float: [Ppad][ldq]
    T *bs = xs + (is_bf16<T> ? (size_t)PARTS * s.Q * Ppad : (size_t)Ppad * ldq);  // bf16: [Q][Npad]; float: [Npad][ldq]

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int h = logical % s.H;
    const int c = (logical / s.H) % s.nc;
    const int b = logical / (s.H * s.nc);
    const int g = h / (s.H / s.G);
    const int t0 = c * s.Q;
    const int tid = threadIdx.x, nthr = blockDim.x;
    const float *arow = dtcs + ((((size_t)b * s.H + h) * s.nc + c) * 3) * s.Q;

    const int xcpr = s.P / VEC, xtotal = s.Q * xcpr;
    const int bcpr = s.N / VEC, btotal = s.Q * bcpr;
    auto load_x = [&](int idx) {
        const int l = idx / xcpr, ch = idx % xcpr;
        return (idx < xtotal && t0 + l < s.L)
                   ? load_vec16(x + (((size_t)b * s.L + t0 + l) * s.H + h) * s.P + ch * VEC)
                   : zero_vec16<T>();
    };
    auto load_b = [&](int idx) {
        const int l = idx / bcpr, ch = idx % bcpr;
        return (idx < btotal && t0 + l < s.L)
                   ? load_vec16(Bm + (((size_t)b * s.L + t0 + l) * s.G + g) * s.N + ch * VEC)
                   : zero_vec16<T>();
    };
    // ---- issue the first batch of every global load before anything waits ----
    Vec16<T> xv[UX], bv[UB];
#pragma unroll
    for (int u = 0; u < UX; ++u) xv[u] = load_x(u * nthr + tid);
#pragma unroll
    for (int u = 0; u < UB; ++u) bv[u] = load_b(u * nthr + tid);
    const float e_hi = arow[s.Q - 1], e_lo = arow[2 * s.Q - 1];
    for (int l = tid; l < s.Q; l += nthr)
        w_s[l] = exp2_hw(fminf(alpha_diff(e_hi, e_lo, arow[l], arow[s.Q + l]), 0.f)) * arow[2 * s.Q + l];
    // zero what no load covers (only when P or N is not a multiple of 32)
    if (is_bf16<T>) {
        if (s.P < Ppad)
            for (int idx = tid; idx < PARTS * s.Q * Ppad; idx += nthr) xs[idx] = (T)0.f;
        if (s.N < Npad)
            for (int idx = tid; idx < s.Q * Npad; idx += nthr) bs[idx] = (T)0.f;
    } else {
        for (int idx = tid; idx < (Ppad - s.P) * ldq; idx += nthr) xs[(size_t)s.P * ldq + idx] = (T)0.f;
        for (int idx = tid; idx < (Npad - s.N) * ldq; idx += nthr) bs[(size_t)s.N * ldq + idx] = (T)0.f;
    }
    __syncthreads();

    // ---- into LDS: weighted x (hi/lo in bf16 mode), B as is ----
    for (int base = 0; base < xtotal; base += UX * nthr) {
        if (base > 0) {
#pragma unroll
            for (int u = 0; u < UX; ++u) xv[u] = load_x(base + u * nthr + tid);
        }
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            const int idx = base + u * nthr + tid;
            if (idx < xtotal) {
                const int l = idx / xcpr, ch = idx % xcpr;
                const float w = w_s[l];
                if constexpr (is_bf16<T>) {
                    Vec16<T> hi, lo;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) Split<T>::split(w * (float)xv[u].e[i], hi.e[i], lo.e[i]);
                    const int o = XT::off(l, ch * VEC);
                    *reinterpret_cast<uint4 *>(xs + o) = hi.u;
                    *reinterpret_cast<uint4 *>(xs + (size_t)s.Q * Ppad + o) = lo.u;
                } else {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) xs[(size_t)(ch * VEC + i) * ldq + l] = w * xv[u].e[i];
                }
            }
        }
    }
    for (int base = 0; base < btotal; base += UB * nthr) {
        if (base > 0) {
#pragma unroll
            for (int u = 0; u < UB; ++u) bv[u] = load_b(base + u * nthr + tid);
        }
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int idx = base + u * nthr + tid;
            if (idx < btotal) {
                const int l = idx / bcpr, ch = idx % bcpr;
                if constexpr (is_bf16<T>) {
                    *reinterpret_cast<uint4 *>(bs + BT::off(l, ch * VEC)) = bv[u].u;
                } else {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) bs[(size_t)(ch * VEC + i) * ldq + l] = bv[u].e[i];
                }
            }
        }
    }
    __syncthreads();

    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, half = lane >> 5;
    const int pb = wave / NB, nb = wave % NB;
    f32x16 acc = {0};
    if constexpr (is_bf16<T>) {
        for (int ks = 0; ks < s.Q; ks += 16) {
            const int k0 = ks + 8 * half;
            const Frag<T> bf = BT::frag(bs, k0, 4, nb * 32, lane);
            acc = mma32(XT::frag(xs, k0, 4, pb * 32, lane), bf, acc);
            acc = mma32(XT::frag(xs + (size_t)s.Q * Ppad, k0, 4, pb * 32, lane), bf, acc);
        }
    } else {
        const T *arow_p = xs + (size_t)(pb * 32 + r) * ldq + half * 8;
        const T *brow_p = bs + (size_t)(nb * 32 + r) * ldq + half * 8;
        for (int ks = 0; ks < s.Q; ks += 16) acc = mma32(load_frag(arow_p + ks), load_frag(brow_p + ks), acc);
    }

    const int n = nb * 32 + r;
    float *out = states + ((((size_t)b * s.nc + c) * s.H + h) * s.P) * s.N;
    if (n < s.N) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int p = pb * 32 + 8 * (v / 4) + 4 * half + (v % 4);
            if (p < s.P) out[(size_t)p * s.N + n] = acc[v];
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
    const float *a_end = dtcs + ((size_t)bh * s.nc) * 3 * s.Q + (s.Q - 1);  // alpha_hi at the chunk end
    const size_t a_stride = (size_t)3 * s.Q;
    float4 st = init ? reinterpret_cast<const float4 *>(init)[(size_t)bh * pn4 + idx] : make_float4(0, 0, 0, 0);
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

// ------------------------------------------------------------------------------------------
// Stage 4: chunk_scan.  One workgroup per (b,c,h); each wave owns 32 output columns
// l in [32*lb, 32*lb+32) and computes the TRANSPOSED output tile yT[p,l]:
//   yT  = exp2(alpha[l]) * (Hc [P x N] . C^T [N x l])                   state readout
//       + sum over s-blocks sb <= lb of  xT [P x s] . M^T [s x l]        intra-chunk
//   M^T[s,l] = (B[s,:] . C[l,:]) * exp2(alpha[l] - alpha[s]) * dt[s]  for s <= l, else 0
// Computing the transpose makes the 32x32 accumulator of B.C^T directly usable as the B
// operand of the second MFMA (its lane already holds column l and 16 rows s), so the masked
// score matrix never leaves registers; the A operand xT is read from LDS in the matching K
// order.  C fragments for the wave's 32 columns stay in registers for both products.
//
// Decay factors.  Only the diagonal block (sb == lb) needs a mask and one exp2 per element
// (mask before exp2: no inf*0).  Below the diagonal the factor separates through the first
// row m = 32*lb of the column block, exp2(alpha[l]-alpha[s]) = exp2(alpha[l]-alpha[m]) *
// exp2(alpha[m]-alpha[s]) with both exponents <= 0: one value per lane times a per-row table
// (dt folded in) that the workgroup builds once in LDS.
//
// In bf16 mode the two operands this kernel manufactures in fp32 -- M and the entering state
// Hc -- are fed to the MFMA as hi + lo bf16 pairs; x, B and C enter exactly as given.
// TO is the element type of y (T, or float for bf16 inputs with float32 output).
// The column-block index is rotated with the workgroup id so that the wave with the most
// s-blocks does not always sit on the same SIMD.
// ------------------------------------------------------------------------------------------
template <typename T, typename TO, int PB, int NK>  // PB = ceil(P/32), NK = N/16
__global__ __launch_bounds__(512) void chunk_scan_kernel(const T *__restrict__ x, const T *__restrict__ Bm,
                                                         const T *__restrict__ Cm,
                                                         const float *__restrict__ dtcs,
                                                         const float *__restrict__ prev,
                                                         const float *__restrict__ D, TO *__restrict__ y,
                                                         ScanShape s) {
    constexpr int VEC = Vec16<T>::N;
    constexpr int PARTS = Split<T>::PARTS;
    constexpr int N = NK * 16;
    constexpr int Ppad = PB * 32;
    constexpr int ldb = N + lds_pad<T>();
    constexpr int UB = N / (2 * VEC);        // B loads per thread: Q*N/VEC chunks over 2Q threads
    constexpr int UX = (Ppad + 2 * VEC - 1) / (2 * VEC);
    constexpr int UH = 4;                    // state float4 loads per thread and batch
    using XT = RowMajorTile<Ppad>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int ldx = s.Q + lds_pad<T>();      // float mode: xs is transposed [Ppad][ldx]
    const int nblk = s.Q / 32;
    float *al_s = reinterpret_cast<float *>(smem);  // [3][Q]: alpha hi, alpha lo, dt
    float *tab = al_s + 3 * s.Q;                    // [nblk][Q]: exp2(alpha[32k]-alpha[s])*dt[s], s < 32k
    T *Bs = reinterpret_cast<T *>(tab + nblk * s.Q);  // [Q][ldb]
    T *Hs = Bs + (size_t)s.Q * ldb;                 // [PARTS][Ppad][ldb]
    T *xs = Hs + (size_t)PARTS * Ppad * ldb;        // bf16: [Q][Ppad] row-major; float: [Ppad][ldx]

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int h = logical % s.H;
    const int c = (logical / s.H) % s.nc;
    const int b = logical / (s.H * s.nc);
    const int g = h / (s.H / s.G);
    const int t0 = c * s.Q;
    const int tid = threadIdx.x, nthr = blockDim.x;  // nthr == 2Q
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, half = lane >> 5;
    const int lb = (wave + logical) % nblk;          // this wave's column block
    const float *arow = dtcs + ((((size_t)b * s.H + h) * s.nc + c) * 3) * s.Q;

    // ---- issue every global load, in the order the data is consumed ----
    float a3[2];
    a3[0] = (tid < 3 * s.Q) ? arow[tid] : 0.f;
    a3[1] = (tid + nthr < 3 * s.Q) ? arow[tid + nthr] : 0.f;
    constexpr int bcpr = N / VEC;
    Vec16<T> bv[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        const int idx = u * nthr + tid;
        const int sr = idx / bcpr, ch = idx % bcpr;
        bv[u] = (t0 + sr < s.L) ? load_vec16(Bm + (((size_t)b * s.L + t0 + sr) * s.G + g) * N + ch * VEC)
                                : zero_vec16<T>();
    }
    const int xcpr = s.P / VEC, xtotal = s.Q * xcpr;
    Vec16<T> xv[UX];
#pragma unroll
    for (int u = 0; u < UX; ++u) {
        const int idx = u * nthr + tid;
        const int sr = idx / xcpr, ch = idx % xcpr;
        xv[u] = (idx < xtotal && t0 + sr < s.L)
                    ? load_vec16(x + (((size_t)b * s.L + t0 + sr) * s.H + h) * s.P + ch * VEC)
                    : zero_vec16<T>();
    }
    const float *hp = prev + ((((size_t)b * s.nc + c) * s.H + h) * s.P) * N;
    constexpr int hcpr = N / 4;
    const int htotal = s.P * hcpr;
    float4 hv[UH];
#pragma unroll
    for (int u = 0; u < UH; ++u) {
        const int idx = u * nthr + tid;
        hv[u] = (idx < htotal) ? *reinterpret_cast<const float4 *>(hp + (size_t)idx * 4) : make_float4(0, 0, 0, 0);
    }
    // C fragments straight from global: column l = 32*lb + r, K = n
    const int l = lb * 32 + r;
    const bool l_valid = (t0 + l) < s.L;
    Frag<T> Cf[NK];
    {
        const T *crow = Cm + (((size_t)b * s.L + t0 + l) * s.G + g) * N + half * 8;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) Cf[kk] = l_valid ? load_frag(crow + kk * 16) : zero_frag<T>();
    }
    // decay table rows k = 1..nblk-1 (row 0 is never read): small, cached reads of the alpha row
    for (int idx = tid; idx < nblk * s.Q; idx += nthr) {
        const int k = idx / s.Q, sr = idx % s.Q;
        if (k > 0 && sr < 32 * k) {
            const float d = alpha_diff(arow[32 * k], arow[s.Q + 32 * k], arow[sr], arow[s.Q + sr]);
            tab[idx] = exp2_hw(fminf(d, 0.f)) * arow[2 * s.Q + sr];
        }
    }

    // ---- into LDS ----
    if (tid < 3 * s.Q) al_s[tid] = a3[0];
    if (tid + nthr < 3 * s.Q) al_s[tid + nthr] = a3[1];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        const int idx = u * nthr + tid;
        const int sr = idx / bcpr, ch = idx % bcpr;
        *reinterpret_cast<uint4 *>(Bs + (size_t)sr * ldb + ch * VEC) = bv[u].u;
    }
    if (is_bf16<T> && s.P < Ppad)
        for (int idx = tid; idx < s.Q * Ppad; idx += nthr) xs[idx] = (T)0.f;
    if (!is_bf16<T>)
        for (int idx = tid; idx < (Ppad - s.P) * ldx; idx += nthr) xs[(size_t)s.P * ldx + idx] = (T)0.f;
    if (is_bf16<T> && s.P < Ppad) __syncthreads();  // the zero fill above overlaps the tile writes below
#pragma unroll
    for (int u = 0; u < UX; ++u) {
        const int idx = u * nthr + tid;
        if (idx < xtotal) {
            const int sr = idx / xcpr, ch = idx % xcpr;
            if constexpr (is_bf16<T>) {
                *reinterpret_cast<uint4 *>(xs + XT::off(sr, ch * VEC)) = xv[u].u;
            } else {
#pragma unroll
                for (int i = 0; i < VEC; ++i) xs[(size_t)(ch * VEC + i) * ldx + sr] = xv[u].e[i];
            }
        }
    }
    for (int base = 0; base < htotal; base += UH * nthr) {
        if (base > 0) {
#pragma unroll
            for (int u = 0; u < UH; ++u) {
                const int idx = base + u * nthr + tid;
                hv[u] = (idx < htotal) ? *reinterpret_cast<const float4 *>(hp + (size_t)idx * 4)
                                       : make_float4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < UH; ++u) {
            const int idx = base + u * nthr + tid;
            if (idx < htotal) {
                const int p = idx / hcpr, n4 = idx % hcpr;
                const float v[4] = {hv[u].x, hv[u].y, hv[u].z, hv[u].w};
                T hi[4], lo[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) Split<T>::split(v[i], hi[i], lo[i]);
                T *dsth = Hs + (size_t)p * ldb + n4 * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i) dsth[i] = hi[i];
                if (PARTS == 2) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) dsth[(size_t)Ppad * ldb + i] = lo[i];
                }
            }
        }
    }
    for (int idx = tid; idx < PARTS * (Ppad - s.P) * ldb; idx += nthr) {
        const int part = idx / ((Ppad - s.P) * ldb), rem = idx % ((Ppad - s.P) * ldb);
        Hs[((size_t)part * Ppad + s.P) * ldb + rem] = (T)0.f;
    }
    __syncthreads();

    const float *ah_s = al_s, *alo_s = al_s + s.Q, *dt_s = al_s + 2 * s.Q;
    const float al_hi = ah_s[l], al_lo = alo_s[l];
    f32x16 accY[PB];
    // state readout, scaled per output column by exp2(alpha[l]) (alpha <= 0)
    {
        const float el = exp2_hw(al_hi + al_lo);
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            f32x16 a = {0};
            const T *hrow = Hs + (size_t)(pb * 32 + r) * ldb + half * 8;
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
                a = mma32(load_frag(hrow + kk * 16), Cf[kk], a);
                if (PARTS == 2) a = mma32(load_frag(hrow + (size_t)Ppad * ldb + kk * 16), Cf[kk], a);
            }
            accY[pb] = a * el;
        }
    }
    // intra-chunk: s-blocks at or below this wave's column block (causal)
    const float lane_dec = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah_s[32 * lb], alo_s[32 * lb]), 0.f));
    const float *tab_row = tab + lb * s.Q;
    for (int sb = 0; sb <= lb; ++sb) {
        f32x16 sc = {0};
        const T *brow = Bs + (size_t)(sb * 32 + r) * ldb + half * 8;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) sc = mma32(load_frag(brow + kk * 16), Cf[kk], sc);
        Frag<T> mh[2], ml[2];
        if (sb < lb) {
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const int s0 = sb * 32 + 8 * vg + 4 * half;
                const float4 t4 = *reinterpret_cast<const float4 *>(tab_row + s0);
                const float tv[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int v = vg * 4 + i;
                    T hi, lo;
                    Split<T>::split(sc[v] * tv[i] * lane_dec, hi, lo);
                    mh[v / 8].v[v % 8] = hi;
                    if (PARTS == 2) ml[v / 8].v[v % 8] = lo;
                }
            }
        } else {
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const int s0 = sb * 32 + 8 * vg + 4 * half;
                const float4 ah4 = *reinterpret_cast<const float4 *>(ah_s + s0);
                const float4 al4 = *reinterpret_cast<const float4 *>(alo_s + s0);
                const float4 dt4 = *reinterpret_cast<const float4 *>(dt_s + s0);
                const float ahv[4] = {ah4.x, ah4.y, ah4.z, ah4.w};
                const float alv[4] = {al4.x, al4.y, al4.z, al4.w};
                const float dtv[4] = {dt4.x, dt4.y, dt4.z, dt4.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int v = vg * 4 + i;
                    const float arg = alpha_diff(al_hi, al_lo, ahv[i], alv[i]);
                    const float w = (s0 + i <= l) ? exp2_hw(fminf(arg, 0.f)) * dtv[i] * sc[v] : 0.f;
                    T hi, lo;
                    Split<T>::split(w, hi, lo);
                    mh[v / 8].v[v % 8] = hi;
                    if (PARTS == 2) ml[v / 8].v[v % 8] = lo;
                }
            }
        }
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                // K order of mh[j]: rows s = sb*32 + 16j + 4*half + {0..3} and the same + 8
                Frag<T> xf;
                if constexpr (is_bf16<T>) {
                    xf = XT::frag(xs, sb * 32 + 16 * j + 4 * half, 8, pb * 32, lane);
                } else {
                    xf = load_frag_split(xs + (size_t)(pb * 32 + r) * ldx + sb * 32 + 16 * j + 4 * half);
                }
                accY[pb] = mma32(xf, mh[j], accY[pb]);
                if (PARTS == 2) accY[pb] = mma32(xf, ml[j], accY[pb]);
            }
        }
    }
    // epilogue: y[t, h, p] = yT[p, l] + D[h] * x[t, h, p]
    if (l_valid) {
        const float dh = D ? D[h] : 0.f;
        TO *yrow = y + (((size_t)b * s.L + t0 + l) * s.H + h) * s.P;
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const int p0 = pb * 32 + 8 * vg + 4 * half;
                if (p0 < s.P) {
                    float xl[4];
                    if constexpr (is_bf16<T>) {
                        const bf16x4 x4 = *reinterpret_cast<const bf16x4 *>(xs + XT::off(l, p0));
#pragma unroll
                        for (int i = 0; i < 4; ++i) xl[i] = (float)x4[i];
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) xl[i] = xs[(size_t)(p0 + i) * ldx + l];
                    }
                    store4<TO>(yrow + p0, accY[pb][vg * 4 + 0] + dh * xl[0], accY[pb][vg * 4 + 1] + dh * xl[1],
                               accY[pb][vg * 4 + 2] + dh * xl[2], accY[pb][vg * 4 + 3] + dh * xl[3]);
                }
            }
        }
    }
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
    constexpr int UN = 4;         // passes whose loads are issued together
    const int lane = threadIdx.x & 63;
    const long long bh = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (bh >= (long long)s.B * s.H) return;
    const int b = (int)(bh / s.H), h = (int)(bh % s.H);
    const int g = h / (s.H / s.G);
    const int nl = lane % NL, rl = lane / NL;
    const float dtv = (float)dt[bh];
    const float decay = expf(dtv * A[h]);
    const float dh = D ? D[h] : 0.f;
    float bv[4], cv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bv[i] = (float)Bm[((size_t)b * s.G + g) * N + nl * 4 + i] * dtv;
        cv[i] = (float)Cm[((size_t)b * s.G + g) * N + nl * 4 + i];
    }
    float4 *st = reinterpret_cast<float4 *>(state) + (size_t)bh * s.P * NL;
    const T *xr = x + (size_t)bh * s.P;
    TO *yr = y + (size_t)bh * s.P;
    for (int p0 = 0; p0 < s.P; p0 += RPP * UN) {
        float4 hv[UN];
        float xv[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int p = p0 + u * RPP + rl;
            if (p < s.P) {
                hv[u] = st[(size_t)p * NL + nl];
                xv[u] = (float)xr[p];
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int p = p0 + u * RPP + rl;
            float part = 0.f;
            if (p < s.P) {
                float4 v = hv[u];
                v.x = decay * v.x + xv[u] * bv[0];
                v.y = decay * v.y + xv[u] * bv[1];
                v.z = decay * v.z + xv[u] * bv[2];
                v.w = decay * v.w + xv[u] * bv[3];
                st[(size_t)p * NL + nl] = v;
                part = v.x * cv[0] + v.y * cv[1] + v.z * cv[2] + v.w * cv[3];
            }
#pragma unroll
            for (int m = NL / 2; m >= 1; m >>= 1) part += __shfl_xor(part, m, 64);
            if (p < s.P && nl == 0) yr[p] = (TO)(part + dh * xv[u]);
        }
    }
}

// ------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------
size_t chunk_state_lds_bytes(const ScanShape &s, int eb) {
    const size_t Ppad = (s.P + 31) & ~31, Npad = (s.N + 31) & ~31;
    if (eb == 2) return (size_t)s.Q * 4 + ((size_t)2 * s.Q * Ppad + (size_t)s.Q * Npad) * 2;
    return (size_t)s.Q * 4 + (Ppad + Npad) * (size_t)(s.Q + 4) * 4;
}

size_t chunk_scan_lds_bytes(const ScanShape &s, int eb) {
    const size_t Ppad = (s.P + 31) & ~31;
    const size_t ldb = s.N + 16 / eb, parts = eb == 2 ? 2 : 1;
    const size_t xs = eb == 2 ? (size_t)s.Q * Ppad : Ppad * (size_t)(s.Q + 4);
    return (size_t)s.Q * 12 + (size_t)(s.Q / 32) * s.Q * 4 + ((size_t)s.Q * ldb + parts * Ppad * ldb + xs) * eb;
}

template <typename K> static hipError_t allow_lds(K kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

template <typename T>
static hipError_t cumsum_dispatch(const ScanShape &s, const void *dt, const float *A, float *dtcs,
                                  hipStream_t st) {
    const dim3 grid(s.B * s.nc), block(256);
    const size_t lds = (size_t)s.H * (s.Q + 1) * sizeof(float);
    const T *d = static_cast<const T *>(dt);
    if (s.Q <= 64) {
        chunk_cumsum_kernel<T, 1><<<grid, block, lds, st>>>(d, A, dtcs, s);
    } else if (s.Q == 128) {
        chunk_cumsum_kernel<T, 2><<<grid, block, lds, st>>>(d, A, dtcs, s);
    } else {
        chunk_cumsum_kernel<T, 4><<<grid, block, lds, st>>>(d, A, dtcs, s);
    }
    return hipGetLastError();
}

hipError_t launch_chunk_cumsum(const ScanShape &s, int dtype, const void *dt, const float *A, float *dtcs,
                               hipStream_t st) {
    return dtype ? cumsum_dispatch<__bf16>(s, dt, A, dtcs, st) : cumsum_dispatch<float>(s, dt, A, dtcs, st);
}

template <typename T, int PB, int NB>
static hipError_t state_launch(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                               float *states, hipStream_t st) {
    const size_t lds = chunk_state_lds_bytes(s, sizeof(T));
    hipError_t e = allow_lds(chunk_state_kernel<T, PB, NB>, lds);
    if (e != hipSuccess) return e;
    chunk_state_kernel<T, PB, NB><<<dim3(s.B * s.nc * s.H), dim3(64 * PB * NB), lds, st>>>(
        static_cast<const T *>(x), static_cast<const T *>(Bm), dtcs, states, s);
    return hipGetLastError();
}

template <typename T, int PB>
static hipError_t state_dispatch_n(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                                   float *states, hipStream_t st) {
    switch ((s.N + 31) / 32) {
        case 1: return state_launch<T, PB, 1>(s, x, Bm, dtcs, states, st);
        case 2: return state_launch<T, PB, 2>(s, x, Bm, dtcs, states, st);
        case 4: return state_launch<T, PB, 4>(s, x, Bm, dtcs, states, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T>
static hipError_t state_dispatch(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                                 float *states, hipStream_t st) {
    return (s.P <= 32) ? state_dispatch_n<T, 1>(s, x, Bm, dtcs, states, st)
                       : state_dispatch_n<T, 2>(s, x, Bm, dtcs, states, st);
}

hipError_t launch_chunk_state(const ScanShape &s, int dtype, const void *x, const void *Bm, const float *dtcs,
                              float *states, hipStream_t st) {
    return dtype ? state_dispatch<__bf16>(s, x, Bm, dtcs, states, st)
                 : state_dispatch<float>(s, x, Bm, dtcs, states, st);
}

hipError_t launch_state_passing(const ScanShape &s, const float *states, const float *dtcs, const float *init,
                                float *prev, float *final_states, hipStream_t st) {
    const long long total = (long long)s.B * s.H * (s.P * s.N / 4);
    const unsigned blocks = (unsigned)((total + 255) / 256);
    state_passing_kernel<<<dim3(blocks), dim3(256), 0, st>>>(states, dtcs, init, prev, final_states, s, total);
    return hipGetLastError();
}

template <typename T, typename TO, int PB, int NK>
static hipError_t scan_launch(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                              const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    const size_t lds = chunk_scan_lds_bytes(s, sizeof(T));
    hipError_t e = allow_lds(chunk_scan_kernel<T, TO, PB, NK>, lds);
    if (e != hipSuccess) return e;
    chunk_scan_kernel<T, TO, PB, NK><<<dim3(s.B * s.nc * s.H), dim3(64 * (s.Q / 32)), lds, st>>>(
        static_cast<const T *>(x), static_cast<const T *>(Bm), static_cast<const T *>(Cm), dtcs, prev, D,
        static_cast<TO *>(y), s);
    return hipGetLastError();
}

template <typename T, typename TO, int PB>
static hipError_t scan_dispatch_n(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                                  const float *dtcs, const float *prev, const float *D, void *y,
                                  hipStream_t st) {
    switch (s.N) {
        case 16: return scan_launch<T, TO, PB, 1>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 32: return scan_launch<T, TO, PB, 2>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 64: return scan_launch<T, TO, PB, 4>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 128: return scan_launch<T, TO, PB, 8>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T, typename TO>
static hipError_t scan_dispatch(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                                const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    return (s.P <= 32) ? scan_dispatch_n<T, TO, 1>(s, x, Bm, Cm, dtcs, prev, D, y, st)
                       : scan_dispatch_n<T, TO, 2>(s, x, Bm, Cm, dtcs, prev, D, y, st);
}

hipError_t launch_chunk_scan(const ScanShape &s, int dtype, const void *x, const void *Bm, const void *Cm,
                             const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    switch (dtype) {
        case 0: return scan_dispatch<float, float>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 1: return scan_dispatch<__bf16, __bf16>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        default: return scan_dispatch<__bf16, float>(s, x, Bm, Cm, dtcs, prev, D, y, st);
    }
}

template <typename T, typename TO>
static hipError_t step_dispatch(const StepShape &s, float *state, const void *x, const void *dt,
                                const float *A, const void *Bm, const void *Cm, const float *D, void *y,
                                hipStream_t st) {
    const long long pairs = (long long)s.B * s.H;
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

}  // namespace ssd
