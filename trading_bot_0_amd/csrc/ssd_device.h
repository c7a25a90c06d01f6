// Device-side building blocks shared by the SSD kernels (gfx950 only): MFMA fragments, 16-byte
// vectors, hi/lo bf16 splitting, row-major LDS tiles read through the transpose load, the
// XCD-aware persistent tile schedule.
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
#pragma once
#include <atomic>
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

// A reset before step t (the state restarts from zero there) is a drop of the cumulative log2-decay by
// kResetLog2 at t: every decay factor that spans the reset becomes exp2(-16384 or less) = 0 and everything
// on one side of it is unchanged, since only differences of alpha are ever used.  In the natural-log units
// of the float64 scan that is kResetDrop per reset.  (Up to 256 resets per chunk keep |alpha| below 2^22,
// where the hi + lo float pair still resolves differences to 1e-8.)
constexpr double kResetLog2 = 16384.0;
constexpr double kResetDrop = kResetLog2 / 1.4426950408889634;

// ------------------------------------------------------------------------------------------
// Wavefront inclusive scan in float64 (DPP data movement)
// ------------------------------------------------------------------------------------------
template <int CTRL, int ROWMASK> __device__ inline double dpp_move(double v) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    // With every row enabled the hardware's own zero for a lane without a source (bound_ctrl) does what the zero
    // "old" value does, and the destination needs no clearing first (two moves per step less).
    constexpr bool kBound = ROWMASK == 0xf;
    lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROWMASK, 0xf, kBound);
    hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROWMASK, 0xf, kBound);
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

// Sum of v over aligned groups of NL consecutive lanes (NL = 4, 8, 16, 32 or 64), left in every lane of the group.
// Inside a row of 16 lanes the data moves by DPP (quads, then the mirrored half row, then the mirrored row: no trip
// through the LDS crossbar); wider groups take one lane exchange per doubling on top.
template <int CTRL> __device__ inline float dpp_move_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int NL> __device__ inline float group_sum(float v) {
    static_assert(NL == 4 || NL == 8 || NL == 16 || NL == 32 || NL == 64, "groups of 4, 8, 16, 32 or 64 lanes");
    v += dpp_move_f<0xB1>(v);                           // quad_perm [1,0,3,2]
    v += dpp_move_f<0x4E>(v);                           // quad_perm [2,3,0,1]
    if constexpr (NL >= 8) v += dpp_move_f<0x141>(v);   // row_half_mirror: lane i <-> 7 - i of its half row
    if constexpr (NL >= 16) v += dpp_move_f<0x140>(v);  // row_mirror: lane i <-> 15 - i of its row
    if constexpr (NL >= 32) v += __shfl_xor(v, 16, 64);
    if constexpr (NL >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// The value lane u (0..7) of this lane's aligned group of NL lanes holds.  A group that is a whole row of 16 lanes
// takes it by DPP (row_newbcast: lane u of every row to all of the row), any other by a lane exchange.
template <int NL> __device__ inline float group_lane(float v, int u) {
    if constexpr (NL == 16) {
        switch (u) {  // u is a constant after unrolling
            case 0: return dpp_move_f<0x150>(v);
            case 1: return dpp_move_f<0x151>(v);
            case 2: return dpp_move_f<0x152>(v);
            case 3: return dpp_move_f<0x153>(v);
            case 4: return dpp_move_f<0x154>(v);
            case 5: return dpp_move_f<0x155>(v);
            case 6: return dpp_move_f<0x156>(v);
            default: return dpp_move_f<0x157>(v);
        }
    } else {
        return __shfl(v, (int)(threadIdx.x & 63) / NL * NL + u, 64);
    }
}

// ------------------------------------------------------------------------------------------
// Output columns of a transposed 32x32 accumulator tile, stored 16 bytes at a time
// ------------------------------------------------------------------------------------------
__device__ inline void swap_halves(unsigned &x, unsigned &y) {
    // x[lanes 32..63] <-> y[lanes 0..31]
    const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
    x = r[0];
    y = r[1];
}
__device__ inline unsigned pack_bf16x2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 v;
    v[0] = (__bf16)a;
    v[1] = (__bf16)b;
    return __builtin_bit_cast(unsigned, v);
}

// One output column block of 32 head-dim values per lane pair: o[v] is element
// p = 8*(v/4) + 4*half + v%4 of column l.  Writes p = 16*half .. 16*half+15 of row `yrow`
// (yrow already points at the column's row and at head-dim offset 32*pb).
template <typename TO> __device__ inline void store_column(TO *yrow, float (&o)[16], int half, int pvalid, bool row_ok);
template <> __device__ inline void store_column<__bf16>(__bf16 *yrow, float (&o)[16], int half, int pvalid, bool row_ok) {
    unsigned X[4], Y[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        X[k] = pack_bf16x2(o[2 * k], o[2 * k + 1]);          // p-groups 0 and 1 (v = 0..7)
        Y[k] = pack_bf16x2(o[8 + 2 * k], o[8 + 2 * k + 1]);  // p-groups 2 and 3 (v = 8..15)
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) swap_halves(X[k], Y[k]);
    if (row_ok) {
        const int p0 = 16 * half;
        if (p0 + 8 <= pvalid) *reinterpret_cast<uint4 *>(yrow + p0) = make_uint4(X[0], X[1], Y[0], Y[1]);
        if (p0 + 16 <= pvalid) *reinterpret_cast<uint4 *>(yrow + p0 + 8) = make_uint4(X[2], X[3], Y[2], Y[3]);
    }
}
template <> __device__ inline void store_column<float>(float *yrow, float (&o)[16], int half, int pvalid, bool row_ok) {
    unsigned X[8], Y[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        X[k] = __float_as_uint(o[k]);
        Y[k] = __float_as_uint(o[8 + k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) swap_halves(X[k], Y[k]);
    if (row_ok) {
        const int p0 = 16 * half;
        if (p0 + 4 <= pvalid) *reinterpret_cast<uint4 *>(yrow + p0) = make_uint4(X[0], X[1], X[2], X[3]);
        if (p0 + 8 <= pvalid) *reinterpret_cast<uint4 *>(yrow + p0 + 4) = make_uint4(Y[0], Y[1], Y[2], Y[3]);
        if (p0 + 12 <= pvalid) *reinterpret_cast<uint4 *>(yrow + p0 + 8) = make_uint4(X[4], X[5], X[6], X[7]);
        if (p0 + 16 <= pvalid) *reinterpret_cast<uint4 *>(yrow + p0 + 12) = make_uint4(Y[4], Y[5], Y[6], Y[7]);
    }
}

// The same through a buffer descriptor: rows that must not be written get an offset beyond the descriptor's range
// and the hardware drops their stores, so the stores themselves are unconditional -- no branch around them.
// byte_off addresses element p = 0 of the column's row, relative to the descriptor's base; all offsets of a
// descriptor stay below 2^31.
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
constexpr unsigned kBufferDropOffset = 0x80000000u;
__device__ inline __amdgpu_buffer_rsrc_t make_buffer(const void *base, unsigned bytes) {
    // raw buffer, stride 0, range-checked: dword 3 = the 32-bit data format of gfx9-family descriptors
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
// One column's 32 outputs packed for the store, and where they go.
template <typename TO> struct PackedColumn {
    static constexpr int NV = sizeof(TO) == 2 ? 2 : 4;
    u32x4 v[NV];
    unsigned off = kBufferDropOffset;  // (nothing packed yet: emitting it writes nothing)
};
template <typename TO>
__device__ inline void pack_column(PackedColumn<TO> &pc, unsigned byte_off, float (&o)[16], int half, bool row_ok);
template <>
__device__ inline void pack_column<__bf16>(PackedColumn<__bf16> &pc, unsigned byte_off, float (&o)[16], int half, bool row_ok) {
    unsigned X[4], Y[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        X[k] = pack_bf16x2(o[2 * k], o[2 * k + 1]);
        Y[k] = pack_bf16x2(o[8 + 2 * k], o[8 + 2 * k + 1]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) swap_halves(X[k], Y[k]);
    pc.off = row_ok ? byte_off + 32u * half : kBufferDropOffset;
    pc.v[0] = u32x4{X[0], X[1], Y[0], Y[1]};
    pc.v[1] = u32x4{X[2], X[3], Y[2], Y[3]};
}
template <>
__device__ inline void pack_column<float>(PackedColumn<float> &pc, unsigned byte_off, float (&o)[16], int half, bool row_ok) {
    unsigned X[8], Y[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        X[k] = __float_as_uint(o[k]);
        Y[k] = __float_as_uint(o[8 + k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) swap_halves(X[k], Y[k]);
    pc.off = row_ok ? byte_off + 64u * half : kBufferDropOffset;
    pc.v[0] = u32x4{X[0], X[1], X[2], X[3]};
    pc.v[1] = u32x4{Y[0], Y[1], Y[2], Y[3]};
    pc.v[2] = u32x4{X[4], X[5], X[6], X[7]};
    pc.v[3] = u32x4{Y[4], Y[5], Y[6], Y[7]};
}
template <typename TO> __device__ inline void emit_column(__amdgpu_buffer_rsrc_t rs, const PackedColumn<TO> &pc) {
#pragma unroll
    for (int i = 0; i < PackedColumn<TO>::NV; ++i) __builtin_amdgcn_raw_buffer_store_b128(pc.v[i], rs, pc.off + 16u * i, 0, 0);
}
template <typename TO>
__device__ inline void store_column_buffer(__amdgpu_buffer_rsrc_t rs, unsigned byte_off, float (&o)[16], int half, bool row_ok) {
    PackedColumn<TO> pc;
    pack_column<TO>(pc, byte_off, o, half, row_ok);
    emit_column<TO>(rs, pc);
}

// hi + lo bf16 pairs of two products a0*f0 and a1*f1 (f = 1 to split plain values): hi is the product
// rounded to bf16, lo the rounded remainder m - hi, which is exact in float before its own rounding.
// The remainder takes one v_dot2c_f32_bf16 per element, m + (-1)*half + 0*other half, which reads the half
// straight out of the packed pair.  Three VALU instructions per element: multiply, half a pack, dot2c, half
// a pack.  The selectors are kept out of the compiler's sight: it would encode the pair (-1, 0) as the
// inline constant -1.0, which the instruction reads as the pair (0, -1).
__device__ inline void split_pair(float a0, float f0, float a1, float f1, unsigned &hi, unsigned &lo) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    unsigned first = 0x0000bf80u, second = 0xbf800000u;
    asm("" : "+s"(first));
    asm("" : "+s"(second));
    const float m0 = a0 * f0, m1 = a1 * f1;
    hi = pack_bf16x2(m0, m1);
    const bf16x2 h = __builtin_bit_cast(bf16x2, hi);
    lo = pack_bf16x2(__builtin_amdgcn_fdot2_f32_bf16(h, __builtin_bit_cast(bf16x2, first), m0, false),
                     __builtin_amdgcn_fdot2_f32_bf16(h, __builtin_bit_cast(bf16x2, second), m1, false));
}
// The same split of eight plain values that stay live afterwards (the running state), as one operand fragment pair.
// The three-operand form of the dot product writes the remainder to a register of its own, where the two-operand form
// above accumulates in place and the compiler has to copy each value first (two moves per pair).  The compiler does not
// select that form, so it is written out; and since it does not look inside such a block, the wait the hardware needs
// between a dot product and the next instruction that reads its result (three wait states, which the compiler inserts
// by itself behind the two-operand form) stands at the end of the block, behind eight independent products.
__device__ inline void split8_keep(const float (&a)[8], unsigned (&hi)[4], unsigned (&lo)[4]) {
    unsigned first = 0x0000bf80u, second = 0xbf800000u;
    asm("" : "+s"(first));
    asm("" : "+s"(second));
#pragma unroll
    for (int k = 0; k < 4; ++k) hi[k] = pack_bf16x2(a[2 * k], a[2 * k + 1]);
    float l0, l1, l2, l3, l4, l5, l6, l7;
    asm("v_dot2_f32_bf16 %0, %8, %12, %14\n\t"
        "v_dot2_f32_bf16 %1, %8, %13, %15\n\t"
        "v_dot2_f32_bf16 %2, %9, %12, %16\n\t"
        "v_dot2_f32_bf16 %3, %9, %13, %17\n\t"
        "v_dot2_f32_bf16 %4, %10, %12, %18\n\t"
        "v_dot2_f32_bf16 %5, %10, %13, %19\n\t"
        "v_dot2_f32_bf16 %6, %11, %12, %20\n\t"
        "v_dot2_f32_bf16 %7, %11, %13, %21\n\t"
        "s_nop 2"
        : "=&v"(l0), "=&v"(l1), "=&v"(l2), "=&v"(l3), "=&v"(l4), "=&v"(l5), "=&v"(l6), "=&v"(l7)
        : "v"(hi[0]), "v"(hi[1]), "v"(hi[2]), "v"(hi[3]), "s"(first), "s"(second), "v"(a[0]), "v"(a[1]), "v"(a[2]),
          "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]));
    lo[0] = pack_bf16x2(l0, l1);
    lo[1] = pack_bf16x2(l2, l3);
    lo[2] = pack_bf16x2(l4, l5);
    lo[3] = pack_bf16x2(l6, l7);
}
struct FragBits {  // an operand fragment as four packed pairs
    unsigned u[4];
    __device__ inline Frag<__bf16> frag() const {
        typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
        u32x4 v = {u[0], u[1], u[2], u[3]};
        Frag<__bf16> f;
        f.v = __builtin_bit_cast(bf16x8, v);
        return f;
    }
};

// Operand fragments of eight products a[i]*f[i]: a hi + lo pair in bf16 mode, the products themselves in
// float mode (lo is then unused).
template <typename T> struct ProductFrags;
template <> struct ProductFrags<__bf16> {
    static __device__ inline void make(const float (&a)[8], const float (&f)[8], Frag<__bf16> &hi, Frag<__bf16> &lo) {
        FragBits fh, fl;
#pragma unroll
        for (int k = 0; k < 4; ++k) split_pair(a[2 * k], f[2 * k], a[2 * k + 1], f[2 * k + 1], fh.u[k], fl.u[k]);
        hi = fh.frag();
        lo = fl.frag();
    }
};
template <> struct ProductFrags<float> {
    static __device__ inline void make(const float (&a)[8], const float (&f)[8], Frag<float> &hi, Frag<float> &) {
#pragma unroll
        for (int i = 0; i < 8; ++i) hi.v[i] = a[i] * f[i];
    }
};

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory, and
// on gfx9 loads and stores share one counter, so it drains every outstanding global load -- among
// them the next tile's prefetch, which must stay in flight across the barrier.  The tile loops
// share nothing through global memory inside a launch, so waiting for LDS (and scalar) operations
// is all the barrier needs.
__device__ inline void block_sync_lds() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Workgroups are dealt round-robin to the 8 XCDs, each with a private L2.  Re-number them so
// that consecutive logical ids (the heads of one (b,c) tile, which share B and C and sit in
// the same cache lines of x) land on the same XCD at nearly the same time.
__device__ inline int xcd_remap(int bid, int total) {
    return (total % 8 == 0) ? (bid % 8) * (total / 8) + bid / 8 : bid;
}

// ------------------------------------------------------------------------------------------
// Persistent tile schedule of stages 2 and 4.  The grid holds as many workgroups as the chip
// keeps resident; each walks a fixed list of (b,c,h) tiles and fetches the next tile's inputs
// into registers while it computes the current one, so HBM requests stay in flight through
// the MFMA phase (with one tile per workgroup and ~4 workgroups per CU the chip alternated
// between loading and computing and sat at a third of the HBM rate).
// Workgroup j runs on XCD j%8; the list is cut so that at any moment the workgroups of one
// XCD work on consecutive logical tiles, i.e. on the heads of the same (b,c).  No workgroup
// ever waits on another: the loop bounds are fixed at launch.
// ------------------------------------------------------------------------------------------
struct TileSched {
    int base, pos, step, per;
    __device__ explicit TileSched(int total) {
        if (total % 8 == 0 && gridDim.x % 8 == 0) {
            per = total / 8;
            base = (int)(blockIdx.x % 8) * per;
            pos = blockIdx.x / 8;
            step = gridDim.x / 8;
        } else {
            per = total;
            base = 0;
            pos = blockIdx.x;
            step = gridDim.x;
        }
    }
    __device__ bool valid() const { return pos < per; }
    __device__ bool has_next() const { return pos + step < per; }
    __device__ int logical() const { return base + pos; }
    __device__ int next_logical() const { return base + pos + step; }
    __device__ void advance() { pos += step; }
};

struct Tile {
    int b, c, h, g, t0;
};
__device__ inline Tile decode_tile(int logical, const ScanShape &s) {
    Tile t;
    t.h = logical % s.H;
    t.c = (logical / s.H) % s.nc;
    t.b = logical / (s.H * s.nc);
    t.g = t.h / (s.H / s.G);
    t.t0 = t.c * s.Q;
    return t;
}


// ------------------------------------------------------------------------------------------
// Per-(kernel, device, launch configuration) facts the launchers need on every call -- the resident workgroups
// per CU, whether the kernel's dynamic LDS limit has been raised -- are asked of the runtime once and kept in a
// small table.  The entry points are re-entrant, so the table is lock-free: a slot is claimed by a compare-and-swap
// on the kernel's address, filled, then published with a release store; a reader that finds a slot claimed but not
// yet published (or the table full) asks the runtime itself.  One table per translation unit.
// ------------------------------------------------------------------------------------------
struct LaunchFacts {
    static constexpr int kSlots = 256;
    struct Slot {
        std::atomic<uintptr_t> kernel{0};
        std::atomic<uint64_t> config{0};
        std::atomic<int> value{0};
        std::atomic<int> ready{0};
    };
    Slot slots[kSlots];
    // value kept for (kernel, config), or -1
    int find(const void *kernel, uint64_t config) const {
        const uintptr_t k = reinterpret_cast<uintptr_t>(kernel);
        for (int i = 0, at = (int)((k >> 4) % kSlots); i < kSlots; ++i, at = (at + 1) % kSlots) {
            const uintptr_t have = slots[at].kernel.load(std::memory_order_acquire);
            if (have == 0) return -1;
            if (have == k && slots[at].ready.load(std::memory_order_acquire) &&
                slots[at].config.load(std::memory_order_relaxed) == config)
                return slots[at].value.load(std::memory_order_relaxed);
        }
        return -1;
    }
    void keep(const void *kernel, uint64_t config, int value) {
        const uintptr_t k = reinterpret_cast<uintptr_t>(kernel);
        for (int i = 0, at = (int)((k >> 4) % kSlots); i < kSlots; ++i, at = (at + 1) % kSlots) {
            uintptr_t empty = 0;
            if (slots[at].kernel.compare_exchange_strong(empty, k, std::memory_order_acq_rel)) {
                slots[at].config.store(config, std::memory_order_relaxed);
                slots[at].value.store(value, std::memory_order_relaxed);
                slots[at].ready.store(1, std::memory_order_release);
                return;
            }
        }
    }
};
static inline LaunchFacts &launch_facts() {
    static LaunchFacts facts;
    return facts;
}
static inline uint64_t launch_config_key(int kind, int dev, int block, size_t lds) {
    return ((uint64_t)kind << 60) | ((uint64_t)(dev & 0xff) << 48) | ((uint64_t)(block & 0xffff) << 32) | (uint64_t)(lds & 0xffffffffu);
}
static inline hipError_t device_cu_count(int dev, int *cus) {
    static std::atomic<int> known[64];
    if (dev >= 0 && dev < 64) {
        const int have = known[dev].load(std::memory_order_relaxed);
        if (have > 0) {
            *cus = have;
            return hipSuccess;
        }
    }
    hipError_t e = hipDeviceGetAttribute(cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess && dev >= 0 && dev < 64) known[dev].store(*cus, std::memory_order_relaxed);
    return e;
}

// Workgroups of a persistent kernel: as many as stay resident on the current device, in whole
// multiples of the 8 XCDs, never more than there are tiles.
template <typename K>
static inline hipError_t persistent_grid(K kernel, int block, size_t lds, int tiles, int *grid) {
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = device_cu_count(dev, &cus);
    if (e != hipSuccess) return e;
    const void *kp = reinterpret_cast<const void *>(kernel);
    const uint64_t key = launch_config_key(1, dev, block, lds);
    int per_cu = launch_facts().find(kp, key);
    if (per_cu < 0) {
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block, lds);
        if (e != hipSuccess) return e;
        // The occupancy query counts a workgroup whose LDS fills the CU to the last byte; measured, that
        // one does not become resident, and a persistent grid larger than residency runs a second round.
        if (lds > 0) {
            const int by_lds = (int)(kLdsLimitBytes / (lds + 1024));
            if (per_cu > by_lds) per_cu = by_lds;
        }
        if (per_cu < 1) per_cu = 1;
        launch_facts().keep(kp, key, per_cu);
    }
    long long g = (long long)cus * per_cu;
    if (g > tiles) g = tiles;
    if (g >= 8) g -= g % 8;
    *grid = (int)(g < 1 ? 1 : g);
    return hipSuccess;
}

// Raises a kernel's dynamic LDS limit (needed above 64 KiB) to the CU's whole LDS, once per kernel and device.  The
// attribute holds the last value set, so a limit set per size would be left at a smaller size by a later call that
// found its own size already noted; the CU's limit serves every size a launcher can ask for.
template <typename K> static inline hipError_t allow_lds(K kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return hipSuccess;
    if (bytes > kLdsLimitBytes) return hipErrorInvalidValue;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const void *kp = reinterpret_cast<const void *>(kernel);
    const uint64_t key = launch_config_key(2, dev, 0, 0);
    if (launch_facts().find(kp, key) == 1) return hipSuccess;
    e = hipFuncSetAttribute(kp, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimitBytes);
    if (e == hipSuccess) launch_facts().keep(kp, key, 1);
    return e;
}

}  // namespace ssd
