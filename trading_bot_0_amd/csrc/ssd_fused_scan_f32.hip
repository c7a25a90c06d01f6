// One-pass forward for float32 inputs (gfx950).
//
// The same decomposition as the bf16 one-pass kernel (ssd_fused_scan.h): a wave owns 32 head-dim columns of one
// head of one batch row for the whole sequence, the running state stays in MFMA accumulators, the eight waves of
// a workgroup share the tile's B and C in LDS; nothing but x, dt, B, C is read and nothing but y and the final
// state written.  What differs is how float operands reach the matrix cores.  gfx950 multiplies floats at a
// sixteenth of its bf16 rate (v_mfma_f32_32x32x2_f32: 64 cycles for K = 2), so every operand is split into three
// bf16 terms h + m + l (8 + 8 + 8 significant bits: the float exactly, up to its last bit) and a product a.b is
// the six term products of weight 2^-16 and above,
//     a_h b_h + a_h b_m + a_m b_h + a_h b_l + a_l b_h + a_m b_m,
// each one v_mfma_f32_32x32x16_bf16 accumulating in float: 192 matrix-pipe cycles per K = 16 instead of 512, and a
// relative error of a few 2^-24 like the float instruction's own.  x, B and C are split once per tile, when the
// registers holding the global loads are written to LDS (three bf16 tiles each, the layout of the bf16 kernel's
// tiles, so the transposing reads apply); the operands the kernel manufactures (the state, the masked decayed
// scores, the weighted x) are split in registers where they are formed.  The weighted x needs float x, which the
// transposing read cannot deliver: a fourth, float tile of x serves phase 2 and the D.x term of the epilogue.
//
// Time is tiled by 32 steps: every tile is one diagonal block (84 MFMAs per tile against 204 per 64 steps with
// tiles of 64, where the matrix pipe is what binds), and the four x tiles fit in LDS.
#include "ssd_fused_scan.h"

namespace ssd {

namespace {

constexpr int kFloatTile = 32;
// log2-decay across a tile up to which the separable factors E[l] F[s] are used: each is exp2 of an argument as
// large as the span, rounded to float, so their product is off by about 2^-24 span ln 2
constexpr float kFloatFastSpan = 4.f;

constexpr int f32_xterm_elems() { return kFloatTile * 32 + 32; }  // bf16 elements per unit of an x term region
constexpr int f32_xfloat_elems() { return kFloatTile * 32 + 16; }  // floats per unit of the float x region
constexpr int f32_table_floats() { return 6 * kFloatTile + 16; }
// bf16 elements from one term tile of B (or C) to the next: 16 bytes more than the tile, so that no two-address
// LDS read (whose two offsets are multiples of 512 bytes) reaches from one term into another -- the compiler
// would pair reads of different terms that way and then move the halves of every fragment into place
constexpr int f32_bcterm_elems(int N) { return kFloatTile * N + 8; }
// ... and the tile's scores B . C^T, which the workgroup's eight units share (one group's B and C), as two partial
// sums over half of the state dimension each, in the accumulator's layout ([half][quarter][lane] 16 bytes)
constexpr size_t fused_scan_f32_lds_bytes(int N, int waves) {
    return (size_t)2 * 3 * f32_bcterm_elems(N) * 2 + (size_t)waves * 3 * f32_xterm_elems() * 2 +
           (size_t)waves * f32_xfloat_elems() * 4 + (size_t)waves * f32_table_floats() * 4 + (size_t)2 * 32 * 32 * 4;
}

// Where unit u's tiles start inside their regions (waves * f32_xterm_elems() bf16 elements per term, waves *
// f32_xfloat_elems() floats): a staging write hits one row and all eight 8-byte pieces (term tiles), or every other
// one (float tile), of several units' tiles at once; these offsets spread the 16 (or 32) lanes served together over
// 128 (256) bytes of banks (the offsets grow with u, so the tiles do not overlap).
__device__ inline int f32_xterm_base(int u) { return u * (kFloatTile * 32) + (u & 3) * 32 + (u >> 2) * 128; }
__device__ inline int f32_xfloat_base(int u) { return u * (kFloatTile * 32) + (u & 1) * 2 + ((u >> 1) & 1) * 32 + (u >> 2) * 64; }

// float x tile [32][32]: the 8-byte pieces of a row XOR-swizzled with the row's low four bits, so that 8-byte reads
// of one column pair of 16 consecutive rows, 4-byte reads along a row and the staging writes all spread over the
// banks
__device__ inline int xfloat_off(int row, int col) { return row * 32 + ((((col >> 1) ^ (row & 15))) << 1) + (col & 1); }

// three bf16 terms of two floats, packed per term: h = bf16(m), m = bf16(m - h), l = bf16(m - h - m); the
// remainders are exact in float (one v_dot2c_f32_bf16 each, see split_pair)
__device__ inline void split3_pair(float m0, float m1, unsigned &h, unsigned &m, unsigned &l) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    unsigned first = 0x0000bf80u, second = 0xbf800000u;
    asm("" : "+s"(first));
    asm("" : "+s"(second));
    const bf16x2 sf = __builtin_bit_cast(bf16x2, first), ss = __builtin_bit_cast(bf16x2, second);
    h = pack_bf16x2(m0, m1);
    const bf16x2 hb = __builtin_bit_cast(bf16x2, h);
    const float r0 = __builtin_amdgcn_fdot2_f32_bf16(hb, sf, m0, false);
    const float r1 = __builtin_amdgcn_fdot2_f32_bf16(hb, ss, m1, false);
    m = pack_bf16x2(r0, r1);
    const bf16x2 mb = __builtin_bit_cast(bf16x2, m);
    l = pack_bf16x2(__builtin_amdgcn_fdot2_f32_bf16(mb, sf, r0, false), __builtin_amdgcn_fdot2_f32_bf16(mb, ss, r1, false));
}

struct Frag3 {  // an operand fragment as three terms
    Frag<__bf16> t[3];
};
struct Bits3 {
    FragBits t[3];
    __device__ inline Frag3 frags() const {
        Frag3 f;
        f.t[0] = t[0].frag();
        f.t[1] = t[1].frag();
        f.t[2] = t[2].frag();
        return f;
    }
};

// c += a . b to float precision; the small products first
__device__ inline f32x16 mma6(const Frag3 &a, const Frag3 &b, f32x16 c) {
    c = mma32(a.t[2], b.t[0], c);
    c = mma32(a.t[0], b.t[2], c);
    c = mma32(a.t[1], b.t[1], c);
    c = mma32(a.t[1], b.t[0], c);
    c = mma32(a.t[0], b.t[1], c);
    c = mma32(a.t[0], b.t[0], c);
    return c;
}

// STATES_ONLY: no outputs, no C: the state a segment of the sequence leaves behind from a zero state, into
// final_states [B, segments, H, P, N], and the segment's total decay into seg_decay [B, segments, H] -- for sequences
// cut into segments of s.seg_tiles tiles (of 32 steps here) that different workgroups walk side by side.  The
// forward on segments (s.seg_local set) starts every segment from the recurrence over those states, run in its
// workgroups' prologue, as in the bf16 kernel.
template <int NK, int WAVES, bool STATES_ONLY>  // dstate N = 16 NK
__global__ __launch_bounds__(64 * WAVES, 1) void fused_scan_f32_kernel(
    const float *__restrict__ x, const float *__restrict__ dt, const float *__restrict__ A, const float *__restrict__ Bm,
    const float *__restrict__ Cm, const float *__restrict__ D, const float *init, const unsigned char *__restrict__ reset,
    float *__restrict__ y, float *final_states, float *seg_decay, ScanShape s) {
    using T = __bf16;
    constexpr int N = 16 * NK, NB = NK / 2, Q = kFloatTile, nthr = 64 * WAVES;
    constexpr int XS = f32_xterm_elems(), XF = f32_xfloat_elems(), TB = f32_bcterm_elems(N), WF = f32_table_floats();
    constexpr int XPR = WAVES * 8;         // 16-byte pieces (4 floats) of one timestep's x for the workgroup
    constexpr int XROWS = nthr / XPR;      // x rows per pass
    constexpr int UX = Q / XROWS;          // passes
    constexpr int BPR = N / 4;             // 16-byte pieces per B (or C) row
    static_assert(Q * BPR <= nthr && Q % XROWS == 0, "one pass of B and C, whole passes of x");
    using XT = ChunkTile<32>;
    using BT = ChunkTile<N>;
    __shared__ __attribute__((aligned(16))) unsigned char smem[fused_scan_f32_lds_bytes(N, WAVES)];
    const int tid = threadIdx.x;
    const int lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    T *Bs = reinterpret_cast<T *>(smem);   // [3][Q][N]
    T *Cs = Bs + 3 * TB;                   // [3][Q][N]
    T *xt_all = Cs + 3 * TB;               // [3][WAVES][XS]
    float *xf_all = reinterpret_cast<float *>(xt_all + 3 * WAVES * XS);  // [WAVES][XF]
    float *wf = xf_all + WAVES * XF + wave * WF;
    float *const G_s = xf_all + WAVES * XF + WAVES * WF;  // [2][4][64][4] floats
    T *xt = xt_all + f32_xterm_base(wave);  // term t of this wave's unit: xt + t * WAVES * XS
    float *xf = xf_all + f32_xfloat_base(wave);
    float *ah_s = wf, *alo_s = wf + Q, *dt_s = wf + 2 * Q, *w_s = wf + 3 * Q, *E_s = wf + 4 * Q, *F_s = wf + 5 * Q;

    // ---- which units this workgroup owns (as the bf16 kernel) ----
    const int PBn = s.P / 32, HG = s.H / s.G;
    const int UW = (HG * PBn) / WAVES;
    const int nc = (s.L + Q - 1) / Q;
    const int S = s.seg_tiles > 0 ? (nc + s.seg_tiles - 1) / s.seg_tiles : 1;
    const int slot = xcd_remap(blockIdx.x, gridDim.x);
    const int seg = slot % S, logical = slot / S;
    // states only: nothing comes after the last segment, its workgroups leave at once
    if (STATES_ONLY && S > 1 && seg == S - 1) return;
    const int c_first = seg * (s.seg_tiles > 0 ? s.seg_tiles : nc);
    const int c_end = s.seg_tiles > 0 ? min(nc, c_first + s.seg_tiles) : nc;
    const int b = logical / (s.G * UW), g = (logical / UW) % s.G, unit0 = (logical % UW) * WAVES;
    const int unit = unit0 + wave, h = g * HG + unit / PBn, pb = unit % PBn;
    const int HP = s.H * s.P;
    const float *xb = x + (size_t)b * s.L * HP + g * HG * s.P + unit0 * 32;
    const float *Bb = Bm + ((size_t)b * s.L * s.G + g) * N, *Cb = Cm + ((size_t)b * s.L * s.G + g) * N;
    const float *dtb = dt + (size_t)b * s.L * s.H + h;
    const unsigned char *rsb = reset ? reset + (size_t)b * s.L : nullptr;
    const __amdgpu_buffer_rsrc_t ybuf = make_buffer(y + (size_t)b * s.L * HP, (unsigned)((size_t)s.L * HP * sizeof(float)));
    const unsigned ycol_bytes = (unsigned)((h * s.P + pb * 32) * sizeof(float));
    const float dh = D ? D[h] : 0.f;
    const double a_h = (double)A[h];

    // ---- registers holding the next tile's inputs ----
    float4 xq[UX], bq, cq;
    float dq;
    unsigned char rq;
    const int x_row0 = tid / XPR, x_pc = tid % XPR, bc_row = tid / BPR, bc_pc = tid % BPR;
    const bool bc_thread = tid < Q * BPR;
    auto prefetch = [&](int c) {
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
        bq = zero;
        cq = zero;
        if (bc_thread && bc_row < rows) {
            const size_t o = (size_t)(t0 + bc_row) * s.G * N + bc_pc * 4;
            bq = *reinterpret_cast<const float4 *>(Bb + o);
            if (!STATES_ONLY) cq = *reinterpret_cast<const float4 *>(Cb + o);
        }
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            xq[u] = zero;
            if (x_row0 + u * XROWS < rows) xq[u] = *reinterpret_cast<const float4 *>(xb + (size_t)(t0 + x_row0 + u * XROWS) * HP + x_pc * 4);
        }
        dq = 0.f;
        rq = 0;
        if (lane < rows) {  // rows <= 32: the upper half of the wave holds no step
            dq = dtb[(size_t)(t0 + lane) * s.H];
            if (rsb != nullptr) rq = rsb[t0 + lane];
        }
    };

    // ---- running state: st[nb][v] = H[p = r, n = 32 nb + 8 (v/4) + 4 half + v%4] ----
    f32x16 st[NB];
    {
        const bool folded = !STATES_ONLY && s.seg_local != nullptr;
        const bool fresh = rsb != nullptr && rsb[0] != 0;  // a restart before the first step: init is not read
        const size_t lane_off = (size_t)(pb * 32 + r) * N + 4 * half;
        const float *ib = !STATES_ONLY && init && !fresh ? init + ((size_t)b * s.H + h) * s.P * N + lane_off : nullptr;
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
        if (folded) {  // enter[j+1] = decay[j] * enter[j] + local[j] over the segments before this one
            for (int j = 0; j < seg; ++j) {
                const float a = s.seg_local_decay[((size_t)b * S + j) * s.H + h];
                const float *lb = s.seg_local + (((size_t)b * S + j) * s.H + h) * s.P * N + lane_off;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq) {
                        const float4 v = *reinterpret_cast<const float4 *>(lb + 32 * nb + 8 * gq);
                        st[nb][4 * gq + 0] = a * st[nb][4 * gq + 0] + v.x;
                        st[nb][4 * gq + 1] = a * st[nb][4 * gq + 1] + v.y;
                        st[nb][4 * gq + 2] = a * st[nb][4 * gq + 2] + v.z;
                        st[nb][4 * gq + 3] = a * st[nb][4 * gq + 3] + v.w;
                    }
                }
            }
        }
    }
    float seg_total = 1.f;  // product of the tiles' decays (states only)

    // where this thread's staged pieces go: 4 floats = one 8-byte piece of each term tile
    const int x_unit = x_pc / 8, x_col = (x_pc % 8) * 4;
    prefetch(c_first);
    for (int c = c_first; c < c_end; ++c) {
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        block_sync_lds();  // every wave is done reading the previous tile
        // ---- registers -> LDS: three bf16 terms of x, B and C, and x as floats ----
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            const int row = x_row0 + u * XROWS;
            if (!STATES_ONLY) {  // the term tiles of x serve phase 1 only
                unsigned t3[3][2];
                split3_pair(xq[u].x, xq[u].y, t3[0][0], t3[1][0], t3[2][0]);
                split3_pair(xq[u].z, xq[u].w, t3[0][1], t3[1][1], t3[2][1]);
                const int o = f32_xterm_base(x_unit) + XT::off(row, x_col);
#pragma unroll
                for (int t = 0; t < 3; ++t) *reinterpret_cast<uint2 *>(xt_all + t * WAVES * XS + o) = make_uint2(t3[t][0], t3[t][1]);
            }
            float *xr = xf_all + f32_xfloat_base(x_unit);
            *reinterpret_cast<float2 *>(xr + xfloat_off(row, x_col)) = make_float2(xq[u].x, xq[u].y);
            *reinterpret_cast<float2 *>(xr + xfloat_off(row, x_col + 2)) = make_float2(xq[u].z, xq[u].w);
        }
        if (bc_thread) {
            unsigned t3[3][2], u3[3][2];
            split3_pair(bq.x, bq.y, t3[0][0], t3[1][0], t3[2][0]);
            split3_pair(bq.z, bq.w, t3[0][1], t3[1][1], t3[2][1]);
            if (!STATES_ONLY) {
                split3_pair(cq.x, cq.y, u3[0][0], u3[1][0], u3[2][0]);
                split3_pair(cq.z, cq.w, u3[0][1], u3[1][1], u3[2][1]);
            }
            const int o = BT::off(bc_row, bc_pc * 4);
#pragma unroll
            for (int t = 0; t < 3; ++t) {
                *reinterpret_cast<uint2 *>(Bs + t * TB + o) = make_uint2(t3[t][0], t3[t][1]);
                if (!STATES_ONLY) *reinterpret_cast<uint2 *>(Cs + t * TB + o) = make_uint2(u3[t][0], u3[t][1]);
            }
        }
        // ---- scan of dt*A over the tile (float64 across the wave) and this unit's decay tables ----
        // alpha[l] = log2(e) * (dt A summed from the tile's first step through l): the reference of the separable factors
        // is the state entering the tile (alpha = 0), E[l] = exp2(alpha[l]), F[s] = exp2(-alpha[s]) dt[s]
        float a_end, span;  // exp2(alpha[Q-1]); the tile's log2-decay
        {
            constexpr double kLog2e = 1.4426950408889634;
            const float dtv = dq;
            const double incl = wave_inclusive_scan((double)dtv * a_h - (rq ? kResetDrop : 0.0));
            const double al = incl * kLog2e;
            const float hi = (float)al, lo = (float)(al - (double)hi);
            const float endh = readlane_f(hi, Q - 1), endl = readlane_f(lo, Q - 1);
            span = fmaxf(-(endh + endl), 0.f);
            a_end = exp2_hw(endh + endl);
            if (lane < Q) {
                ah_s[lane] = hi;
                alo_s[lane] = lo;
                dt_s[lane] = dtv;
                w_s[lane] = exp2_hw(fminf(alpha_diff(endh, endl, hi, lo), 0.f)) * dtv;
                E_s[lane] = exp2_hw(fminf(hi + lo, 0.f));
                F_s[lane] = exp2_hw(fminf(-(hi + lo), 126.f)) * dtv;
            }
        }
        if (c + 1 < c_end) prefetch(c + 1);
        block_sync_lds();  // tiles and tables are visible

        // ---- the tile's scores S[s, l] = B_s . C_l, once per workgroup: six products per float product make them a
        // quarter of a tile's matrix instructions.  Two waves sum half of the state dimension each; every wave adds the
        // two partial sums where it needs the scores (behind a second barrier, after its state readout) ----
        if constexpr (!STATES_ONLY) {
            if (wave < 2) {
                // (the wave index hidden from the compiler, which would otherwise keep these addresses -- a wave-uniform
                // offset from the ones every wave uses -- in registers of their own across the tile loop)
                int pw = wave;
                asm volatile("" : "+s"(pw));
                f32x16 part = {0};
#pragma unroll
                for (int j = 0; j < NK / 2; ++j) {
                    const int col = 16 * (pw * (NK / 2) + j) + 4 * half;
                    Frag3 Bf, Cp;
#pragma unroll
                    for (int t = 0; t < 3; ++t) {
                        Bf.t[t] = BT::split_frag(Bs + t * TB, r, col);
                        Cp.t[t] = BT::split_frag(Cs + t * TB, r, col);
                    }
                    part = mma6(Bf, Cp, part);
                }
                float *gd = G_s + pw * 1024 + lane * 4;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<float4 *>(gd + q * 256) = make_float4(part[4 * q], part[4 * q + 1], part[4 * q + 2], part[4 * q + 3]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- phase 1: y of this tile from the state entering it ----
        if constexpr (!STATES_ONLY) {
            const bool fast = __builtin_amdgcn_readfirstlane(__float_as_int(span)) <= __float_as_int(kFloatFastSpan);
            Frag3 Cf[NK];  // C[l = r, n in the accumulator's row order]
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
#pragma unroll
                for (int t = 0; t < 3; ++t) Cf[kk].t[t] = BT::split_frag(Cs + t * TB, r, 16 * kk + 4 * half);
            }
            // state readout H . C_l (times E[l] below): the accumulators as the A operand, split in registers
            f32x16 acc = {0};
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
                Bits3 hb;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int v = 8 * (kk % 2) + 2 * i;
                    split3_pair(st[kk / 2][v], st[kk / 2][v + 1], hb.t[0].u[i], hb.t[1].u[i], hb.t[2].u[i]);
                }
                acc = mma6(hb.frags(), Cf[kk], acc);
            }
            // scores S[s, l] = B_s . C_l: the two partial sums the workgroup shares
            block_sync_lds();
            f32x16 sc;
            {
                const float *gs = G_s + lane * 4;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 t0 = *reinterpret_cast<const float4 *>(gs + q * 256);
                    const float4 t1 = *reinterpret_cast<const float4 *>(gs + 1024 + q * 256);
                    sc[4 * q] = t0.x + t1.x;
                    sc[4 * q + 1] = t0.y + t1.y;
                    sc[4 * q + 2] = t0.z + t1.z;
                    sc[4 * q + 3] = t0.w + t1.w;
                }
            }
            Frag3 xfr[2];  // x^T: K order rows 16 j + 4 half + {0..3} and the same + 8
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int t = 0; t < 3; ++t) xfr[j].t[t] = XT::frag(xt + t * WAVES * XS, 16 * j + 4 * half, 8, 0, lane);
            }
            // decay factors of this lane's score elements (rows s = 8 vg + 4 half + i, column l = r)
            float4 fv[4];
            const float El = E_s[r];
            if (fast) {
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) fv[vg] = *reinterpret_cast<const float4 *>(F_s + 8 * vg + 4 * half);
            } else {
                acc = acc * El;
                const float al_hi = ah_s[r], al_lo = alo_s[r];
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int s0 = 8 * vg + 4 * half;
                    const float4 ah4 = *reinterpret_cast<const float4 *>(ah_s + s0);
                    const float4 al4 = *reinterpret_cast<const float4 *>(alo_s + s0);
                    const float4 dt4 = *reinterpret_cast<const float4 *>(dt_s + s0);
                    // exponents clamped at 0: entries above the diagonal stay finite and are masked below
                    fv[vg].x = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.x, al4.x), 0.f)) * dt4.x;
                    fv[vg].y = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.y, al4.y), 0.f)) * dt4.y;
                    fv[vg].z = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.z, al4.z), 0.f)) * dt4.z;
                    fv[vg].w = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.w, al4.w), 0.f)) * dt4.w;
                }
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                Bits3 mb;
#pragma unroll
                for (int k = 0; k < 4; ++k) {  // accumulator registers v = 8 j + 2 k, + 1
                    const int v = 8 * j + 2 * k, vg = v / 4, i = v % 4;
                    const float f0 = i == 0 ? fv[vg].x : fv[vg].z, f1 = i == 0 ? fv[vg].y : fv[vg].w;
                    // causal mask: row 8 vg + 4 half + i <= column r
                    const float s0 = (8 * vg + 4 * half + i <= r) ? sc[v] * f0 : 0.f;
                    const float s1 = (8 * vg + 4 * half + i + 1 <= r) ? sc[v + 1] * f1 : 0.f;
                    split3_pair(s0, s1, mb.t[0].u[k], mb.t[1].u[k], mb.t[2].u[k]);
                }
                acc = mma6(xfr[j], mb.frags(), acc);
            }
            if (fast) acc = acc * El;  // everything summed shares the factor E[l]
            // epilogue: y[t, h, p] = yT[p, l] + D[h] x[t, h, p]; acc[4 vg + i] is (l = r, p = 8 vg + 4 half + i)
            float o[16];
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const float2 xa = *reinterpret_cast<const float2 *>(xf + xfloat_off(r, 8 * vg + 4 * half));
                const float2 xb2 = *reinterpret_cast<const float2 *>(xf + xfloat_off(r, 8 * vg + 4 * half + 2));
                o[vg * 4 + 0] = acc[vg * 4 + 0] + dh * xa.x;
                o[vg * 4 + 1] = acc[vg * 4 + 1] + dh * xa.y;
                o[vg * 4 + 2] = acc[vg * 4 + 2] + dh * xb2.x;
                o[vg * 4 + 3] = acc[vg * 4 + 3] + dh * xb2.y;
            }
            store_column_buffer<float>(ybuf, (unsigned)(t0 + r) * (unsigned)(HP * sizeof(float)) + ycol_bytes, o, half, r < rows);
        }

        // ---- phase 2: the state leaving this tile (nobody reads the one the last tile leaves unless asked) ----
        // (the forward's last tile of a segment other than the last, or of a call that asks for no final state)
        if (!STATES_ONLY && c + 1 == c_end && !(final_states != nullptr && seg == S - 1)) break;
        seg_total *= a_end;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) st[nb] = st[nb] * a_end;
#pragma unroll
        for (int ks = 0; ks < Q; ks += 16) {
            const int k0 = ks + 8 * half;
            // (w o x)[l = k0 .. k0+7, p = r]
            const float4 wa = *reinterpret_cast<const float4 *>(w_s + k0);
            const float4 wb = *reinterpret_cast<const float4 *>(w_s + k0 + 4);
            const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
            Bits3 xw;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                split3_pair(xf[xfloat_off(k0 + 2 * i, r)] * wv[2 * i], xf[xfloat_off(k0 + 2 * i + 1, r)] * wv[2 * i + 1],
                            xw.t[0].u[i], xw.t[1].u[i], xw.t[2].u[i]);
            const Frag3 xwf = xw.frags();
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                Frag3 bf;  // B^T[n = 32 nb + r, l = k0 .. k0+7]
#pragma unroll
                for (int t = 0; t < 3; ++t) {
                    const bf16x4 lo4 = BT::tr_read(Bs + t * TB + BT::tr_off(ks + 8 * half, nb * 32, lane));
                    const bf16x4 hi4 = BT::tr_read(Bs + t * TB + BT::tr_off(ks + 8 * half + 4, nb * 32, lane));
                    bf.t[t].v = __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
                }
                st[nb] = mma6(bf, xwf, st[nb]);
            }
        }
    }

    if (STATES_ONLY || (final_states != nullptr && seg == S - 1)) {
        float *fb = final_states + ((((size_t)b * (STATES_ONLY ? S : 1) + (STATES_ONLY ? seg : 0)) * s.H + h) * s.P + pb * 32 + r) * N + 4 * half;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq)
                *reinterpret_cast<float4 *>(fb + 32 * nb + 8 * gq) =
                    make_float4(st[nb][4 * gq], st[nb][4 * gq + 1], st[nb][4 * gq + 2], st[nb][4 * gq + 3]);
        }
        if (STATES_ONLY && pb == 0 && lane == 0) seg_decay[((size_t)b * S + seg) * s.H + h] = seg_total;
    }
}

}  // namespace

// 8 when float inputs of this shape can run on the one-pass kernel (the waves per workgroup), else 0
int fused_scan_f32_waves(const ScanShape &s) {
    if (s.P % 32 != 0 || (s.N != 32 && s.N != 64)) return 0;
    if (s.mode != 0 || s.x_groups != 0) return 0;
    const int units = (s.H / s.G) * (s.P / 32);
    if (units % 8 != 0) return 0;
    if ((long long)s.L * s.H * s.P * 4 >= (1LL << 31)) return 0;  // y rows go through a 32-bit-offset buffer descriptor
    return 8;
}

// s.seg_tiles (tiles of kFloatTile steps per segment, 0 = not cut) and s.seg_local / s.seg_local_decay as for the
// bf16 kernel
hipError_t launch_fused_scan_f32(const ScanShape &s, const void *x, const void *dt, const float *A, const void *Bm,
                                 const void *Cm, const float *D, const float *init, const unsigned char *reset, void *y,
                                 float *final_states, hipStream_t st) {
    if (fused_scan_f32_waves(s) != 8) return hipErrorInvalidValue;
    const int nc = (s.L + kFloatTile - 1) / kFloatTile;
    const int segments = s.seg_tiles > 0 ? (nc + s.seg_tiles - 1) / s.seg_tiles : 1;
    if ((segments > 1) != (s.seg_local != nullptr)) return hipErrorInvalidValue;
    const int grid = s.B * s.G * ((s.H / s.G) * (s.P / 32) / 8) * segments;
    const float *xx = static_cast<const float *>(x), *dd = static_cast<const float *>(dt);
    const float *bb = static_cast<const float *>(Bm), *cc = static_cast<const float *>(Cm);
    if (s.N == 64)
        fused_scan_f32_kernel<4, 8, false><<<dim3(grid), dim3(512), 0, st>>>(xx, dd, A, bb, cc, D, init, reset, static_cast<float *>(y), final_states, nullptr, s);
    else
        fused_scan_f32_kernel<2, 8, false><<<dim3(grid), dim3(512), 0, st>>>(xx, dd, A, bb, cc, D, init, reset, static_cast<float *>(y), final_states, nullptr, s);
    return hipGetLastError();
}

int fused_scan_f32_tile() { return kFloatTile; }

// The float forward on `segments` segments of the sequence: the states-only pass, then the forward per segment
// (seg_states [B, segments, H, P, N] and seg_decay [B, segments, H] floats of scratch).
hipError_t launch_fused_scan_f32_segmented(const ScanShape &s, int segments, const void *x, const void *dt, const float *A,
                                           const void *Bm, const void *Cm, const float *D, const float *init,
                                           const unsigned char *reset, void *y, float *final_states, float *seg_states,
                                           float *seg_decay, hipStream_t st) {
    if (segments < 2 || fused_scan_f32_waves(s) != 8) return hipErrorInvalidValue;
    const int nc = (s.L + kFloatTile - 1) / kFloatTile;
    ScanShape t = s;
    t.seg_tiles = (nc + segments - 1) / segments;
    if ((nc + t.seg_tiles - 1) / t.seg_tiles != segments) return hipErrorInvalidValue;
    const int grid = s.B * s.G * ((s.H / s.G) * (s.P / 32) / 8) * segments;
    const float *xx = static_cast<const float *>(x), *dd = static_cast<const float *>(dt);
    const float *bb = static_cast<const float *>(Bm);
    if (s.N == 64)
        fused_scan_f32_kernel<4, 8, true><<<dim3(grid), dim3(512), 0, st>>>(xx, dd, A, bb, bb, nullptr, nullptr, reset, nullptr, seg_states, seg_decay, t);
    else
        fused_scan_f32_kernel<2, 8, true><<<dim3(grid), dim3(512), 0, st>>>(xx, dd, A, bb, bb, nullptr, nullptr, reset, nullptr, seg_states, seg_decay, t);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    t.seg_local = seg_states;
    t.seg_local_decay = seg_decay;
    return launch_fused_scan_f32(t, x, dt, A, Bm, Cm, D, init, reset, y, final_states, st);
}

}  // namespace ssd
