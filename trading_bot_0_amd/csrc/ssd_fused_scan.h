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
//                       + sum_{s-blocks sb < lb} xT . (B.C^T o F_lb) )     intra-chunk, below the diagonal
//              + xT . (B.C^T o mask o E[l] F_lb)                           diagonal block
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

template <int COLS> struct ChunkTile {  // bf16 [rows][COLS], COLS = 32, 64 or 128
    static_assert(COLS == 32 || COLS == 64 || COLS == 128, "tile rows are 64, 128 or 256 bytes");
    // XOR mask on the index of an 8-byte piece within its row (period: 32 rows).  Two descriptions of this chip's LDS
    // had to be satisfied at once.  Timed with a 16-wave probe, a plain 8-byte access is served 16 consecutive lanes
    // at a time from 128 bytes of banks (4.2 cycles per wave-instruction at best, 8 when two of the 16 lanes share an
    // 8-byte slot) and the transposing read 32 lanes at a time from 256 bytes.  The hardware's bank-conflict counter,
    // though, charges a plain 8-byte access by 32 lanes over 256 bytes: a mask that is a bijection of the low four
    // row bits only (free of conflicts by the timing) doubled the counter against one that spreads 32 rows over 256
    // bytes (free of conflicts by the counter, 8 cycles by the timing), with no difference in the kernels' run time
    // either way.  The masks below satisfy both: for the 8-byte reads of one logical piece of 32 consecutive rows,
    // any aligned 16 rows fill the 16 slots of 128 bytes and all 32 rows fill the 32 slots of 256 bytes; and the
    // transposing read's four consecutive rows keep their 64-byte pieces in different quarters of 256 bytes.
    static __device__ inline int f(int row) {
        const int r0 = row & 1, r1 = (row >> 1) & 1, r2 = (row >> 2) & 1, r3 = (row >> 3) & 1, r4 = (row >> 4) & 1;
        if constexpr (COLS == 32) {
            // 64-byte rows, 8 pieces: per row parity a bijection of rows 1-3 (16 rows, 128 bytes), per row mod 4 a
            // bijection of rows 2-4 (32 rows, 256 bytes)
            return (r3 << 2) | (r2 << 1) | (r1 ^ r4);
        } else if constexpr (COLS == 128) {
            // 256-byte rows, 32 pieces: the 64-byte quarter from the row's low two bits, the low four mask bits a
            // bijection of the row's low four bits, all five of all five
            return ((r1 ^ r4) << 4) | (r0 << 3) | (r1 << 2) | (r2 << 1) | r3;
        } else {
            // 128-byte rows, 16 pieces: a bijection of the low four row bits, and per row parity of rows 1-4; the
            // 64-byte half from row bit 1
            return (r1 << 3) | (r3 << 2) | (r2 << 1) | (r0 ^ r4);
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
    static __device__ inline int tr_off(int k0, int c0, int lane) {  // element offset this lane hands to the read
        const int q = lane >> 4, a = (lane >> 2) & 3, b = lane & 3;
        return off(k0 + a, c0 + 16 * (q & 1) + 4 * b);
    }
    static __device__ inline bf16x4 tr_read(const __bf16 *src) {
        const bf16x4_gcc v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((SSD_LDS_AS bf16x4_gcc *)(src));
        return __builtin_bit_cast(bf16x4, v);
    }
    static __device__ inline bf16x4 tr4(const __bf16 *tile, int k0, int c0, int lane) {
        return tr_read(tile + tr_off(k0, c0, lane));
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

// Time steps per tile of the one-pass kernel.  The kernel has no workspace whose layout the caller's chunk
// length would fix, so it tiles time by what runs fastest: with 64 a tile has one s-block below the diagonal
// per two on it (128: three per two; 32: none, but the per-tile work doubles again); measured 210 us against
// 238 us at 128 for batch 256, seqlen 2048, 8 heads of 32, state 64.
constexpr int kOnePassTile = 64;

constexpr float kFastDiagSpan = 120.f;  // log2-decay across a diagonal block up to which E*F is safe

// LDS of one workgroup: B and C tiles, one x tile per wave, (5 + Q/32) float rows and 16 block scalars per wave.
constexpr int fused_scan_xtile_elems(int Q) { return Q * 32 + 16; }
// Where unit u's x tile starts inside the x region of the forward's layout (waves * fused_scan_xtile_elems(Q)
// elements): tiles of exactly Q * 32 elements, odd units 8 bytes further, every pair of units 64 bytes further.
// A staging write hits one row and four 8-byte pieces of the same parity in each of the workgroup's tiles at once;
// with these offsets the 16 (or 32) lanes served together fill 128 (256) bytes of banks exactly.
__device__ inline int fused_scan_xtile_base(int Q, int u) { return u * (Q * 32) + (u & 1) * 4 + (u >> 1) * 32; }
// The eight-wave forward with a state of 64 or less keeps two sets of tiles and alternates between them: a tile's
// staging writes then go to the set last read two tiles ago, which every wave left before the barrier of the tile in
// between, so the barrier in front of the staging writes is not needed (one barrier per tile instead of two; the tile
// loop is unrolled by two so that the set is a compile-time offset).  Measured 201 against 209 us at batch 256, 2048
// steps, 8 heads of 32, state 64; the four-wave instance for a 128-wide state is slower with it (1615 against 1455 us
// at batch 32, 16384 steps: its loop body is about three times as long, and unrolled by two it runs slower) and keeps one set.
constexpr bool fused_scan_two_tile_sets(int N, int waves) { return waves == 8 && N <= 64; }
constexpr size_t fused_scan_lds_bytes(int N, int Q, int waves) {
    return ((size_t)2 * Q * N * 2 + (size_t)waves * fused_scan_xtile_elems(Q) * 2) * (fused_scan_two_tile_sets(N, waves) ? 2 : 1) +
           (size_t)waves * ((size_t)(5 + Q / 32) * Q * 4 + 64);
}

// KIND 0: the forward.  KIND 1: the reversed-adjoint recurrence of the backward pass.  KIND 2: states only --
// no outputs, no C: the state a segment of the sequence leaves behind (from its own initial state) and the
// segment's total decay, for sequences cut into segments that run side by side.
// KIND 3 and 4: the backward pass's two scans of the transposed state (3 forward in time, 4 reversed-adjoint).
// There B and C are per head and x is shared by the heads of a group, the opposite of the forward, so a
// workgroup is eight heads on one 32-column slice of x: every wave stages its own B and C tile, the x tile is
// shared, and instead of writing y per head the waves add their tiles in LDS and the workgroup writes the sum
// over its heads (dC, or dB with the heads' dt as weights) -- the per-head outputs never reach memory.  KIND 3
// also writes, per head, the part of C_t . y_t that its slice holds.  Whichever of the two runs second also takes
// (ScanAnchors) the inner products of the state entering each of its tiles with the other scan's state at the same
// timestep, which the decay gradient hangs on: KIND 3 and 7 hold that code.
// KIND 5: the reversed-adjoint scan of the backward pass with the row products in its epilogue (headdim 32: a wave
// holds a head's whole row).  With r_t the recurrence's output it writes dx_t = dt_t r_t + D x_t (x being the
// scan's x operand, dy) instead of r, and per (b, t, h) the pair (aux_t . r_t, aux_t . x_t) -- aux is the forward's
// x, so these are e1 = x . r and dd = dy . x -- into seg_decay as float2 [B, L, H].
// LDS of a workgroup of the transposed scans: a B and a C tile per wave (eight waves), the shared x tile and
// second-operand tile, the per-wave tables, and a [Q][33] float tile per wave for the heads' outputs (summed in a
// fixed order when the workgroup writes them out, so that results do not depend on timing).
// KIND 6 and 7 are 3 and 4 for a 64-wide transposed state (dstate 64) with both 32-column slices of a head in one
// wave: the head's masked, decayed score tile -- the part of a tile's work that does not shrink with the state's
// width -- and its B and C tiles are then formed and staged once instead of once per slice.  Their LDS holds two x
// tiles and two tiles of the second operand of C . y, 4 elements apart (a staging write puts 8-byte halves of one row
// into both tiles of a pair: one takes the even 8-byte slots of the row's banks, the other the odd ones), and a
// float tile per wave of 32 rows only: the workgroup writes its sums out after every block of 32 rows.  That tile's
// rows are 64 floats with their 16-byte pieces XOR-swizzled by the row's low four bits, so that a lane's four
// consecutive columns go out and come back as one 16-byte access and 16 consecutive rows of one logical piece
// cover 256 bytes of banks.
constexpr int wide_transposed_tile_elems(int Q) { return Q * 32 + 4; }
constexpr size_t wide_transposed_scan_lds_bytes(int Q) {
    return (size_t)(2 * 8) * fused_scan_xtile_elems(Q) * 2 + (size_t)4 * wide_transposed_tile_elems(Q) * 2 +
           (size_t)8 * ((5 + Q / 32) * Q * 4 + 64) + (size_t)8 * 32 * 64 * 4;
}
constexpr size_t transposed_scan_lds_bytes(int Q) {
    return (size_t)(2 * 8 + 2) * fused_scan_xtile_elems(Q) * 2 + (size_t)8 * ((5 + Q / 32) * Q * 4 + 64) +
           (size_t)8 * Q * 33 * 4;
}

template <typename TO, int NK, int QB, int WAVES, int KIND>  // N = 16*NK, Q = 32*QB
__global__ __launch_bounds__(64 * WAVES, (WAVES == 8 || NK == 8) ? 1 : 2) void fused_scan_kernel(
    const __bf16 *__restrict__ x, const __bf16 *__restrict__ dt, const float *__restrict__ A,
    const __bf16 *__restrict__ Bm, const __bf16 *__restrict__ Cm, const float *__restrict__ D,
    const float *init, const unsigned char *__restrict__ reset, TO *__restrict__ y, float *final_states,
    float *tile_states, float *seg_decay, const __bf16 *__restrict__ aux, ScanShape s, ScanAnchors an) {
    using T = __bf16;
    constexpr bool ADJ = KIND == 1 || KIND == 4 || KIND == 5 || KIND == 7, STATES_ONLY = KIND == 2;
    constexpr bool TR = KIND == 3 || KIND == 4 || KIND == 6 || KIND == 7;
    constexpr bool TR_FWD = KIND == 3 || KIND == 6, TR_ADJ = KIND == 4 || KIND == 7;
    constexpr int SL = (KIND == 6 || KIND == 7) ? 2 : 1;  // 32-column slices of x (and of the state) per wave
    constexpr bool ROWS = KIND == 5;
    static_assert(!TR || (NK == 2 && WAVES == 8), "the transposed scans: 32-wide state, eight heads per workgroup");
    constexpr int N = 16 * NK, NB = NK / 2, Q = 32 * QB, nthr = 64 * WAVES;
    constexpr int EPL = Q >= 64 ? Q / 64 : 1;  // chunk positions per lane in the scan
    constexpr int BPR = N / 8;                 // 16-byte pieces per B (or C) row
    constexpr int BSL = Q * BPR;               // pieces of a B (or C) tile
    constexpr int UBC = (BSL + nthr - 1) / nthr;
    constexpr int BRP = nthr / BPR;            // B rows per pass of the workgroup (a multiple of 32)
    constexpr int XPR = WAVES * 4;             // 16-byte pieces of one timestep's x for the workgroup
    constexpr int UX = Q / 16;                 // passes of 16 rows
    static_assert((BRP % 32 == 0 || BRP == 16) && nthr / XPR == 16, "staging offsets rely on the swizzle period of 32 rows");
    constexpr bool kSharedBcOffsets = BRP % 32 == 0;  // else every pass of B and C computes its own offsets
    using XT = ChunkTile<32>;
    using BT = ChunkTile<N>;
    // static, so that LDS addresses are compile-time offsets
    constexpr int XS = SL == 2 ? wide_transposed_tile_elems(Q) : fused_scan_xtile_elems(Q);
    // The eight units of a workgroup are the eight heads (or head slices) of one group: they share B and C, and so the
    // scores B . C^T of a tile -- three blocks of 32 x 32 with tiles of 64 steps.  Three waves form one block each and
    // leave it in LDS in the accumulator's own layout, every wave reads the three from there: 12 matrix instructions
    // per tile and workgroup instead of 96, for 12 KB of LDS and a second barrier per tile (behind the first block's
    // readout, where the scores are first needed).
    constexpr bool kSharedScores = !TR && KIND != 2 && WAVES == 8 && QB == 2 && NK <= 4;
    __shared__ __attribute__((aligned(16))) unsigned char smem[SL == 2 ? wide_transposed_scan_lds_bytes(Q)
                                                                        : TR ? transposed_scan_lds_bytes(Q)
                                                                             : fused_scan_lds_bytes(N, Q, WAVES) + (kSharedScores ? 3 * 32 * 32 * 4 : 0)];  // (kind 5 uses one set of the two)
    const int tid = threadIdx.x;
    const int lane0 = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // forward: B and C tiles [Q][N] of the workgroup, then one x tile [Q][32] per wave (+16 elements between tiles).
    // transposed: a B and a C tile [Q][32] per wave, then the shared x tile and the shared tile of the second
    // operand of the C . y products, each [Q][32].
    // (forward with two tile sets: B, B', C, C', the x tiles, the x tiles')
    // (kind 5 spills ten registers with two sets and its early request of the next tile; with two sets and the late
    // request the backward pass measured 1145 against 1123 us, so it keeps one set)
    constexpr bool kTwoSets = !TR && KIND != 5 && fused_scan_two_tile_sets(N, WAVES);
    constexpr int SETS = kTwoSets ? 2 : 1;
    T *tiles = reinterpret_cast<T *>(smem);
    // (transposed: the heads' B tiles, then their C tiles, each set laid out like the forward's x tiles -- the staging
    // writes are the same, a row of every head's tile at once -- then the shared tiles, XS apart)
    constexpr int TRB = WAVES * fused_scan_xtile_elems(Q);  // the eight heads' B (or C) tiles
    T *const Bs0 = TR ? tiles + fused_scan_xtile_base(Q, wave) : tiles;
    T *const Cs0 = TR ? tiles + TRB + fused_scan_xtile_base(Q, wave) : tiles + SETS * Q * N;
    T *const xs_all0 = TR ? tiles + 2 * TRB : tiles + 2 * SETS * Q * N;
    T *aux_s = xs_all0 + SL * XS;  // transposed only (one tile per slice, behind the x tiles)
    float *wf0 = reinterpret_cast<float *>(TR ? xs_all0 + 2 * SL * XS : xs_all0 + SETS * WAVES * XS);
    float *wf = wf0 + wave * ((5 + QB) * Q + 16);
    // transposed only: every head's output tile, [WAVES][Q][33], or [WAVES][32][64] (swizzled) with two slices per wave
    float *red = wf0 + WAVES * ((5 + QB) * Q + 16);
    float *const G_s = red;  // shared scores (not transposed): [3 blocks][4 quarters][64 lanes][4 floats]
    constexpr int RS = SL == 2 ? 64 : 33;
    float *ah_s = wf, *alo_s = wf + Q, *dt_s = wf + 2 * Q, *w_s = wf + 3 * Q, *E_s = wf + 4 * Q, *F_s = wf + 5 * Q;
    float *blk_s = wf + (5 + QB) * Q;  // [0..QB): exp2(alpha[32 lb]); [8..8+QB): log2-decay across block lb

    // ---- which units this workgroup owns ----
    const int PBn = s.P / 32, HG = s.H / s.G;
    const int UW = (HG * PBn) / WAVES;  // workgroups per (batch, group)
    // A sequence may be cut into S segments of s.seg_tiles tiles that different workgroups walk: initial states
    // are then given per segment ([B,S,H,P,N]) and, in KIND 2, final states and decays written per segment.
    const int S = s.seg_tiles > 0 ? (s.nc + s.seg_tiles - 1) / s.seg_tiles : 1;
    const int slot = xcd_remap(blockIdx.x, gridDim.x);
    const int seg = slot % S, logical = slot / S;
    // states only: nothing comes after the last segment, so what it adds to the state is not needed (the final
    // state comes from the forward over that segment) -- its workgroups leave at once
    if (STATES_ONLY && S > 1 && seg == S - 1) return;
    const int c_first = seg * (s.seg_tiles > 0 ? s.seg_tiles : s.nc);
    const int c_end = s.seg_tiles > 0 ? min(s.nc, c_first + s.seg_tiles) : s.nc;
    // transposed: the workgroup is heads h0 .. h0+7 (one per wave) on x slice pb; s.G == s.H there, and
    // s.x_groups says how many groups of heads x is given for
    const int TW = TR ? (s.H / 8) * (SL == 2 ? 1 : PBn) : 1;  // transposed workgroups per batch row
    const int b = TR ? logical / TW : logical / (s.G * UW);
    const int g = TR ? 0 : (logical / UW) % s.G;
    const int unit0 = TR ? 0 : (logical % UW) * WAVES;
    const int unit = unit0 + wave;
    const int h0 = TR ? (SL == 2 ? logical % TW : (logical % TW) / PBn) * 8 : 0;
    const int h = TR ? h0 + wave : g * HG + unit / PBn;
    const int pb = TR ? (SL == 2 ? 0 : (logical % TW) % PBn) : unit % PBn;
    const int xcol0 = g * HG * s.P + unit0 * 32;  // first element of the workgroup's slice of an x row
    const int HP = s.H * s.P;
    // x rows: one per timestep, HP wide -- or, when x is shared by groups of heads (s.x_groups, with G == H so
    // that the workgroup is one head, or eight heads of one group in the transposed scans), x_groups * P wide
    // with this group's columns
    const int XLD = s.x_groups ? s.x_groups * s.P : HP;
    const int xcol = TR ? (h0 / (s.H / s.x_groups)) * s.P + pb * 32
                        : (s.x_groups ? (h / (s.H / s.x_groups)) * s.P + (unit0 % PBn) * 32 : xcol0);
    // ADJ: x, B, C, dt, the reset mask and y are the forward sequence's tensors, dt_len rows per batch row, and row
    // tau of the scan is their row L - 1 - tau (rows outside them are no-op steps in front of the reversed sequence)
    const int trows = ADJ ? s.dt_len : s.L;
    const T *xb = x + (size_t)b * trows * XLD + xcol;
    const T *Bb = Bm + ((size_t)b * trows * s.G + (TR ? h0 : g)) * N;  // transposed: eight heads' rows side by side
    const T *Cb = Cm + ((size_t)b * trows * s.G + (TR ? h0 : g)) * N;
    const T *auxb = TR_FWD && aux ? aux + (size_t)b * trows * XLD + xcol : nullptr;
    // mode 1 (the time-reversed adjoint recurrence): step t decays by the dt of step L - t of a dt tensor of
    // dt_len rows, steps outside it do not decay, and every step's input weighs one instead of dt
    const int dt_rows = ADJ ? s.dt_len : s.L;
    const T *dtb = dt + (size_t)b * dt_rows * s.H + h;
    const unsigned char *rsb = reset ? reset + (size_t)b * dt_rows : nullptr;  // state restarts, see kResetLog2
    // this batch row's y as a range-checked buffer (the launchers keep a row below 2^31 bytes): the epilogue's stores
    // go through it, so rows outside the sequence are dropped by the hardware instead of branched around
    const __amdgpu_buffer_rsrc_t ybuf = make_buffer(y + (size_t)b * trows * HP, (unsigned)((size_t)trows * HP * sizeof(TO)));
    const unsigned ycol_bytes = (unsigned)((h * s.P + pb * 32) * sizeof(TO));
    const float dh = D ? D[h] : 0.f;
    const double a_h = (double)A[h];

    // ---- registers holding the next chunk's inputs ----
    // A thread's pieces sit at one fixed 32-bit element offset from a pointer that is uniform per pass.
    // Tiles of 64 steps leave room for every lane-derived offset and LDS address to stay in registers for
    // the whole kernel.  Longer tiles do not: there the offsets are recomputed where they are used, from a
    // copy of the thread index that an empty asm hides from the compiler, so that it cannot hoist them out
    // of the tile loop again (hoisted, they held about a hundred registers through all phases and forced
    // spills whose reloads, each an s_waitcnt vmcnt(0), serialised the prefetch).
    constexpr bool kRecomputeOffsets = QB > 2 || SL == 2;
    auto phase_tid = [&]() {
        int t = tid;
        if (kRecomputeOffsets) asm volatile("" : "+v"(t));
        return t;
    };
    // When the next tile's inputs are requested: after phase 1 (they are then in flight during phase 2 only, but
    // hold no registers through phase 1), or before phase 1 -- for the two-wave workgroups, whose per-head B and C
    // rows are short and slow to arrive, and for the eight-wave forward, where it costs 6 registers and measures 2 %
    // faster with bf16 y, 8 % with float y (217 against 222 us and 245 against 268 us at batch 256, 2048 steps, 8 heads
    // of 32, state 64).  The four-wave forward with a 128-wide state is 5 % slower with it and keeps the late request.
    // Of the backward pass's kinds, 5 and 6 take it without spilling (the pass 1.10 against 1.12 ms); 7 would spill.
    constexpr bool kEarlyPrefetch = WAVES == 2 || (WAVES == 8 && (KIND == 0 || KIND == 5 || KIND == 6));
    // (transposed: UX passes of the eight heads' B and C rows, one piece of the shared x tile and of the second
    // operand's tile)
    uint4 bq[TR ? UX : UBC], cq[TR ? UX : UBC], xq[TR ? 1 : UX], auxq = make_uint4(0, 0, 0, 0);
    unsigned short dq[EPL];
    unsigned char rq[EPL];
    auto prefetch = [&](int c) {
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        const int tv = phase_tid();
        const int bc_row0 = tv / BPR, x_row0 = tv / XPR;
        const unsigned bc_off0 = bc_row0 * s.G * N + (tv % BPR) * 8;
        const unsigned x_off0 = x_row0 * XLD + (tv % XPR) * 8;
        const unsigned dt_off0 = (tv & 63) * EPL * s.H;
        const T *bp = Bb + (size_t)t0 * s.G * N, *cp = Cb + (size_t)t0 * s.G * N;
        const T *xp = xb + (size_t)t0 * XLD, *dp = dtb + (size_t)t0 * s.H;
        auto reset_byte = [&](int e, bool ok) {  // the restart flag that applies at row t0 + lane*EPL + e
            const int row = t0 + (tv & 63) * EPL + e;
            if (rsb == nullptr || !ok) return (unsigned char)0;
            if (ADJ) {  // the restart before forward step L - row cuts the adjoint at this reversed step
                const int src = s.L - row;
                return (src >= 1 && src < dt_rows) ? rsb[src] : (unsigned char)0;
            }
            return rsb[row];
        };
        auto dt_bits = [&](int e, bool ok) {  // dt of row t0 + lane*EPL + e as raw bits, zero where it does not apply
            const int row = t0 + (tv & 63) * EPL + e;
            if (ADJ) {
                const int src = s.L - row;
                return (ok && src >= 1 && src < dt_rows) ? __builtin_bit_cast(unsigned short, dtb[(size_t)src * s.H])
                                                         : (unsigned short)0;
            }
            return ok ? __builtin_bit_cast(unsigned short, dp[dt_off0 + e * s.H]) : (unsigned short)0;
        };
        // (a conditional expression over *ptr and a zero constant would become a load through a selected
        // pointer, with the constant in scratch memory)
        auto ld16 = [](const T *ptr, bool ok) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ok) v = *reinterpret_cast<const uint4 *>(ptr);
            return v;
        };
        if constexpr (TR) {
            const int prow = tv / XPR, srow = tv / (4 * SL);
            const unsigned pcol = (tv % XPR) * 8, scol = (tv % (4 * SL)) * 8;
            auto source = [&](int row, bool &ok) {  // the tensors' row of this tile's row `row`
                const int src = ADJ ? s.L - 1 - t0 - row : t0 + row;
                ok = ADJ ? (src >= 0 && src < trows) : row < rows;
                return src;
            };
#pragma unroll
            for (int u = 0; u < UX; ++u) {
                bool ok;
                const int src = source(prow + 16 * u, ok);
                bq[u] = ld16(Bb + (size_t)src * s.G * N + pcol, ok);
                cq[u] = ld16(Cb + (size_t)src * s.G * N + pcol, ok);
            }
            {
                bool ok;
                const int src = source(srow, ok);
                ok = ok && tv < Q * 4 * SL;
                xq[0] = ld16(xb + (size_t)src * XLD + scol, ok);
                if (TR_FWD && auxb != nullptr) auxq = ld16(auxb + (size_t)src * XLD + scol, ok);
            }
#pragma unroll
            for (int e = 0; e < EPL; ++e) dq[e] = dt_bits(e, (tv & 63) * EPL + e < rows);
#pragma unroll
            for (int e = 0; e < EPL; ++e) rq[e] = reset_byte(e, (tv & 63) * EPL + e < rows);
        } else if (ADJ) {
            const int first = s.L - 1 - t0;  // the tensors' row of this tile's first row; later rows count down
#pragma unroll
            for (int u = 0; u < UBC; ++u) {
                const int src = first - (bc_row0 + u * BRP);
                const bool ok = (BSL % nthr == 0 || tv + u * nthr < BSL) && src >= 0 && src < trows;
                bq[u] = ld16(Bb + (size_t)src * s.G * N + (tv % BPR) * 8, ok);
                if (!STATES_ONLY) cq[u] = ld16(Cb + (size_t)src * s.G * N + (tv % BPR) * 8, ok);
            }
#pragma unroll
            for (int u = 0; u < UX; ++u) {
                const int src = first - (x_row0 + u * 16);
                xq[u] = ld16(xb + (size_t)src * XLD + (tv % XPR) * 8, src >= 0 && src < trows);
            }
#pragma unroll
            for (int e = 0; e < EPL; ++e) dq[e] = dt_bits(e, (tv & 63) * EPL + e < rows);
#pragma unroll
            for (int e = 0; e < EPL; ++e) rq[e] = reset_byte(e, (tv & 63) * EPL + e < rows);
        } else if (rows == Q) {
#pragma unroll
            for (int u = 0; u < UBC; ++u) {
                const bool ok = BSL % nthr == 0 || tv + u * nthr < BSL;
                bq[u] = ld16(bp + (size_t)u * BRP * s.G * N + bc_off0, ok);
                if (!STATES_ONLY) cq[u] = ld16(cp + (size_t)u * BRP * s.G * N + bc_off0, ok);
            }
#pragma unroll
            for (int u = 0; u < UX; ++u) xq[u] = *reinterpret_cast<const uint4 *>(xp + (size_t)u * 16 * XLD + x_off0);
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                dq[e] = dt_bits(e, Q >= 64 || (tv & 63) < Q);
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                rq[e] = reset_byte(e, Q >= 64 || (tv & 63) < Q);
        } else {  // ragged last chunk: rows past the sequence read as zero (dt = 0 makes them no-ops)
#pragma unroll
            for (int u = 0; u < UBC; ++u) {
                const bool ok = (BSL % nthr == 0 || tv + u * nthr < BSL) && bc_row0 + u * BRP < rows;
                bq[u] = ld16(bp + (size_t)u * BRP * s.G * N + bc_off0, ok);
                if (!STATES_ONLY) cq[u] = ld16(cp + (size_t)u * BRP * s.G * N + bc_off0, ok);
            }
#pragma unroll
            for (int u = 0; u < UX; ++u) xq[u] = ld16(xp + (size_t)u * 16 * XLD + x_off0, x_row0 + u * 16 < rows);
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                dq[e] = dt_bits(e, (tv & 63) * EPL + e < rows);
#pragma unroll
            for (int e = 0; e < EPL; ++e)
                rq[e] = reset_byte(e, (tv & 63) * EPL + e < rows);
        }
    };

    // ---- running state of this unit: st[nb][v] = H[p = r, n = 32 nb + 8 (v/4) + 4 half + v%4] ----
    // (with two slices per wave: slice sl in st[sl * NB ..])
    f32x16 st[SL * NB];
    // a restart before the first step: the initial state is not read at all (it may hold anything)
    const bool folded = KIND == 0 && s.seg_local != nullptr;  // the entering state comes from the recurrence below
    const bool fresh = !ADJ && rsb != nullptr && (seg == 0 || folded) && rsb[0] != 0;
    // the first tile's inputs are requested ahead of the state's, so that the two trips to memory overlap (and behind
    // the restart flag's, which the state's loads branch on)
    prefetch(c_first);
#pragma unroll
    for (int sl = 0; sl < SL; ++sl) {
        const size_t lane_off = (size_t)((pb + sl) * 32 + (lane0 & 31)) * N + 4 * (lane0 >> 5);
        // (one uniform branch around all of the state's loads: with a condition on each, the compiler waits for every
        // load before the next -- eight or sixteen trips to memory before the first tile)
        const bool have_init = init != nullptr && !fresh;
        float4 iq[NB][4];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) iq[nb][gq] = make_float4(0, 0, 0, 0);
        }
        if (have_init) {
            const float *ib = init + (((size_t)b * (folded ? 1 : S) + (folded ? 0 : seg)) * s.H + h) * s.P * N + lane_off;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) iq[nb][gq] = *reinterpret_cast<const float4 *>(ib + 32 * nb + 8 * gq);
            }
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                st[sl * NB + nb][4 * gq + 0] = iq[nb][gq].x;
                st[sl * NB + nb][4 * gq + 1] = iq[nb][gq].y;
                st[sl * NB + nb][4 * gq + 2] = iq[nb][gq].z;
                st[sl * NB + nb][4 * gq + 3] = iq[nb][gq].w;
            }
        }
        if constexpr (KIND == 0) {
            if (folded) {  // enter[j+1] = decay[j] * enter[j] + local[j] over the segments before this one
                // two segments per round, both requested before the first is used: half the trips to memory
                for (int j = 0; j < seg; j += 2) {
                    const int j1 = min(j + 1, seg - 1);
                    const float a0 = s.seg_local_decay[((size_t)b * S + j) * s.H + h];
                    const float a1 = s.seg_local_decay[((size_t)b * S + j1) * s.H + h];
                    const float *l0 = s.seg_local + (((size_t)b * S + j) * s.H + h) * s.P * N + lane_off;
                    const float *l1 = s.seg_local + (((size_t)b * S + j1) * s.H + h) * s.P * N + lane_off;
                    float4 v0[NB][4], v1[NB][4];
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                        for (int gq = 0; gq < 4; ++gq) {
                            v0[nb][gq] = *reinterpret_cast<const float4 *>(l0 + 32 * nb + 8 * gq);
                            v1[nb][gq] = *reinterpret_cast<const float4 *>(l1 + 32 * nb + 8 * gq);
                        }
                    }
                    const bool two = j + 1 < seg;  // (uniform)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                        for (int gq = 0; gq < 4; ++gq) {
                            f32x16 &t = st[sl * NB + nb];
                            t[4 * gq + 0] = a0 * t[4 * gq + 0] + v0[nb][gq].x;
                            t[4 * gq + 1] = a0 * t[4 * gq + 1] + v0[nb][gq].y;
                            t[4 * gq + 2] = a0 * t[4 * gq + 2] + v0[nb][gq].z;
                            t[4 * gq + 3] = a0 * t[4 * gq + 3] + v0[nb][gq].w;
                            if (two) {
                                t[4 * gq + 0] = a1 * t[4 * gq + 0] + v1[nb][gq].x;
                                t[4 * gq + 1] = a1 * t[4 * gq + 1] + v1[nb][gq].y;
                                t[4 * gq + 2] = a1 * t[4 * gq + 2] + v1[nb][gq].z;
                                t[4 * gq + 3] = a1 * t[4 * gq + 3] + v1[nb][gq].w;
                            }
                        }
                    }
                }
            }
        }
    }

    // this lane's part of the unit's [32 columns, N] block of a [P,N] state
    auto store_state = [&](float *state_bh) {
#pragma unroll
        for (int sl = 0; sl < SL; ++sl) {
            float *fb = state_bh + (size_t)((pb + sl) * 32 + (lane0 & 31)) * N + 4 * (lane0 >> 5);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                for (int gq = 0; gq < 4; ++gq)
                    *reinterpret_cast<float4 *>(fb + 32 * nb + 8 * gq) =
                        make_float4(st[sl * NB + nb][4 * gq], st[sl * NB + nb][4 * gq + 1], st[sl * NB + nb][4 * gq + 2],
                                    st[sl * NB + nb][4 * gq + 3]);
            }
        }
    };

    // The anchors (KIND 3 and 7): this slice's part of <this scan's state, the other scan's state> at the start of this
    // scan's tile j (j = nc: its final state).  The other scan ran over the sequence in the opposite direction, so its
    // tile nc - j begins where this one's tile j does; this scan's initial state meets the other's final state and
    // the other way round.  The piece goes to out[b, k, h, slice] with k counted in forward time.
    constexpr bool ANCH = KIND == 3 || KIND == 7;
    // (where the other scan has no state to meet -- no initial state, no gradient on the final state -- the anchor is
    // zero: the loads then read the other scan's first tile state, so that none of them stands under a condition, and
    // `zero` drops the result.  A load under a condition sits in a block of its own with its first use, and the wave
    // waits for it there instead of during the phase it was meant to overlap.)
    auto adjoint_state = [&](int j, bool &zero) -> const float * {
        const float *g = j == 0 ? an.other_final : j == s.nc ? an.other_init : an.other_tiles;
        zero = g == nullptr;
        const bool tiles = zero || (j != 0 && j != s.nc);
        // (the other scan kept the states entering its tiles phase, phase + stride, ..: anchor_here says which j meet one)
        const int kept = s.nc > an.phase ? (s.nc - 1 - an.phase) / an.stride + 1 : 1;
        const size_t bh = tiles ? ((size_t)b * kept + (zero ? 0 : (s.nc - j - an.phase) / an.stride)) * s.H + h
                                : (size_t)b * s.H + h;
        return (zero ? an.other_tiles : g) + (bh * s.P + pb * 32 + (lane0 & 31)) * N + 4 * (lane0 >> 5);
    };
    // one slice at a time, so that at most one slice of the other scan's state is held in registers
    // whether the two scans meet where this scan's tile j starts (j = nc: where it ends)
    auto anchor_here = [&](int j) {
        const int o = s.nc - j - an.phase;  // the other scan's tile that starts there, counted from its first kept one
        return j == 0 || j == s.nc || (o >= 0 && o % an.stride == 0);
    };
    auto load_other = [&](const float *g, int sl, float4 (&gq)[NB][4]) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) gq[nb][q4] = *reinterpret_cast<const float4 *>(g + sl * 32 * N + 32 * nb + 8 * q4);
        }
    };
    auto write_anchor = [&](int k, int sl, const float4 (&gq)[NB][4], bool zero) {
        double part = 0.0;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int sn = sl * NB + nb;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
                part += (double)st[sn][4 * q4] * gq[nb][q4].x + (double)st[sn][4 * q4 + 1] * gq[nb][q4].y +
                        (double)st[sn][4 * q4 + 2] * gq[nb][q4].z + (double)st[sn][4 * q4 + 3] * gq[nb][q4].w;
        }
        part = wave_inclusive_scan(zero ? 0.0 : part);
        if (lane0 == 63) an.out[(((size_t)b * (s.nc + 1) + (ADJ ? s.nc - k : k)) * s.H + h) * PBn + pb + sl] = part;
    };
    if constexpr (ANCH) {
        if (an.out != nullptr) {
            bool zero0;
            const float *g0 = adjoint_state(0, zero0);
            zero0 = zero0 || init == nullptr;  // no initial state: a zero anchor
#pragma unroll
            for (int sl = 0; sl < SL; ++sl) {
                float4 gq[NB][4];
                load_other(g0, sl, gq);
                write_anchor(0, sl, gq, zero0);
            }
        }
    }

    float seg_total = 1.f;  // product of the tiles' decays (KIND 2)
    // one tile; `set` (a compile-time 0 or 1) is the set of LDS tiles it uses; false when the scan ends inside it
    auto tile = [&](const int c, auto set) -> bool {
        constexpr int SET = decltype(set)::value;
        T *const Bs = Bs0 + SET * Q * N, *const Cs = Cs0 + SET * Q * N, *const xs_all = xs_all0 + SET * WAVES * XS;
        T *const xs = TR ? xs_all : xs_all + fused_scan_xtile_base(Q, wave);
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        // the state entering every tile, for a caller that needs it (the backward pass): [B, nc, H, P, N]
        // (of every an.stride-th tile from an.phase on, where the backward pass's other scan asks for fewer)
        if constexpr (TR) {
            if (tile_states && c >= an.phase && (c - an.phase) % an.stride == 0) {
                const int kept = (s.nc - 1 - an.phase) / an.stride + 1;
                store_state(tile_states + (((size_t)b * kept + (c - an.phase) / an.stride) * s.H + h) * s.P * N);
            }
        } else {  // (the other kinds keep every tile's)
            if (tile_states) store_state(tile_states + (((size_t)b * s.nc + c) * s.H + h) * s.P * N);
        }
        if (!kTwoSets) block_sync_lds();  // every wave is done reading the previous chunk's tiles
        // ---- registers -> LDS tiles ----
        // where the pieces go: the swizzle repeats every 32 rows, so all passes of a thread share the
        // offsets of its first (B, C) or first two (x: passes are 16 rows apart) rows
        const int tw = phase_tid();
        int bw[2], xw[2][2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            bw[hf] = BT::off(tw / BPR, (tw % BPR) * 8 + 4 * hf);
#pragma unroll
            for (int par = 0; par < 2; ++par)
                xw[par][hf] = fused_scan_xtile_base(Q, (tw % XPR) / 4) +
                              XT::off(tw / XPR + 16 * par, ((tw % XPR) % 4) * 8 + 4 * hf);
        }
        if constexpr (TR) {
#pragma unroll
            for (int u = 0; u < UX; ++u) {  // the eight heads' B and C rows, as the forward stages its x rows
                T *tb = tiles + xw[u & 1][0] + (u >> 1) * 1024, *tb1 = tiles + xw[u & 1][1] + (u >> 1) * 1024;
                *reinterpret_cast<uint2 *>(tb) = make_uint2(bq[u].x, bq[u].y);
                *reinterpret_cast<uint2 *>(tb1) = make_uint2(bq[u].z, bq[u].w);
                *reinterpret_cast<uint2 *>(tb + TRB) = make_uint2(cq[u].x, cq[u].y);
                *reinterpret_cast<uint2 *>(tb1 + TRB) = make_uint2(cq[u].z, cq[u].w);
            }
            if (tw < Q * 4 * SL) {
                const int col = (tw % (4 * SL)) * 8;
                XT::put16(xs_all + (col / 32) * XS, tw / (4 * SL), col % 32, xq[0]);
                if (TR_FWD) XT::put16(aux_s + (col / 32) * XS, tw / (4 * SL), col % 32, auxq);
            }
        }
#pragma unroll
        for (int u = 0; u < (TR ? 0 : UBC); ++u) {
            if (BSL % nthr == 0 || tw + u * nthr < BSL) {
                const int o0 = kSharedBcOffsets ? bw[0] + u * BRP * N : BT::off(tw / BPR + u * BRP, (tw % BPR) * 8);
                const int o1 = kSharedBcOffsets ? bw[1] + u * BRP * N : BT::off(tw / BPR + u * BRP, (tw % BPR) * 8 + 4);
                *reinterpret_cast<uint2 *>(Bs + o0) = make_uint2(bq[u].x, bq[u].y);
                *reinterpret_cast<uint2 *>(Bs + o1) = make_uint2(bq[u].z, bq[u].w);
                if (!STATES_ONLY) {
                    *reinterpret_cast<uint2 *>(Cs + o0) = make_uint2(cq[u].x, cq[u].y);
                    *reinterpret_cast<uint2 *>(Cs + o1) = make_uint2(cq[u].z, cq[u].w);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < (TR ? 0 : UX); ++u) {
            *reinterpret_cast<uint2 *>(xs_all + xw[u & 1][0] + (u >> 1) * 1024) = make_uint2(xq[u].x, xq[u].y);
            *reinterpret_cast<uint2 *>(xs_all + xw[u & 1][1] + (u >> 1) * 1024) = make_uint2(xq[u].z, xq[u].w);
        }
        // ---- scan of dt*A over the chunk and the decay tables of this unit ----
        float a_end;  // exp2(alpha[Q-1]): the chunk's total decay
        {
            const int lane = tw & 63;
            constexpr double kLog2e = 1.4426950408889634;
            float dtv[EPL], hi[EPL], lo[EPL];
            double cs[EPL], run = 0.0;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                dtv[e] = (float)__builtin_bit_cast(__bf16, dq[e]);
                run += (double)dtv[e] * a_h - (rq[e] ? kResetDrop : 0.0);
                if (ADJ) dtv[e] = (t0 + lane * EPL + e < s.L) ? 1.f : 0.f;  // from here on dtv is the input weight
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
                if (!STATES_ONLY && lane == 0) {
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
                    if constexpr (!STATES_ONLY) {
                        ah_s[l] = hi[e];
                        alo_s[l] = lo[e];
                        dt_s[l] = dtv[e];
                    }
                    w_s[l] = exp2_hw(fminf(alpha_diff(endh[QB - 1], endl[QB - 1], hi[e], lo[e]), 0.f)) * dtv[e];
                    if constexpr (!STATES_ONLY) {  // (phase 1's tables: the states-only pass has no phase 1)
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
        }
        if (kEarlyPrefetch && c + 1 < c_end) prefetch(c + 1);
        block_sync_lds();  // tiles and tables are visible

        if constexpr (kSharedScores) {
            if (wave < 3) {  // block g = sb + lb: (0,0), (0,1), (1,1)
                const int lane = phase_tid() & 63, r = lane & 31, half = lane >> 5;
                // (the wave index hidden from the compiler here: it would otherwise keep the sixteen addresses below,
                // which differ from the ones every wave uses by a wave-uniform offset only, in registers of their own
                // across the tile loop, and spill them)
                int pw = wave;
                asm volatile("" : "+s"(pw));
                const int psb = pw == 2 ? 1 : 0, plb = pw == 0 ? 0 : 1;
                Frag<T> Cp[NK], Bp[NK];
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) {
                    Cp[kk] = BT::split_frag(Cs + plb * 32 * N, r, 16 * kk + 4 * half);
                    Bp[kk] = BT::split_frag(Bs + psb * 32 * N, r, 16 * kk + 4 * half);
                }
                f32x16 sc = {0};
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) sc = mma32(Bp[kk], Cp[kk], sc);
                float *gd = G_s + pw * 1024 + lane * 4;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<float4 *>(gd + q * 256) = make_float4(sc[4 * q], sc[4 * q + 1], sc[4 * q + 2], sc[4 * q + 3]);
            }
            __builtin_amdgcn_sched_barrier(0);  // (the producers' fragments are dead before the state's operand form is made)
        }
        // ---- phase 1: outputs of this chunk from the state entering it ----
        if constexpr (!STATES_ONLY) {
            const int lane = phase_tid() & 63;
            const int r = lane & 31, half = lane >> 5;
            Frag<T> Hhi[SL * NK], Hlo[SL * NK];
#pragma unroll
            for (int sk = 0; sk < SL * NK; ++sk) {  // slice sk / NK, K step sk % NK
                const int kk = sk % NK, sn = (sk / NK) * NB + kk / 2;
                FragBits fh, fl;
                float sv[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) sv[i] = st[sn][8 * (kk % 2) + i];
                split8_keep(sv, fh.u, fl.u);
                Hhi[sk] = fh.frag();
                Hlo[sk] = fl.frag();
            }
            // masked, decayed scores of one s-block as hi/lo operands; fv = the block's four F vectors
            auto make_m = [&](const f32x16 &sc, const float4 (&fv)[4], bool masked, Frag<T>(&mh)[2], Frag<T>(&ml)[2]) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    FragBits fh, fl;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {  // accumulator registers v = 8 j + 2 k, + 1
                        const int v = 8 * j + 2 * k, vg = v / 4, i = v % 4;
                        const float f0 = i == 0 ? fv[vg].x : fv[vg].z, f1 = i == 0 ? fv[vg].y : fv[vg].w;
                        float s0 = sc[v], s1 = sc[v + 1];
                        if (masked) {  // causal mask inside the diagonal block: row 8 vg + 4 half + i <= column r
                            s0 = (8 * vg + 4 * half + i <= r) ? s0 : 0.f;
                            s1 = (8 * vg + 4 * half + i + 1 <= r) ? s1 : 0.f;
                        }
                        split_pair(s0, f0, s1, f1, fh.u[k], fl.u[k]);
                    }
                    mh[j] = fh.frag();
                    ml[j] = fl.frag();
                }
            };
            // rolled where registers are tight; the 128-wide-state instance has a wave's whole register file
            constexpr int kUnrollBlocks = (NK == 8 || ((KIND == 0 || KIND == 5) && WAVES == 8)) ? QB : 1;
#pragma unroll kUnrollBlocks
            for (int lb = 0; lb < QB; ++lb) {
                const int l = lb * 32 + r;
                // non-negative floats order like their bit patterns: a scalar compare
                const bool fast = __builtin_amdgcn_readfirstlane(__float_as_int(blk_s[8 + lb])) <= __float_as_int(kFastDiagSpan);
                // KIND 5: this lane's pieces of the second operand's rows and the rows' dt, requested here and used in
                // the epilogue (lane = (row l, half): elements 8 vg + 4 half .. + 3 of the head's row)
                uint2 aq[4] = {make_uint2(0, 0), make_uint2(0, 0), make_uint2(0, 0), make_uint2(0, 0)};
                float wt = 1.f;
                if constexpr (TR_ADJ) {
                    // the heads' dt of this block's rows (dB sums the heads' outputs weighted by it), requested here and
                    // used in the epilogue; a row outside the sequence reads a row inside it and weighs zero
                    const int trow = s.L - 1 - (t0 + l);
                    wt = (float)dt[((size_t)b * trows + min(max(trow, 0), trows - 1)) * s.H + h];
                }
                if constexpr (ROWS) {
                    // (no condition on the loads: a row outside the sequence reads a row inside it, and nothing of it is
                    // stored -- under a condition the loads sit in a block of their own where the wave waits for them)
                    const int arow = min(max(s.L - 1 - (t0 + l), 0), trows - 1);
                    const T *ar = aux + ((size_t)b * trows + arow) * HP + h * s.P + pb * 32 + 4 * half;
#pragma unroll
                    for (int vg = 0; vg < 4; ++vg) aq[vg] = *reinterpret_cast<const uint2 *>(ar + 8 * vg);
                    wt = (float)dt[((size_t)b * trows + arow) * s.H + h];
                }
                // The tiles' swizzles repeat every 32 rows, so a row's address is its block's base plus the offset of
                // the row inside its block -- the same lane-derived offsets for every block, B or C tile alike, which
                // stay in registers across the blocks and tiles (computed from the full row index they were formed
                // again per block: 50 address instructions per column block).
                const T *const Cs_lb = Cs + lb * 32 * N, *const xs_lb = xs + lb * 32 * 32;
                Frag<T> Cf[NK];
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) Cf[kk] = BT::split_frag(Cs_lb, r, 16 * kk + 4 * half);
                f32x16 accs[SL];  // one output tile per slice
#pragma unroll
                for (int sl = 0; sl < SL; ++sl) {
                    accs[sl] = f32x16{0};
#pragma unroll
                    for (int kk = 0; kk < NK; ++kk) {
                        accs[sl] = mma32(Hhi[sl * NK + kk], Cf[kk], accs[sl]);
#ifndef SSD_ABLATE_STATE_LO
                        accs[sl] = mma32(Hlo[sl * NK + kk], Cf[kk], accs[sl]);
#endif
                    }
                    accs[sl] = accs[sl] * blk_s[lb];
                }
                if constexpr (kSharedScores) {
                    if (lb == 0) block_sync_lds();  // the three blocks of scores are in LDS
                }
                f32x16 &acc = accs[0];
                const float *F_row = F_s + lb * Q;
                // one s-block.  On the separable path the diagonal block is one more term of the sum that E[l]
                // scales at the end; on the exact path the sum is scaled first and the block carries its full factors.
                auto block = [&](int sb, bool diag) {
                    f32x16 sc = {0};
                    if constexpr (kSharedScores) {
                        const float *gs = G_s + (sb + lb) * 1024 + lane * 4;
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float4 t = *reinterpret_cast<const float4 *>(gs + q * 256);
                            sc[4 * q] = t.x;
                            sc[4 * q + 1] = t.y;
                            sc[4 * q + 2] = t.z;
                            sc[4 * q + 3] = t.w;
                        }
                    } else {
                        Frag<T> Bf[NK];
#pragma unroll
                        for (int kk = 0; kk < NK; ++kk) Bf[kk] = BT::split_frag(Bs + sb * 32 * N, r, 16 * kk + 4 * half);
#pragma unroll
                        for (int kk = 0; kk < NK; ++kk) sc = mma32(Bf[kk], Cf[kk], sc);
                    }
                    // requested while the score MFMAs run
                    Frag<T> xf[SL][2];
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) {
#pragma unroll
                        for (int j = 0; j < 2; ++j)  // K order of mh[j]: rows 32 sb + 16 j + 4 half + {0..3} and the same + 8
                            xf[sl][j] = XT::frag(xs + sl * XS + sb * 32 * 32, 16 * j + 4 * half, 8, 0, lane);
                    }
                    float4 fv[4];
                    if (!diag || fast) {
#pragma unroll
                        for (int vg = 0; vg < 4; ++vg) fv[vg] = *reinterpret_cast<const float4 *>(F_row + sb * 32 + 8 * vg + 4 * half);
                    }
                    float El = 1.f, Eend = 1.f;  // Eend: what scales the finished sum (1 on the exact path, which scales first)
                    if (diag) {
                        El = E_s[l];
                        Eend = fast ? El : 1.f;
                        if (!fast) {
#pragma unroll
                            for (int sl = 0; sl < SL; ++sl) accs[sl] = accs[sl] * El;
                            const float al_hi = ah_s[l], al_lo = alo_s[l];
#pragma unroll
                            for (int vg = 0; vg < 4; ++vg) {
                                const int s0 = lb * 32 + 8 * vg + 4 * half;
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
                    }
                    Frag<T> mh[2], ml[2];
                    make_m(sc, fv, diag, mh, ml);
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) {
#pragma unroll
                        for (int j = 0; j < 2; ++j) {
                            accs[sl] = mma32(xf[sl][j], mh[j], accs[sl]);
#ifndef SSD_ABLATE_M_LO
                            accs[sl] = mma32(xf[sl][j], ml[j], accs[sl]);
#endif
                        }
                        if (diag) accs[sl] = accs[sl] * Eend;  // everything summed so far shares the factor E[l]
                    }
                };
                // compile-time block index: every LDS address is a lane offset plus an immediate
#pragma unroll
                for (int sb = 0; sb < QB - 1; ++sb)
                    if (sb < lb) block(sb, false);
                block(lb, true);
                if constexpr (TR) {
                    // this head's tile goes into the workgroup's sum; acc[4 vg + i] is element (t = 32 lb + lane%32,
                    // p = 8 vg + 4 half + i)
                    const int le = phase_tid() & 63, he = le >> 5, ll = lb * 32 + (le & 31);
                    const int trow = ADJ ? s.L - 1 - (t0 + ll) : t0 + ll;
                    const bool live = ll < rows && trow >= 0 && trow < trows;
                    if (TR_ADJ) wt = live ? wt : 0.f;
#pragma unroll
                    for (int sl = 0; sl < SL; ++sl) {
                        float part = 0.f;  // forward: this slice's part of C_t . y_t
                        // where this lane's 16 elements of the head's tile go (two slices: tiles of 32 rows, side by side)
                        float *rw = SL == 2 ? red + (wave * 32 + (le & 31)) * RS : red + (wave * Q + ll) * RS;
#pragma unroll
                        for (int vg = 0; vg < 4; ++vg) {
                            if (TR_FWD && aux != nullptr) {
                                const bf16x4 c4 = XT::row4(aux_s + sl * XS, ll, 8 * vg + 4 * he);
#pragma unroll
                                for (int i = 0; i < 4; ++i) part += accs[sl][vg * 4 + i] * (float)c4[i];
                            }
                            if constexpr (SL == 2) {  // logical piece 8 sl + 2 vg + he of the row
                                *reinterpret_cast<float4 *>(rw + 4 * ((8 * sl + 2 * vg + he) ^ (le & 15))) =
                                    make_float4(wt * accs[sl][vg * 4], wt * accs[sl][vg * 4 + 1], wt * accs[sl][vg * 4 + 2],
                                                wt * accs[sl][vg * 4 + 3]);
                            } else {
#pragma unroll
                                for (int i = 0; i < 4; ++i) rw[8 * vg + 4 * he + i] = wt * accs[sl][vg * 4 + i];
                            }
                        }
                        if (TR_FWD && seg_decay != nullptr) {  // (seg_decay: the per-head parts [B, L, H, P/32])
                            part += __shfl_xor(part, 32, 64);
                            if (he == 0 && live) seg_decay[(((size_t)b * trows + trow) * s.H + h) * PBn + pb + sl] = part;
                        }
                    }
                    if constexpr (SL == 2) {
                        // the sum over the workgroup's heads of these 32 rows, [32][64], goes to the group's rows of
                        // the gradient: 4 elements per thread
                        block_sync_lds();
                        const int tq = phase_tid();
                        const int row = tq >> 4, c4 = (tq & 15) * 4;
                        float v0 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f;
#pragma unroll
                        for (int wv = 0; wv < WAVES; ++wv) {  // heads in order
                            const float4 rr = *reinterpret_cast<const float4 *>(red + (wv * 32 + row) * RS + 4 * ((tq & 15) ^ (row & 15)));
                            v0 += rr.x;
                            v1 += rr.y;
                            v2 += rr.z;
                            v3 += rr.w;
                        }
                        const int lr = lb * 32 + row;
                        const int orow = ADJ ? s.L - 1 - (t0 + lr) : t0 + lr;
                        if (lr < rows && orow >= 0 && orow < trows)
                            *reinterpret_cast<uint2 *>(y + ((size_t)b * trows + orow) * XLD + xcol + c4) =
                                make_uint2(pack_bf16x2(v0, v1), pack_bf16x2(v2, v3));
                        if (lb + 1 < QB) block_sync_lds();  // the next block of rows overwrites the tiles
                    }
                } else if constexpr (ROWS) {
                    // epilogue: dx[t, h, p] = dt[t, h] * rT[p, l] + D[h] * x[t, h, p], and the row's two inner products
                    const int le = phase_tid() & 63, he = le >> 5, ll = lb * 32 + (le & 31);
                    float o[16], pe = 0.f, pd = 0.f;
#pragma unroll
                    for (int vg = 0; vg < 4; ++vg) {
                        const bf16x4 x4 = XT::row4(xs_lb, le & 31, 8 * vg + 4 * he);
                        const bf16x4 a4 = __builtin_bit_cast(bf16x4, aq[vg]);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            o[vg * 4 + i] = wt * acc[vg * 4 + i] + dh * (float)x4[i];
                            pe += acc[vg * 4 + i] * (float)a4[i];
                            pd += (float)x4[i] * (float)a4[i];
                        }
                    }
                    pe += __shfl_xor(pe, 32, 64);
                    pd += __shfl_xor(pd, 32, 64);
                    const int yrow = s.L - 1 - (t0 + ll);
                    const bool live = ll < rows && yrow >= 0 && yrow < trows;
                    store_column_buffer<TO>(ybuf, (unsigned)yrow * (unsigned)(HP * sizeof(TO)) + ycol_bytes, o, he, live);
                    if (he == 0 && live)
                        *reinterpret_cast<float2 *>(seg_decay + 2 * (((size_t)b * trows + yrow) * s.H + h)) = make_float2(pe, pd);
                } else {
                    // epilogue: y[t, h, p] = yT[p, l] + D[h] * x[t, h, p]
                    const int le = phase_tid() & 63, he = le >> 5, ll = lb * 32 + (le & 31);
                    float o[16];
#pragma unroll
                    for (int vg = 0; vg < 4; ++vg) {
                        const bf16x4 x4 = XT::row4(xs_lb, le & 31, 8 * vg + 4 * he);
#pragma unroll
                        // (an explicit fused multiply-add: left to the compiler, the scaling of acc by E[l] just above and
                        // this sum contract one way in the bf16-y instance and the other in the float-y one, and the
                        // stored bf16 y is no longer the float y rounded once)
                        for (int i = 0; i < 4; ++i) o[vg * 4 + i] = __builtin_fmaf(dh, (float)x4[i], acc[vg * 4 + i]);
                    }
                    const int yrow = ADJ ? s.L - 1 - (t0 + ll) : t0 + ll;
                    store_column_buffer<TO>(ybuf, (unsigned)yrow * (unsigned)(HP * sizeof(TO)) + ycol_bytes, o, he,
                                            ll < rows && (!ADJ || (yrow >= 0 && yrow < trows)));
                }
            }
        }

        if constexpr (TR && SL == 1) {
            // the sum over the workgroup's heads (a whole group: eight heads) of this tile's outputs, [Q][32], goes
            // to the group's rows of the gradient
            block_sync_lds();
            const int tq = phase_tid();
            const int ll = tq >> 3, p4 = (tq & 7) * 4;
            float v0 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) {  // heads in order
                const float *rr = red + (wv * Q + ll) * 33 + p4;
                v0 += rr[0];
                v1 += rr[1];
                v2 += rr[2];
                v3 += rr[3];
            }
            const int trow = ADJ ? s.L - 1 - (t0 + ll) : t0 + ll;
            if (ll < rows && trow >= 0 && trow < trows) {
                TO *dst = y + ((size_t)b * trows + trow) * XLD + xcol + p4;
                if constexpr (sizeof(TO) == 2) {
                    *reinterpret_cast<uint2 *>(dst) = make_uint2(pack_bf16x2(v0, v1), pack_bf16x2(v2, v3));
                } else {
                    *reinterpret_cast<float4 *>(dst) = make_float4(v0, v1, v2, v3);
                }
            }
        }
        // ---- phase 2: the state leaving this chunk ----
        // (the forward's last tile of a segment other than the last, or of a call that asks for no final state: nobody
        // reads the state it leaves)
        if (KIND == 0 && c + 1 == c_end && !(final_states != nullptr && seg == S - 1)) return false;
        if (!kEarlyPrefetch && c + 1 < c_end) prefetch(c + 1);
        // the other scan's state where this tile ends: the first slice in flight during phase 2, the second (two
        // slices per wave leave no registers to hold both) requested after it
        float4 gq[ANCH ? NB : 1][4];
        bool gzero = false;
        const float *gnext = nullptr;
        const bool anchor_next = ANCH && an.out != nullptr && anchor_here(c + 1);
        if constexpr (ANCH) {
            if (anchor_next) {
                gnext = adjoint_state(c + 1, gzero);
                load_other(gnext, 0, gq);
            }
        }
        seg_total *= a_end;
        const int lane = phase_tid() & 63, half = lane >> 5;
#pragma unroll
        for (int sn = 0; sn < SL * NB; ++sn) st[sn] = st[sn] * a_end;
        // Offsets of this lane's transposing reads for K steps 0 and 1.  Both swizzles repeat every 32 rows, so
        // step i reads at the offset of step i%2 plus (i/2)*32 rows: immediates after unrolling.
        int xo[2][2], bo[2][2][NB];
#pragma unroll
        for (int par = 0; par < 2; ++par) {
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                xo[par][z] = XT::tr_off(16 * par + 8 * half + 4 * z, 0, lane);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) bo[par][z][nb] = BT::tr_off(16 * par + 8 * half + 4 * z, nb * 32, lane);
            }
        }
        auto join = [](const bf16x4 &lo, const bf16x4 &hi) {
            Frag<T> fr;
            fr.v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return fr;
        };
#pragma unroll
        for (int ks = 0; ks < Q; ks += 16) {
            const int k0 = ks + 8 * half;
            const int par = (ks / 16) & 1, rb = (ks / 32) * 32;
            // x[l = k0..k0+7, p = r] and B[l = k0..k0+7, n = 32 nb + r]
            Frag<T> xr[SL];
#pragma unroll
            for (int sl = 0; sl < SL; ++sl)
                xr[sl] = join(XT::tr_read(xs + sl * XS + xo[par][0] + rb * 32), XT::tr_read(xs + sl * XS + xo[par][1] + rb * 32));
            Frag<T> bf[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
                bf[nb] = join(BT::tr_read(Bs + bo[par][0][nb] + rb * N), BT::tr_read(Bs + bo[par][1][nb] + rb * N));
            const float4 wa = *reinterpret_cast<const float4 *>(w_s + k0);
            const float4 wb = *reinterpret_cast<const float4 *>(w_s + k0 + 4);
            const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
            for (int sl = 0; sl < SL; ++sl) {
                FragBits xh, xl;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    split_pair((float)xr[sl].v[2 * i], wv[2 * i], (float)xr[sl].v[2 * i + 1], wv[2 * i + 1], xh.u[i], xl.u[i]);
                const Frag<T> xhf = xh.frag(), xlf = xl.frag();
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    st[sl * NB + nb] = mma32(bf[nb], xhf, st[sl * NB + nb]);
#ifndef SSD_ABLATE_WX_LO
                    st[sl * NB + nb] = mma32(bf[nb], xlf, st[sl * NB + nb]);
#endif
                }
            }
        }
        if constexpr (ANCH) {
            if (anchor_next) {
                // (the other scan's values are used from here on, not before: left alone, the compiler converts them to
                // float64 right behind their loads, in front of phase 2, and the wave waits for them there)
                auto pin = [&](float4 (&q)[NB][4]) {
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4)
                            asm volatile("" : "+v"(q[nb][q4].x), "+v"(q[nb][q4].y), "+v"(q[nb][q4].z), "+v"(q[nb][q4].w));
                    }
                };
                pin(gq);
                // the second slice is requested here and arrives during the first slice's sums (requested ahead of phase
                // 2 with the first, the compiler copies registers right behind the loads and waits for them there)
                float4 gq1[SL == 2 ? NB : 1][4];
                if constexpr (SL == 2) load_other(gnext, 1, gq1);
                write_anchor(c + 1, 0, gq, gzero);
                if constexpr (SL == 2) {
                    pin(gq1);
                    write_anchor(c + 1, 1, gq1, gzero);
                }
            }
        }
        return true;
    };
    // Nothing in flight when the tile loop is entered: the wait for a tile's inputs at the loop's head is then counted
    // from the loop's own path alone -- they are older than the tile's stores of y, so the wave need not wait for
    // those to be acknowledged -- instead of from the prologue's, where they are the youngest requests.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    if constexpr (kTwoSets) {
        for (int c = c_first; c < c_end; c += 2) {
            if (!tile(c, std::integral_constant<int, 0>{})) break;
            if (c + 1 < c_end && !tile(c + 1, std::integral_constant<int, 1>{})) break;
        }
    } else {
        for (int c = c_first; c < c_end; ++c)
            if (!tile(c, std::integral_constant<int, 0>{})) break;
    }

    if (STATES_ONLY) {
        store_state(final_states + (((size_t)b * S + seg) * s.H + h) * s.P * N);
        if (pb == 0 && lane0 == 0) seg_decay[((size_t)b * S + seg) * s.H + h] = seg_total;
    } else if (final_states && seg == S - 1) {
        store_state(final_states + ((size_t)b * s.H + h) * s.P * N);
    }
}

// ------------------------------------------------------------------------------------------
// Launchers (one translation unit per output type instantiates fused_dispatch)
// ------------------------------------------------------------------------------------------
template <typename TO, int NK, int QB, int WAVES>
static hipError_t fused_launch(const ScanShape &s, const void *x, const void *dt, const float *A, const void *Bm,
                               const void *Cm, const float *D, const float *init, const unsigned char *reset, void *y,
                               float *final_states, float *tile_states, hipStream_t st) {
    const int units = (s.H / s.G) * (s.P / 32);
    const int segments = s.seg_tiles > 0 ? (s.nc + s.seg_tiles - 1) / s.seg_tiles : 1;
    const int grid = s.B * s.G * (units / WAVES) * segments;
    const __bf16 *xx = static_cast<const __bf16 *>(x), *dd = static_cast<const __bf16 *>(dt);
    const __bf16 *bb = static_cast<const __bf16 *>(Bm), *cc = static_cast<const __bf16 *>(Cm);
    if (s.mode != 0) {
        // the reversed-adjoint mode serves the backward pass, which takes float outputs only
        if constexpr (sizeof(TO) == 4) {
            if (segments != 1) return hipErrorInvalidValue;
            fused_scan_kernel<TO, NK, QB, WAVES, 1><<<dim3(grid), dim3(64 * WAVES), 0, st>>>(
                xx, dd, A, bb, cc, D, init, reset, static_cast<TO *>(y), final_states, tile_states, nullptr, nullptr, s, ScanAnchors{});
            return hipGetLastError();
        } else {
            return hipErrorInvalidValue;
        }
    }
    fused_scan_kernel<TO, NK, QB, WAVES, 0><<<dim3(grid), dim3(64 * WAVES), 0, st>>>(
        xx, dd, A, bb, cc, D, init, reset, static_cast<TO *>(y), final_states, tile_states, nullptr, nullptr, s, ScanAnchors{});
    return hipGetLastError();
}

// States only (KIND 2): per segment, the state it leaves behind from `init` ([B,S,H,P,N] or NULL = zero) into
// seg_states [B,S,H,P,N] and its total decay into seg_decay [B,S,H].
template <int NK, int QB, int WAVES>
static hipError_t fused_launch_states(const ScanShape &s, const void *x, const void *dt, const float *A, const void *Bm,
                                      const float *init, const unsigned char *reset, float *seg_states, float *seg_decay,
                                      hipStream_t st) {
    const int units = (s.H / s.G) * (s.P / 32);
    const int segments = s.seg_tiles > 0 ? (s.nc + s.seg_tiles - 1) / s.seg_tiles : 1;
    const int grid = s.B * s.G * (units / WAVES) * segments;
    const __bf16 *bb = static_cast<const __bf16 *>(Bm);
    fused_scan_kernel<__bf16, NK, QB, WAVES, 2><<<dim3(grid), dim3(64 * WAVES), 0, st>>>(
        static_cast<const __bf16 *>(x), static_cast<const __bf16 *>(dt), A, bb, bb, nullptr, init, reset, nullptr, seg_states,
        nullptr, seg_decay, nullptr, s, ScanAnchors{});
    return hipGetLastError();
}

// The backward pass's scans of the transposed state (KIND 3 forward in time, 4 reversed-adjoint): s is the
// transposed shape (P = the forward's dstate, N = 32 = its headdim, G = H), x [B,L,x_groups,P] the operand the
// heads of a group share, Bm, Cm [B,L,H,32] per head; out [B,L,x_groups,P] receives the sum over each group's
// eight heads of the per-head outputs (weighted by dt in KIND 4); KIND 3 also writes, per head and 32-column
// slice, aux_t . y_t into parts [B,L,H,P/32] (aux [B,L,x_groups,P]), and the anchors `an` asks for.
template <typename TO, int KIND>
static hipError_t fused_launch_transposed(const ScanShape &s, const void *x, const void *dt, const float *A, const void *Bm,
                                          const void *Cm, const void *aux, const float *init, const unsigned char *reset,
                                          void *out, float *final_states, float *tile_states, float *parts,
                                          const ScanAnchors &an, hipStream_t st) {
    if (s.N != 32 || s.G != s.H || s.x_groups <= 0 || s.H != 8 * s.x_groups || s.P % 32 != 0 || s.seg_tiles != 0)
        return hipErrorInvalidValue;
    constexpr bool kWide = KIND == 6 || KIND == 7;  // both slices of a 64-wide state in one wave
    if (kWide && s.P != 64) return hipErrorInvalidValue;
    const int grid = s.B * (s.H / 8) * (kWide ? 1 : s.P / 32);
    fused_scan_kernel<TO, 2, kOnePassTile / 32, 8, KIND><<<dim3(grid), dim3(512), 0, st>>>(
        static_cast<const __bf16 *>(x), static_cast<const __bf16 *>(dt), A, static_cast<const __bf16 *>(Bm),
        static_cast<const __bf16 *>(Cm), nullptr, init, reset, static_cast<TO *>(out), final_states, tile_states, parts,
        static_cast<const __bf16 *>(aux), s, an);
    return hipGetLastError();
}

// The reversed-adjoint scan with the row products (KIND 5): x, Bm, Cm, dt, aux are the forward sequence's tensors
// (s.dt_len rows, s.L the padded length of the reversed sequence); dx [B,L,H,32] bf16, pairs float2 [B,L,H].
template <int NK>
static hipError_t fused_launch_adjoint_rows(const ScanShape &s, const void *x, const void *dt, const float *A, const void *Bm,
                                            const void *Cm, const float *D, const void *aux, const float *init,
                                            const unsigned char *reset, void *dx, float *final_states, float *pairs,
                                            hipStream_t st) {
    const int units = (s.H / s.G) * (s.P / 32);
    if (s.P != 32 || units % 8 != 0 || s.seg_tiles != 0 || s.x_groups != 0 || s.N != 16 * NK || aux == nullptr ||
        pairs == nullptr)
        return hipErrorInvalidValue;
    const int grid = s.B * s.G * (units / 8);
    fused_scan_kernel<__bf16, NK, kOnePassTile / 32, 8, 5><<<dim3(grid), dim3(512), 0, st>>>(
        static_cast<const __bf16 *>(x), static_cast<const __bf16 *>(dt), A, static_cast<const __bf16 *>(Bm),
        static_cast<const __bf16 *>(Cm), D, init, reset, static_cast<__bf16 *>(dx), final_states, nullptr, pairs,
        static_cast<const __bf16 *>(aux), s, ScanAnchors{});
    return hipGetLastError();
}

template <typename TO, int NK, int QB>
static hipError_t fused_dispatch_w(const ScanShape &s, int waves, const void *x, const void *dt, const float *A,
                                   const void *Bm, const void *Cm, const float *D, const float *init,
                                   const unsigned char *reset, void *y, float *final_states, float *tile_states,
                                   hipStream_t st) {
    if constexpr (NK == 8) {
        // a 128-wide state: four waves per workgroup, one per SIMD, each with the whole register file
        if (waves == 4)
            return fused_launch<TO, NK, QB, 4>(s, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
        return hipErrorInvalidValue;
    } else {  // (an else, so that no eight-wave kernel is instantiated for the 128-wide state)
        if (waves == 8)
            return fused_launch<TO, NK, QB, 8>(s, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
        if (waves == 4)
            return fused_launch<TO, NK, QB, 4>(s, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
        // two waves: one head of 64 columns with its own B and C (the transposed scans of the backward pass);
        // the staging offsets fit a 32-wide state only, and only the float-output library instantiates it
        if constexpr (NK == 2 && sizeof(TO) == 4) {
            if (waves == 2)
                return fused_launch<TO, NK, QB, 2>(s, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
        }
        return hipErrorInvalidValue;
    }
}

template <typename TO>
hipError_t fused_dispatch(const ScanShape &s, int waves, const void *x, const void *dt, const float *A,
                          const void *Bm, const void *Cm, const float *D, const float *init,
                          const unsigned char *reset, void *y, float *final_states, float *tile_states, hipStream_t st) {
#define SSD_FUSED_CASE(NKv, QBv) \
    if (s.N == 16 * NKv && s.Q == 32 * QBv) \
        return fused_dispatch_w<TO, NKv, QBv>(s, waves, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
    SSD_FUSED_CASE(2, kOnePassTile / 32)
    SSD_FUSED_CASE(4, kOnePassTile / 32)
    SSD_FUSED_CASE(8, kOnePassTile / 32)
#undef SSD_FUSED_CASE
    return hipErrorInvalidValue;
}

}  // namespace ssd
