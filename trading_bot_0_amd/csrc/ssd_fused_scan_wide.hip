// The one-pass forward for a 128-wide state (gfx950, bf16 inputs): two waves per unit.
//
// fused_scan_kernel keeps a unit's running state H^T [N x 32] in one wave's accumulators.  At N = 128 that is 64
// registers, its hi/lo operand form 128 more, and the wave needs the whole register file of its SIMD: one wave per
// SIMD, nothing to fill the issue slots while it waits for its own MFMAs, LDS reads and barriers (a tile of 64 steps
// took 11 800 cycles for 5 700 of vector and 3 200 of matrix issue).  Here a unit -- 32 head-dim columns of one head
// of one batch row -- belongs to TWO waves on the same SIMD, 256 registers each:
//   * each holds half of the state (64 of the 128 state columns, 32 accumulator registers) and, in phase 2, adds the
//     tile's B^T . (w o x) to its half;
//   * the state readout C . H of a tile is divided by the state dimension: each wave splits its own half into hi + lo
//     bf16 operands in registers and multiplies it by its 64 columns of C for BOTH 32-step output blocks; the partial
//     sum of the block that is not its own goes to the other wave through LDS (4 KB each way per tile, at the barrier
//     the workgroup holds anyway; the state's operand form through LDS would be 16 KB written and 32 KB read);
//   * the rest of phase 1 is divided by output block: wave 0 of the unit produces the tile's first 32 timesteps (the
//     diagonal score block), wave 1 the second 32 (one block below the diagonal, the diagonal block) -- so the masked,
//     decayed score tiles, the part of a tile's work that does not shrink with the state, are each formed once.
// A workgroup is four units (eight waves, two per SIMD: wave w and w + 4 are the two halves of unit w, on SIMD w),
// sharing the B and C tiles of their (batch, group) as before.  The scan of dt*A and the decay tables of a unit are
// computed by its first wave for both (250 vector instructions, about what the second wave's extra score block costs).
//
// Everything else -- tiling of time by 64 steps whatever chunk length the caller names, the separable decay factors
// with the exact path for blocks that decay by more than 2^-120, hi + lo operands for everything the kernel
// manufactures, restarts as a drop of the cumulative log-decay, ragged last tiles, swizzled LDS tiles read with the
// transposing load -- is fused_scan_kernel's, whose comments explain it.
#include "ssd_fused_scan.h"

namespace ssd {

namespace {

constexpr int kWideN = 128, kWideNK = 8, kWideUnits = 4, kWideWaves = 8, kWideQ = kOnePassTile, kWideQB = kWideQ / 32;
// LDS: B and C tiles [Q][128], four x tiles [Q][32], the partial readout sums the two waves of a unit hand each other
// ([unit][sending wave][quarter][lane] 16 bytes, the accumulator's layout), per-unit tables
constexpr int kWideTableFloats = (5 + kWideQB) * kWideQ + 16;
// (the x tiles keep the eight-unit layout's offsets, fused_scan_xtile_base: by the hardware's bank-conflict counter the
// staging writes of four units are free of conflicts with them, and were not with the second pair of units 128 instead
// of 64 bytes further)
constexpr int kWideXArea = kWideUnits * fused_scan_xtile_elems(kWideQ);
// ... and the tile's three blocks of scores B . C^T, which the workgroup's four units share (one group's B and C): three
// waves form a block each, in the accumulator's layout ([block][quarter][lane] 16 bytes), and every wave reads its blocks
constexpr size_t kWideLdsBytes = (size_t)2 * kWideQ * kWideN * 2 + (size_t)kWideXArea * 2 +
                                 (size_t)kWideUnits * 2 * 32 * 32 * 4 + (size_t)kWideUnits * kWideTableFloats * 4 +
                                 (size_t)3 * 32 * 32 * 4;

template <typename TO>
__global__ __launch_bounds__(64 * kWideWaves, 1) void fused_scan_wide_kernel(
    const __bf16 *__restrict__ x, const __bf16 *__restrict__ dt, const float *__restrict__ A,
    const __bf16 *__restrict__ Bm, const __bf16 *__restrict__ Cm, const float *__restrict__ D, const float *init,
    const unsigned char *__restrict__ reset, TO *__restrict__ y, float *final_states, ScanShape s) {
    using T = __bf16;
    constexpr int N = kWideN, NK = kWideNK, Q = kWideQ, QB = kWideQB, nthr = 64 * kWideWaves, UNITS = kWideUnits;
    constexpr int HNB = 2;                     // 32-column blocks of this wave's half of the state
    constexpr int BPR = N / 8;                 // 16-byte pieces per B (or C) row
    constexpr int UBC = Q * BPR / nthr;        // passes over a B (or C) tile: 32 rows each
    constexpr int BRP = nthr / BPR;
    constexpr int XPR = UNITS * 4;             // 16-byte pieces of one timestep's x for the workgroup
    constexpr int XRP = nthr / XPR;            // x rows per pass: 32
    constexpr int UX = Q / XRP;
    static_assert(BRP == 32 && XRP == 32 && UBC == 2 && UX == 2, "staging offsets rely on the swizzle period of 32 rows");
    using XT = ChunkTile<32>;
    using BT = ChunkTile<N>;
    __shared__ __attribute__((aligned(16))) unsigned char smem[kWideLdsBytes];
    const int tid = threadIdx.x;
    const int lane0 = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ul = wave & 3, role = wave >> 2;  // the unit within the workgroup; which half of it this wave is
    T *const Bs = reinterpret_cast<T *>(smem);
    T *const Cs = Bs + Q * N;
    T *const xs_all = Cs + Q * N;
    // what a unit's two waves hand each other: each one's readout of ITS half of the state for the OTHER's output block,
    // in the accumulator's layout ([unit][wave of the unit][quarter][lane] 16 bytes)
    float *const part_all = reinterpret_cast<float *>(xs_all + kWideXArea);
    float *const wf = part_all + UNITS * 2 * 1024 + ul * kWideTableFloats;  // (per unit)
    float *const G_s = part_all + UNITS * 2 * 1024 + UNITS * kWideTableFloats;
    float *ah_s = wf, *alo_s = wf + Q, *dt_s = wf + 2 * Q, *w_s = wf + 3 * Q, *E_s = wf + 4 * Q, *F_s = wf + 5 * Q;
    float *blk_s = wf + (5 + QB) * Q;  // [0..QB): exp2(alpha[32 lb]); [4]: exp2(alpha[Q-1]); [8..8+QB): log2-decay across block lb
    T *const xs = xs_all + fused_scan_xtile_base(Q, ul);
    float *const part_unit = part_all + ul * 2 * 1024;

    // ---- which units this workgroup owns ----
    const int PBn = s.P / 32, HG = s.H / s.G;
    const int UW = (HG * PBn) / UNITS;  // workgroups per (batch, group)
    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    const int b = logical / (s.G * UW), g = (logical / UW) % s.G;
    const int unit0 = (logical % UW) * UNITS, unit = unit0 + ul;
    const int h = g * HG + unit / PBn, pb = unit % PBn;
    const int HP = s.H * s.P;
    const int xcol0 = g * HG * s.P + unit0 * 32;  // first element of the workgroup's slice of an x row
    const T *xb = x + (size_t)b * s.L * HP + xcol0;
    const T *Bb = Bm + ((size_t)b * s.L * s.G + g) * N;
    const T *Cb = Cm + ((size_t)b * s.L * s.G + g) * N;
    const T *dtb = dt + (size_t)b * s.L * s.H + h;
    const unsigned char *rsb = reset ? reset + (size_t)b * s.L : nullptr;
    const __amdgpu_buffer_rsrc_t ybuf = make_buffer(y + (size_t)b * s.L * HP, (unsigned)((size_t)s.L * HP * sizeof(TO)));
    const unsigned ycol_bytes = (unsigned)((h * s.P + pb * 32) * sizeof(TO));
    const float dh = D ? D[h] : 0.f;
    const double a_h = (double)A[h];

    // ---- registers holding the next tile's inputs ----
    uint4 bq[UBC], cq[UBC], xq[UX];
    unsigned short dq;
    unsigned char rq;
    auto prefetch = [&](int c) {
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        const int bc_row0 = tid / BPR, x_row0 = tid / XPR;
        const unsigned bc_off0 = bc_row0 * s.G * N + (tid % BPR) * 8;
        const unsigned x_off0 = x_row0 * HP + (tid % XPR) * 8;
        const T *bp = Bb + (size_t)t0 * s.G * N, *cp = Cb + (size_t)t0 * s.G * N;
        const T *xp = xb + (size_t)t0 * HP, *dp = dtb + (size_t)t0 * s.H;
        // (a conditional expression over *ptr and a zero constant would become a load through a selected pointer)
        auto ld16 = [](const T *ptr, bool ok) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ok) v = *reinterpret_cast<const uint4 *>(ptr);
            return v;
        };
        if (rows == Q) {
#pragma unroll
            for (int u = 0; u < UBC; ++u) {
                bq[u] = *reinterpret_cast<const uint4 *>(bp + (size_t)u * BRP * s.G * N + bc_off0);
                cq[u] = *reinterpret_cast<const uint4 *>(cp + (size_t)u * BRP * s.G * N + bc_off0);
            }
#pragma unroll
            for (int u = 0; u < UX; ++u) xq[u] = *reinterpret_cast<const uint4 *>(xp + (size_t)u * XRP * HP + x_off0);
            dq = __builtin_bit_cast(unsigned short, dp[(size_t)lane0 * s.H]);
            rq = rsb ? rsb[t0 + lane0] : (unsigned char)0;
        } else {  // ragged last tile: rows past the sequence read as zero (dt = 0 makes them no-ops)
#pragma unroll
            for (int u = 0; u < UBC; ++u) {
                const bool ok = bc_row0 + u * BRP < rows;
                bq[u] = ld16(bp + (size_t)u * BRP * s.G * N + bc_off0, ok);
                cq[u] = ld16(cp + (size_t)u * BRP * s.G * N + bc_off0, ok);
            }
#pragma unroll
            for (int u = 0; u < UX; ++u) xq[u] = ld16(xp + (size_t)u * XRP * HP + x_off0, x_row0 + u * XRP < rows);
            const bool ok = lane0 < rows;
            dq = ok ? __builtin_bit_cast(unsigned short, dp[(size_t)lane0 * s.H]) : (unsigned short)0;
            rq = (rsb && ok) ? rsb[t0 + lane0] : (unsigned char)0;
        }
    };

    // ---- this wave's half of the unit's running state: st[j][v] = H[p = lane % 32, n = 32 (2 role + j) + 8 (v/4) +
    // 4 (lane / 32) + v%4] ----
    f32x16 st[HNB];
    const bool fresh = rsb != nullptr && rsb[0] != 0;  // a restart before the first step: the initial state is not read
    prefetch(0);
    const size_t lane_off = (size_t)(pb * 32 + (lane0 & 31)) * N + 64 * role + 4 * (lane0 >> 5);
    {
        float4 iq[HNB][4];
#pragma unroll
        for (int j = 0; j < HNB; ++j) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) iq[j][gq] = make_float4(0, 0, 0, 0);
        }
        if (init != nullptr && !fresh) {  // (one uniform branch around all of the state's loads)
            const float *ib = init + ((size_t)b * s.H + h) * s.P * N + lane_off;
#pragma unroll
            for (int j = 0; j < HNB; ++j) {
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) iq[j][gq] = *reinterpret_cast<const float4 *>(ib + 32 * j + 8 * gq);
            }
        }
#pragma unroll
        for (int j = 0; j < HNB; ++j) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                st[j][4 * gq + 0] = iq[j][gq].x;
                st[j][4 * gq + 1] = iq[j][gq].y;
                st[j][4 * gq + 2] = iq[j][gq].z;
                st[j][4 * gq + 3] = iq[j][gq].w;
            }
        }
    }

    const int lane = lane0, r = lane & 31, half = lane >> 5;

    // Nothing in flight when the tile loop is entered: the wait for a tile's inputs at the loop's head is then counted
    // along the loop's own path, where they are older than the tile's stores of y (which the wave need not see
    // acknowledged), not along the prologue's, where they are the youngest requests.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    for (int c = 0; c < s.nc; ++c) {
        const int t0 = c * Q;
        const int rows = min(Q, s.L - t0);
        block_sync_lds();  // every wave is done reading the previous tile's tiles and operand fragments
        // ---- registers -> LDS tiles ----
        // where the staged pieces go: the swizzles repeat every 32 rows, and a pass is 32 rows.  Computed per tile from
        // a copy of the thread index that an empty asm hides from the compiler: hoisted out of the tile loop the
        // offsets would hold registers through both phases, which have none to spare.
        // A B or C row is 256 bytes, twice the width of the banks, and the 16 lanes served together hold one row's 16
        // pieces: writing the same 8-byte half of every piece at once would put 16 values on the even (or odd) 8-byte
        // slots of 256 bytes, which fold onto 128 bytes of banks two by two.  So the lanes of the row's upper eight pieces
        // write their halves in the other order (and odd rows the other way round, for the pair of rows that 32 lanes
        // cover): each instruction then fills 128 bytes of banks exactly.
        int bw[2], xw[2];
        bool swap;
        {
            int tw = tid;
            asm volatile("" : "+v"(tw));
            swap = ((((tw % BPR) >> 3) ^ (tw / BPR)) & 1) != 0;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                bw[hf] = BT::off(tw / BPR, (tw % BPR) * 8 + 4 * (swap ? 1 - hf : hf));
                xw[hf] = fused_scan_xtile_base(Q, (tw % XPR) / 4) + XT::off(tw / XPR, ((tw % XPR) % 4) * 8 + 4 * hf);
            }
        }
#pragma unroll
        for (int u = 0; u < UBC; ++u) {
            *reinterpret_cast<uint2 *>(Bs + bw[0] + u * BRP * N) = swap ? make_uint2(bq[u].z, bq[u].w) : make_uint2(bq[u].x, bq[u].y);
            *reinterpret_cast<uint2 *>(Bs + bw[1] + u * BRP * N) = swap ? make_uint2(bq[u].x, bq[u].y) : make_uint2(bq[u].z, bq[u].w);
            *reinterpret_cast<uint2 *>(Cs + bw[0] + u * BRP * N) = swap ? make_uint2(cq[u].z, cq[u].w) : make_uint2(cq[u].x, cq[u].y);
            *reinterpret_cast<uint2 *>(Cs + bw[1] + u * BRP * N) = swap ? make_uint2(cq[u].x, cq[u].y) : make_uint2(cq[u].z, cq[u].w);
        }
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            *reinterpret_cast<uint2 *>(xs_all + xw[0] + u * XRP * 32) = make_uint2(xq[u].x, xq[u].y);
            *reinterpret_cast<uint2 *>(xs_all + xw[1] + u * XRP * 32) = make_uint2(xq[u].z, xq[u].w);
        }
        // ---- scan of dt*A over the tile and the decay tables: the unit's first wave, for both (the second has one
        // more score block in phase 1, about as much work) ----
        if (role == 0) {
            constexpr double kLog2e = 1.4426950408889634;
            const float dtv = (float)__builtin_bit_cast(__bf16, dq);
            const double run = (double)dtv * a_h - (rq ? kResetDrop : 0.0);
            const double al = wave_inclusive_scan(run) * kLog2e;
            const float hi = (float)al, lo = (float)(al - (double)hi);
            float refh[QB], refl[QB], endh[QB], endl[QB];  // alpha at the first / last row of each block
#pragma unroll
            for (int lb = 0; lb < QB; ++lb) {
                refh[lb] = readlane_f(hi, 32 * lb);
                refl[lb] = readlane_f(lo, 32 * lb);
                endh[lb] = readlane_f(hi, 32 * lb + 31);
                endl[lb] = readlane_f(lo, 32 * lb + 31);
                if (lane == 0) {
                    blk_s[lb] = exp2_hw(refh[lb] + refl[lb]);
                    blk_s[8 + lb] = fmaxf(alpha_diff(refh[lb], refl[lb], endh[lb], endl[lb]), 0.f);
                }
            }
            if (lane == 0) blk_s[4] = exp2_hw(endh[QB - 1] + endl[QB - 1]);  // the tile's total decay
            const int l = lane, blk = l >> 5;
            ah_s[l] = hi;
            alo_s[l] = lo;
            dt_s[l] = dtv;
            w_s[l] = exp2_hw(fminf(alpha_diff(endh[QB - 1], endl[QB - 1], hi, lo), 0.f)) * dtv;
            const float rh = blk >= 1 ? refh[1] : refh[0], rl = blk >= 1 ? refl[1] : refl[0];
            E_s[l] = exp2_hw(fminf(alpha_diff(hi, lo, rh, rl), 0.f));
#pragma unroll
            for (int lb = 0; lb < QB; ++lb)
                if (lb >= blk) F_s[lb * Q + l] = exp2_hw(fminf(alpha_diff(refh[lb], refl[lb], hi, lo), 126.f)) * dtv;
        }
        block_sync_lds();  // tiles, operand fragments and tables are visible
        const float a_end = blk_s[4];  // exp2(alpha[Q-1])
        // ---- the tile's scores, once per workgroup: block g = sb + lb, (0,0), (0,1), (1,1), by the first waves of three
        // units (which have one score block to apply in phase 1 where the second waves have two) ----
        if (wave < 3) {
            // (the wave index hidden from the compiler: it would keep these sixteen addresses, which differ from the
            // ones every wave uses by a wave-uniform offset only, in registers of their own across the tile loop)
            int pw = wave;
            asm volatile("" : "+s"(pw));
            const int psb = pw == 2 ? 1 : 0, plb = pw == 0 ? 0 : 1;
            f32x16 sc = {0};
#pragma unroll
            for (int kk = 0; kk < NK; ++kk)
                sc = mma32(BT::split_frag(Bs + psb * 32 * N, r, 16 * kk + 4 * half), BT::split_frag(Cs + plb * 32 * N, r, 16 * kk + 4 * half), sc);
            float *gd = G_s + pw * 1024 + lane * 4;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<float4 *>(gd + q * 256) = make_float4(sc[4 * q], sc[4 * q + 1], sc[4 * q + 2], sc[4 * q + 3]);
        }
        __builtin_amdgcn_sched_barrier(0);
        // the next tile's inputs: requested here, in flight during both phases, stored to LDS at the top of the next tile
        if (c + 1 < s.nc) prefetch(c + 1);
        __builtin_amdgcn_sched_barrier(0);  // (left alone, the scheduler moves the loads down to where their values are used)

        // ---- phase 1: the outputs of this wave's block of 32 timesteps ----
        auto phase1 = [&](auto lbc) {
            constexpr int lb = decltype(lbc)::value;
            const int l = lb * 32 + r;
            // non-negative floats order like their bit patterns: a scalar compare
            const bool fast = __builtin_amdgcn_readfirstlane(__float_as_int(blk_s[8 + lb])) <= __float_as_int(kFastDiagSpan);
            // State readout, divided by the state dimension: this wave holds columns 64 role .. + 63 of the state and reads
            // out both output blocks over them -- its own block's sum stays in registers, the other block's goes to LDS
            // for the unit's other wave, which does the same for its half.  (A readout of the own block over the whole
            // state needs the other half in operand form: 16 KB written and 32 KB read per unit and tile, where the
            // partial sums are 4 KB each way.)
            f32x16 acc = {0}, oth = {0};
#pragma unroll
            for (int k4 = 0; k4 < NK / 2; ++k4) {
                const int col = 16 * (4 * role + k4) + 4 * half;
                const Frag<T> Cown = BT::split_frag(Cs, l, col), Coth = BT::split_frag(Cs, (1 - lb) * 32 + r, col);
                FragBits fh, fl;
                float sv[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) sv[i] = st[k4 / 2][8 * (k4 % 2) + i];
                split8_keep(sv, fh.u, fl.u);
                const Frag<T> Hh = fh.frag(), Hl = fl.frag();
                acc = mma32(Hh, Cown, acc);
                oth = mma32(Hh, Coth, oth);
                acc = mma32(Hl, Cown, acc);
                oth = mma32(Hl, Coth, oth);
            }
            {
                float *pd = part_unit + role * 1024 + lane * 4;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<float4 *>(pd + q * 256) = make_float4(oth[4 * q], oth[4 * q + 1], oth[4 * q + 2], oth[4 * q + 3]);
            }
            __builtin_amdgcn_sched_barrier(0);
            block_sync_lds();  // the unit's other partial sum, and the three blocks of scores, are in LDS
            {
                const float *ps = part_unit + (1 - role) * 1024 + lane * 4;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 t = *reinterpret_cast<const float4 *>(ps + q * 256);
                    acc[4 * q] += t.x;
                    acc[4 * q + 1] += t.y;
                    acc[4 * q + 2] += t.z;
                    acc[4 * q + 3] += t.w;
                }
            }
            acc = acc * blk_s[lb];
            __builtin_amdgcn_sched_barrier(0);
            const float *F_row = F_s + lb * Q;
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
            auto block = [&](auto sbc, auto diagc) {
                constexpr int sb = decltype(sbc)::value;
                constexpr bool diag = decltype(diagc)::value;
                f32x16 sc;
                {
                    const float *gs = G_s + (sb + lb) * 1024 + lane * 4;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4 t = *reinterpret_cast<const float4 *>(gs + q * 256);
                        sc[4 * q] = t.x;
                        sc[4 * q + 1] = t.y;
                        sc[4 * q + 2] = t.z;
                        sc[4 * q + 3] = t.w;
                    }
                }
                Frag<T> xf[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) xf[j] = XT::frag(xs, sb * 32 + 16 * j + 4 * half, 8, 0, lane);
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
                        acc = acc * El;
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
                for (int j = 0; j < 2; ++j) {
                    acc = mma32(xf[j], mh[j], acc);
                    acc = mma32(xf[j], ml[j], acc);
                }
                if (diag) acc = acc * Eend;  // everything summed so far shares the factor E[l]
                __builtin_amdgcn_sched_barrier(0);  // (one block's fragments at a time)
            };
            if constexpr (lb == 1) block(std::integral_constant<int, 0>{}, std::false_type{});
            block(std::integral_constant<int, lb>{}, std::true_type{});
            // epilogue: y[t, h, p] = yT[p, l] + D[h] * x[t, h, p]
            float o[16];
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const bf16x4 x4 = XT::row4(xs, l, 8 * vg + 4 * half);
#pragma unroll
                // (an explicit fused multiply-add, so that the bf16-y and the float-y instance round alike)
                for (int i = 0; i < 4; ++i) o[vg * 4 + i] = __builtin_fmaf(dh, (float)x4[i], acc[vg * 4 + i]);
            }
            const int yrow = t0 + l;
            store_column_buffer<TO>(ybuf, (unsigned)yrow * (unsigned)(HP * sizeof(TO)) + ycol_bytes, o, half, l < rows);
        };
        if (role == 0)
            phase1(std::integral_constant<int, 0>{});
        else
            phase1(std::integral_constant<int, 1>{});

        // ---- phase 2: this half of the state leaving the tile ----
        if (c + 1 == s.nc && final_states == nullptr) break;  // nobody reads the state the last tile leaves
#pragma unroll
        for (int j = 0; j < HNB; ++j) st[j] = st[j] * a_end;
        int xo[2][2], bo[2][2][HNB];
#pragma unroll
        for (int par = 0; par < 2; ++par) {
#pragma unroll
            for (int z = 0; z < 2; ++z) {
                xo[par][z] = XT::tr_off(16 * par + 8 * half + 4 * z, 0, lane);
#pragma unroll
                for (int j = 0; j < HNB; ++j) bo[par][z][j] = BT::tr_off(16 * par + 8 * half + 4 * z, (2 * role + j) * 32, lane);
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
            const Frag<T> xr = join(XT::tr_read(xs + xo[par][0] + rb * 32), XT::tr_read(xs + xo[par][1] + rb * 32));
            Frag<T> bf[HNB];
#pragma unroll
            for (int j = 0; j < HNB; ++j)
                bf[j] = join(BT::tr_read(Bs + bo[par][0][j] + rb * N), BT::tr_read(Bs + bo[par][1][j] + rb * N));
            const float4 wa = *reinterpret_cast<const float4 *>(w_s + k0);
            const float4 wb = *reinterpret_cast<const float4 *>(w_s + k0 + 4);
            const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
            FragBits xh, xl;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                split_pair((float)xr.v[2 * i], wv[2 * i], (float)xr.v[2 * i + 1], wv[2 * i + 1], xh.u[i], xl.u[i]);
            const Frag<T> xhf = xh.frag(), xlf = xl.frag();
#pragma unroll
            for (int j = 0; j < HNB; ++j) {
                st[j] = mma32(bf[j], xhf, st[j]);
                st[j] = mma32(bf[j], xlf, st[j]);
            }
        }
    }

    if (final_states != nullptr) {
        float *fb = final_states + ((size_t)b * s.H + h) * s.P * N + lane_off;
#pragma unroll
        for (int j = 0; j < HNB; ++j) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq)
                *reinterpret_cast<float4 *>(fb + 32 * j + 8 * gq) =
                    make_float4(st[j][4 * gq], st[j][4 * gq + 1], st[j][4 * gq + 2], st[j][4 * gq + 3]);
        }
    }
}

}  // namespace

// Whether the two-waves-per-unit kernel takes the shape: a 128-wide state, units in fours, forward in time, uncut.
bool fused_scan_wide_supported(const ScanShape &s) {
    return s.N == kWideN && s.P % 32 == 0 && ((s.H / s.G) * (s.P / 32)) % kWideUnits == 0 && s.mode == 0 && s.x_groups == 0 &&
           s.seg_tiles == 0 && s.seg_local == nullptr && (long long)s.L * s.H * s.P * 4 < (1LL << 31);
}

// s.Q and s.nc are the kernel's own tiling of time (kOnePassTile); dtype 1: bf16 y, 2: float y.
hipError_t launch_fused_scan_wide(const ScanShape &s, int dtype, const void *x, const void *dt, const float *A, const void *Bm,
                                  const void *Cm, const float *D, const float *init, const unsigned char *reset, void *y,
                                  float *final_states, hipStream_t st) {
    if (!fused_scan_wide_supported(s) || s.Q != kWideQ || s.nc != (s.L + kWideQ - 1) / kWideQ) return hipErrorInvalidValue;
    const int grid = s.B * s.G * (((s.H / s.G) * (s.P / 32)) / kWideUnits);
    const __bf16 *xx = static_cast<const __bf16 *>(x), *dd = static_cast<const __bf16 *>(dt);
    const __bf16 *bb = static_cast<const __bf16 *>(Bm), *cc = static_cast<const __bf16 *>(Cm);
    if (dtype == 2)
        fused_scan_wide_kernel<float><<<dim3(grid), dim3(64 * kWideWaves), 0, st>>>(xx, dd, A, bb, cc, D, init, reset,
                                                                                   static_cast<float *>(y), final_states, s);
    else
        fused_scan_wide_kernel<__bf16><<<dim3(grid), dim3(64 * kWideWaves), 0, st>>>(xx, dd, A, bb, cc, D, init, reset,
                                                                                    static_cast<__bf16 *>(y), final_states, s);
    return hipGetLastError();
}

}  // namespace ssd
