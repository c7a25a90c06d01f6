// Stage 4 of the SSD forward for gfx950: chunk_scan.  One tile per (b,c,h); each wave owns 32 output columns
// l in [32*lb, 32*lb+32) and computes the TRANSPOSED output tile yT[p,l]:
//   yT  = exp2(alpha[l]) * (Hc [P x N] . C^T [N x l])                   state readout
//       + sum over s-blocks sb <= lb of  xT [P x s] . M^T [s x l]        intra-chunk
//   M^T[s,l] = (B[s,:] . C[l,:]) * exp2(alpha[l] - alpha[s]) * dt[s]  for s <= l, else 0
// Computing the transpose makes the 32x32 accumulator of B.C^T directly usable as the B
// operand of the second MFMA (its lane already holds column l and 16 rows s), so the masked
// score matrix never leaves registers; the A operand xT is read from LDS in the matching K
// order.  C fragments for the wave's 32 columns stay in registers for both products.
//
// Decay factors.  The factor separates through the first row m = 32*lb of the column block,
// exp2(alpha[l]-alpha[s]) dt[s] = E[l] F_lb[s],  E[l] = exp2(alpha[l]-alpha[m]),
// F_lb[s] = exp2(alpha[m]-alpha[s]) dt[s]: a score element costs one multiply by a per-row table
// value (the workgroup builds the table once per tile in LDS), and everything summed for a column
// is scaled by E[l] once at the end.  Below the diagonal both exponents are <= 0.  On the
// diagonal block (plus the causal mask) the table exponent is >= 0, which is safe as long as the
// block's total log2-decay stays below 120; a block that decays more takes the exact path, one
// exp2 of the hi/lo difference per element, after the sum so far has been scaled.  The choice is
// uniform per wave.
//
// In bf16 mode the two operands this kernel manufactures in fp32 -- M and the entering state
// Hc -- are fed to the MFMA as hi + lo bf16 pairs; x, B and C enter exactly as given.
// TO is the element type of y (T, or float for bf16 inputs with float32 output).
// The column-block index is rotated with the workgroup id so that the wave with the most
// s-blocks does not always sit on the same SIMD.
//
// Persistent and software-pipelined like stage 2: the next tile's B, x, entering state and
// alpha rows sit in registers while the current tile's MFMAs run.  Everything that shapes the
// inner code (head-dim blocks, state width, chunk length) is a template parameter.
// y leaves in 16-byte pieces: the two lanes that hold one output column swap halves of their
// values (v_permlane32_swap) so that each stores 8 consecutive head-dim elements.
#pragma once
#include "ssd_device.h"

namespace ssd {

template <typename T, typename TO, int PB, int NK, int QB>  // Ppad = 32*PB >= P, N = 16*NK, Q = 32*QB
__global__ __launch_bounds__(64 * QB, (is_bf16<T> && PB == 1 && NK <= 4 && QB >= 4) ? 3 : 2) void chunk_scan_kernel(
    const T *__restrict__ x, const T *__restrict__ Bm, const T *__restrict__ Cm, const float *__restrict__ dtcs,
    const float *__restrict__ prev, const float *__restrict__ D, TO *__restrict__ y, ScanShape s) {
    constexpr int VEC = Vec16<T>::N;
    constexpr int PARTS = Split<T>::PARTS;
    constexpr int N = NK * 16, Ppad = PB * 32, Q = QB * 32, nthr = 64 * QB, nblk = QB;
    constexpr int ldb = N + lds_pad<T>();
    constexpr int ldx = Q + lds_pad<T>();    // float mode: xs is transposed [Ppad][ldx]
    // Load mapping over the 2Q threads: a thread owns one 16-byte column slot of rows l0, l0+rpp, ...
    constexpr int bcpr = N / VEC, xcpr = Ppad / VEC;
    constexpr int brpp = nthr / bcpr, xrpp = nthr / xcpr;
    constexpr int UB = bcpr / 2, UX = xcpr / 2;   // passes = Q / rows per pass; both slot counts are even
    constexpr int hcpr = N / 4;
    constexpr int UHfull = (Ppad * hcpr + nthr - 1) / nthr;
    constexpr int UH = UHfull < 4 ? UHfull : 4;   // entering-state float4 loads per thread held across tiles
    using XT = RowMajorTile<Ppad>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *al_s = reinterpret_cast<float *>(smem);  // [3][Q]: alpha hi, alpha lo, dt
    float *tab = al_s + 3 * Q;                      // [nblk][Q]: F_k[s] = exp2(alpha[32k]-alpha[s])*dt[s], s < 32(k+1)
    T *Bs = reinterpret_cast<T *>(tab + nblk * Q);  // [Q][ldb]
    T *Hs = Bs + Q * ldb;                           // [PARTS][Ppad][ldb]
    T *xs = Hs + PARTS * Ppad * ldb;                // bf16: [Q][Ppad] row-major; float: [Ppad][ldx]
    const float *ah_s = al_s, *alo_s = al_s + Q, *dt_s = al_s + 2 * Q;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, and known to be
    const int r = lane & 31, half = lane >> 5;
    const int xl0 = tid / xcpr, xch = tid % xcpr, bl0 = tid / bcpr, bch = tid % bcpr;
    const bool xslot = xch * VEC < s.P;      // column slots past P stay zero
    const int xoff0 = xl0 * s.H * s.P + xch * VEC, xstep = xrpp * s.H * s.P;   // elements
    const int boff0 = bl0 * s.G * N + bch * VEC, bstep = brpp * s.G * N;
    const int htotal = s.P * hcpr;

    // ---- registers holding the next tile's inputs ----
    float a3[2];
    Vec16<T> bv[UB], xv[UX];
    float4 hv[UH];
    auto prefetch = [&](int logical) {
        const Tile t = decode_tile(logical, s);
        const float *arow = dtcs + ((((size_t)t.b * s.H + t.h) * s.nc + t.c) * 4) * Q;
        a3[0] = (tid < 3 * Q) ? arow[tid] : 0.f;
        a3[1] = (tid + nthr < 3 * Q) ? arow[tid + nthr] : 0.f;
        const int rows = min(Q, s.L - t.t0);  // valid rows of a ragged last chunk
        const T *bb = Bm + (((size_t)t.b * s.L + t.t0) * s.G + t.g) * N;
        const T *xb = x + (((size_t)t.b * s.L + t.t0) * s.H + t.h) * s.P;
        if (rows == Q) {
#pragma unroll
            for (int u = 0; u < UB; ++u) bv[u] = load_vec16(bb + boff0 + u * bstep);
#pragma unroll
            for (int u = 0; u < UX; ++u) xv[u] = xslot ? load_vec16(xb + xoff0 + u * xstep) : zero_vec16<T>();
        } else {
#pragma unroll
            for (int u = 0; u < UB; ++u)
                bv[u] = (bl0 + u * brpp < rows) ? load_vec16(bb + boff0 + u * bstep) : zero_vec16<T>();
#pragma unroll
            for (int u = 0; u < UX; ++u)
                xv[u] = (xslot && xl0 + u * xrpp < rows) ? load_vec16(xb + xoff0 + u * xstep) : zero_vec16<T>();
        }
        const float4 *hp = reinterpret_cast<const float4 *>(prev + ((((size_t)t.b * s.nc + t.c) * s.H + t.h) * s.P) * N);
#pragma unroll
        for (int u = 0; u < UH; ++u) {
            const int idx = u * nthr + tid;
            hv[u] = (idx < htotal) ? hp[idx] : make_float4(0, 0, 0, 0);
        }
    };
    auto put_state = [&](int idx, const float4 &h4) {
        const int p = idx / hcpr, n4 = idx % hcpr;
        const float v[4] = {h4.x, h4.y, h4.z, h4.w};
        if constexpr (is_bf16<T>) {
            __bf16 hi[4], lo[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) Split<T>::split(v[i], hi[i], lo[i]);
            bf16x4 h4v, l4v;
#pragma unroll
            for (int i = 0; i < 4; ++i) { h4v[i] = hi[i]; l4v[i] = lo[i]; }
            *reinterpret_cast<bf16x4 *>(Hs + p * ldb + n4 * 4) = h4v;
            *reinterpret_cast<bf16x4 *>(Hs + (Ppad + p) * ldb + n4 * 4) = l4v;
        } else {
            *reinterpret_cast<float4 *>(Hs + p * ldb + n4 * 4) = h4;
        }
    };

    TileSched sched(s.B * s.nc * s.H);
    if (sched.valid()) prefetch(sched.logical());
    // zero the state rows no tile write covers (only when P is not a multiple of 32)
    for (int idx = tid; idx < PARTS * (Ppad - s.P) * ldb; idx += nthr) {
        const int part = idx / ((Ppad - s.P) * ldb), rem = idx % ((Ppad - s.P) * ldb);
        Hs[(part * Ppad + s.P) * ldb + rem] = (T)0.f;
    }

    for (; sched.valid(); sched.advance()) {
        const int logical = sched.logical();
        const Tile t = decode_tile(logical, s);
        const int rows = min(Q, s.L - t.t0);
        const int lb = (wave + logical) % nblk;  // this wave's column block
        const int l = lb * 32 + r;
        // C fragments straight from global: column l of the tile, K = n
        Frag<T> Cf[NK];
        {
            const T *crow = Cm + (((size_t)t.b * s.L + t.t0 + l) * s.G + t.g) * N + half * 8;
            if (rows == Q) {
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) Cf[kk] = load_frag(crow + kk * 16);
            } else {
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) Cf[kk] = (l < rows) ? load_frag(crow + kk * 16) : zero_frag<T>();
            }
        }

        block_sync_lds();  // the previous tile's LDS reads are done (and the zero fill is visible)
        // ---- registers -> LDS ----
        if (tid < 3 * Q) al_s[tid] = a3[0];
        if (tid + nthr < 3 * Q) al_s[tid + nthr] = a3[1];
#pragma unroll
        for (int u = 0; u < UB; ++u)
            *reinterpret_cast<uint4 *>(Bs + (bl0 + u * brpp) * ldb + bch * VEC) = bv[u].u;
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            const int sr = xl0 + u * xrpp;
            if constexpr (is_bf16<T>) {
                *reinterpret_cast<uint4 *>(xs + XT::off(sr, xch * VEC)) = xv[u].u;
            } else {
#pragma unroll
                for (int i = 0; i < VEC; ++i) xs[(xch * VEC + i) * ldx + sr] = xv[u].e[i];
            }
        }
#pragma unroll
        for (int u = 0; u < UH; ++u) {
            const int idx = u * nthr + tid;
            if (idx < htotal) put_state(idx, hv[u]);
        }
        if constexpr (UHfull > UH) {  // the part of the entering state the register batch does not hold
            const float4 *hp = reinterpret_cast<const float4 *>(prev + ((((size_t)t.b * s.nc + t.c) * s.H + t.h) * s.P) * N);
            for (int idx = UH * nthr + tid; idx < htotal; idx += nthr) put_state(idx, hp[idx]);
        }
        block_sync_lds();  // alpha and dt are visible
        // decay table: row k holds F_k[s] for the rows at or below column block k
#pragma unroll
        for (int i = 0; i < (nblk * Q + nthr - 1) / nthr; ++i) {
            const int idx = i * nthr + tid;
            const int k = idx / Q, sr = idx % Q;
            if (idx < nblk * Q && sr < 32 * (k + 1)) {
                const float d = alpha_diff(ah_s[32 * k], alo_s[32 * k], ah_s[sr], alo_s[sr]);
                tab[idx] = exp2_hw(fminf(d, 126.f)) * dt_s[sr];
            }
        }
        if (sched.has_next()) prefetch(sched.next_logical());
        block_sync_lds();

        const float al_hi = ah_s[l], al_lo = alo_s[l];
        const float rf_hi = ah_s[32 * lb], rf_lo = alo_s[32 * lb];   // alpha at the column block's first row
        const float El = exp2_hw(fminf(alpha_diff(al_hi, al_lo, rf_hi, rf_lo), 0.f));
        // non-negative floats order like their bit patterns: a scalar compare
        const float span = fmaxf(alpha_diff(rf_hi, rf_lo, ah_s[32 * lb + 31], alo_s[32 * lb + 31]), 0.f);
        // The separable factors E[l] F[s] are exp2 of two arguments as large as the span, each rounded to float: their
        // product carries a relative error of about 2^-24 * span * ln 2, nothing next to bf16 operands (2^-17), but in
        // float mode a span of 64 would cost 30 ulps on the largest outputs.  Float mode therefore separates only
        // blocks that hardly decay; its MFMAs leave the VALU idle enough for the exact path's exp2 per element.
        constexpr float kSeparableSpan = is_bf16<T> ? 120.f : 4.f;
        const bool fast = __builtin_amdgcn_readfirstlane(__float_as_int(span)) <= __float_as_int(kSeparableSpan);
        f32x16 accY[PB];
        // state readout, brought to the column block's first row (alpha <= 0)
        {
            const float g0 = exp2_hw(rf_hi + rf_lo);
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                f32x16 a = {0};
                const T *hrow = Hs + (pb * 32 + r) * ldb + half * 8;
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) {
                    a = mma32(load_frag(hrow + kk * 16), Cf[kk], a);
                    if (PARTS == 2) a = mma32(load_frag(hrow + Ppad * ldb + kk * 16), Cf[kk], a);
                }
                accY[pb] = a * g0;
            }
        }
        // intra-chunk: s-blocks at or below this wave's column block (causal)
        const float *tab_row = tab + lb * Q;
        for (int sb = 0; sb <= lb; ++sb) {
            f32x16 sc = {0};
            const T *brow = Bs + (sb * 32 + r) * ldb + half * 8;
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) sc = mma32(load_frag(brow + kk * 16), Cf[kk], sc);
            const bool diag = sb == lb;
            float fv[16];
            if (!diag || fast) {
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const float4 t4 = *reinterpret_cast<const float4 *>(tab_row + sb * 32 + 8 * vg + 4 * half);
                    fv[4 * vg] = t4.x; fv[4 * vg + 1] = t4.y; fv[4 * vg + 2] = t4.z; fv[4 * vg + 3] = t4.w;
                }
            } else {
                // exact path: scale what has been summed, then full factors (exponents clamped at 0: entries
                // above the diagonal stay finite and are masked below)
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) accY[pb] = accY[pb] * El;
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int s0 = sb * 32 + 8 * vg + 4 * half;
                    const float4 ah4 = *reinterpret_cast<const float4 *>(ah_s + s0);
                    const float4 al4 = *reinterpret_cast<const float4 *>(alo_s + s0);
                    const float4 dt4 = *reinterpret_cast<const float4 *>(dt_s + s0);
                    fv[4 * vg] = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.x, al4.x), 0.f)) * dt4.x;
                    fv[4 * vg + 1] = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.y, al4.y), 0.f)) * dt4.y;
                    fv[4 * vg + 2] = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.z, al4.z), 0.f)) * dt4.z;
                    fv[4 * vg + 3] = exp2_hw(fminf(alpha_diff(al_hi, al_lo, ah4.w, al4.w), 0.f)) * dt4.w;
                }
            }
            Frag<T> mh[2], ml[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float sv[8], fj[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int v = 8 * j + i;
                    // causal mask inside the diagonal block: row 8 (v/4) + 4 half + v%4 <= column r
                    sv[i] = (!diag || 8 * (v / 4) + 4 * half + (v % 4) <= r) ? sc[v] : 0.f;
                    fj[i] = fv[v];
                }
                ProductFrags<T>::make(sv, fj, mh[j], ml[j]);
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
                        xf = load_frag_split(xs + (pb * 32 + r) * ldx + sb * 32 + 16 * j + 4 * half);
                    }
                    accY[pb] = mma32(xf, mh[j], accY[pb]);
                    if (PARTS == 2) accY[pb] = mma32(xf, ml[j], accY[pb]);
                }
            }
            if (diag && fast) {  // everything summed so far shares the factor E[l]
#pragma unroll
                for (int pb = 0; pb < PB; ++pb) accY[pb] = accY[pb] * El;
            }
        }
        // epilogue: y[t, h, p] = yT[p, l] + D[h] * x[t, h, p]
        {
            const float dh = D ? D[t.h] : 0.f;
            TO *yrow = y + (((size_t)t.b * s.L + t.t0 + l) * s.H + t.h) * s.P;
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                float o[16];
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int p0 = pb * 32 + 8 * vg + 4 * half;
                    float xl[4];
                    if constexpr (is_bf16<T>) {
                        const bf16x4 x4 = *reinterpret_cast<const bf16x4 *>(xs + XT::off(l, p0));
#pragma unroll
                        for (int i = 0; i < 4; ++i) xl[i] = (float)x4[i];
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) xl[i] = xs[(p0 + i) * ldx + l];
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[vg * 4 + i] = accY[pb][vg * 4 + i] + dh * xl[i];
                }
                store_column<TO>(yrow + pb * 32, o, half, s.P - pb * 32, l < rows);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Launchers (one translation unit per input/output type pair instantiates scan_dispatch)
// ------------------------------------------------------------------------------------------
template <typename T, typename TO, int PB, int NK, int QB>
static hipError_t scan_launch(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                              const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    const size_t lds = chunk_scan_lds_bytes(s, sizeof(T));
    hipError_t e = allow_lds(chunk_scan_kernel<T, TO, PB, NK, QB>, lds);
    if (e != hipSuccess) return e;
    int grid = 1;
    e = persistent_grid(chunk_scan_kernel<T, TO, PB, NK, QB>, 64 * QB, lds, s.B * s.nc * s.H, &grid);
    if (e != hipSuccess) return e;
    chunk_scan_kernel<T, TO, PB, NK, QB><<<dim3(grid), dim3(64 * QB), lds, st>>>(
        static_cast<const T *>(x), static_cast<const T *>(Bm), static_cast<const T *>(Cm), dtcs, prev, D,
        static_cast<TO *>(y), s);
    return hipGetLastError();
}

template <typename T, typename TO, int PB, int NK>
static hipError_t scan_dispatch_q(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                                  const float *dtcs, const float *prev, const float *D, void *y,
                                  hipStream_t st) {
    switch (s.Q) {
        case 32: return scan_launch<T, TO, PB, NK, 1>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 64: return scan_launch<T, TO, PB, NK, 2>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 128: return scan_launch<T, TO, PB, NK, 4>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 256: return scan_launch<T, TO, PB, NK, 8>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T, typename TO, int PB>
static hipError_t scan_dispatch_n(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                                  const float *dtcs, const float *prev, const float *D, void *y,
                                  hipStream_t st) {
    switch (s.N) {
        case 16: return scan_dispatch_q<T, TO, PB, 1>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 32: return scan_dispatch_q<T, TO, PB, 2>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 64: return scan_dispatch_q<T, TO, PB, 4>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 128: return scan_dispatch_q<T, TO, PB, 8>(s, x, Bm, Cm, dtcs, prev, D, y, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T, typename TO>
hipError_t scan_dispatch(const ScanShape &s, const void *x, const void *Bm, const void *Cm, const float *dtcs,
                         const float *prev, const float *D, void *y, hipStream_t st) {
    return (s.P <= 32) ? scan_dispatch_n<T, TO, 1>(s, x, Bm, Cm, dtcs, prev, D, y, st)
                       : scan_dispatch_n<T, TO, 2>(s, x, Bm, Cm, dtcs, prev, D, y, st);
}

}  // namespace ssd
