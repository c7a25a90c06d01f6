// Stage 2 of the SSD forward for gfx950: per-chunk states
//   S[b,c,h] = (w o x)^T [P x Q] . B [Q x N],   w[l] = exp2(alpha[Q-1] - alpha[l]) * dt[l]
// (w is row 3 of the stage-1 output).  One tile per (b,c,h); one wave per 32x32 block of S.
//
// The same kernel, instantiated with SCAN = true, also does stage 3 in the same pass: a
// workgroup then walks whole (b,h) sequences chunk by chunk and keeps the running state in the
// MFMA accumulators, H_{c+1} = exp2(alpha_c[Q-1]) H_c + S_c (the accumulator is scaled by the
// chunk's total decay and the MFMAs add S_c on top).  It writes the state ENTERING each chunk
// straight into the chunk-state buffer and the final state at the end of the sequence, so the
// per-chunk states never make the round trip through HBM that a separate stage 3 needs.
//
// The decay weight goes onto the x side (the smaller tile) in fp32; in bf16 mode the weighted
// x is kept as a hi + lo pair of bf16 (two MFMAs per K step) so that the result carries the
// inputs' precision rather than one extra bf16 rounding.  B enters exactly as given.
// Both operands have K = l as their slow axis in memory: bf16 tiles are stored row-major and
// transposed by the LDS transpose read; float tiles are transposed on their way into LDS.
//
// Persistent and software-pipelined: a workgroup holds the next TWO tiles' x, B and w in
// registers (two register sets used alternately), so a tile's loads are issued two tile
// iterations before they are needed.  Everything that shapes the inner code
// (head-dim blocks, state width, chunk length) is a template parameter, so the tile loop is
// straight-line code with 32-bit offsets from per-tile base pointers.
#pragma once
#include "ssd_device.h"

namespace ssd {

template <typename T, int PB, int NK, int QB, bool SCAN>  // Ppad = 32*PB >= P, N = 16*NK, Q = 32*QB
__global__ __launch_bounds__(64 * PB * ((NK + 1) / 2)) void chunk_state_kernel(
    const T *__restrict__ x, const T *__restrict__ Bm, const float *__restrict__ dtcs,
    const float *init, float *__restrict__ states, float *final_states, ScanShape s) {
    constexpr int VEC = Vec16<T>::N;
    constexpr int PARTS = Split<T>::PARTS;
    constexpr int N = NK * 16, NB = (N + 31) / 32, Npad = NB * 32, Ppad = PB * 32, Q = QB * 32;
    constexpr int nthr = 64 * PB * NB;
    // Load mapping: a thread owns one 16-byte column slot of the tile rows l0, l0+rpp, ...
    constexpr int xcpr = Ppad / VEC, bcpr = N / VEC;
    constexpr int xrpp = nthr / xcpr, brpp = nthr / bcpr;
    constexpr int UX = (Q + xrpp - 1) / xrpp, UB = (Q + brpp - 1) / brpp;
    constexpr bool xrows_exact = (Q % xrpp) == 0, brows_exact = (Q % brpp) == 0;
    constexpr int ldq = Q + lds_pad<T>();  // float mode: transposed tiles [p or n][ldq]
    using XT = RowMajorTile<Ppad>;
    using BT = RowMajorTile<Npad>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T *xs = reinterpret_cast<T *>(smem);  // bf16: [PARTS][Q][Ppad] row-major; float: [Ppad][ldq]
    T *bs = xs + (is_bf16<T> ? PARTS * Q * Ppad : Ppad * ldq);  // bf16: [Q][Npad]; float: [Npad][ldq]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, and known to be
    const int r = lane & 31, half = lane >> 5;
    const int pb = wave / NB, nb = wave % NB;
    const int xl0 = tid / xcpr, xch = tid % xcpr, bl0 = tid / bcpr, bch = tid % bcpr;
    const bool xslot = xch * VEC < s.P;  // column slots past P stay zero
    const int xoff0 = xl0 * s.H * s.P + xch * VEC, xstep = xrpp * s.H * s.P;  // elements
    const int boff0 = bl0 * s.G * N + bch * VEC, bstep = brpp * s.G * N;

    struct TileRegs {
        Vec16<T> xv[UX], bv[UB];
        float wv[UX];
        float a_end;  // SCAN: alpha at the end of the chunk (its total log2-decay)
    };
    // two sets when they are small enough to stay in registers, else one
    constexpr int DEPTH = (UX * 5 + UB * 4 <= 64) ? 2 : 1;
    TileRegs regs[DEPTH];
    auto prefetch = [&](const Tile &t, TileRegs &R) {
        Vec16<T>(&xv)[UX] = R.xv;
        Vec16<T>(&bv)[UB] = R.bv;
        float(&wv)[UX] = R.wv;
        const float *wrow = dtcs + ((((size_t)t.b * s.H + t.h) * s.nc + t.c) * 4 + 3) * Q;
        if (SCAN) R.a_end = wrow[-2 * Q - 1];  // row 0 (alpha hi), element Q-1
        const T *xb = x + (((size_t)t.b * s.L + t.t0) * s.H + t.h) * s.P;
        const T *bb = Bm + (((size_t)t.b * s.L + t.t0) * s.G + t.g) * N;
        const int rows = min(Q, s.L - t.t0);  // valid rows of a ragged last chunk
        if (rows == Q) {
#pragma unroll
            for (int u = 0; u < UX; ++u) {
                const int l = xl0 + u * xrpp;
                const bool in = xslot && (xrows_exact || l < Q);
                xv[u] = in ? load_vec16(xb + xoff0 + u * xstep) : zero_vec16<T>();
                wv[u] = wrow[(xrows_exact || l < Q) ? l : 0];
            }
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const int l = bl0 + u * brpp;
                bv[u] = (brows_exact || l < Q) ? load_vec16(bb + boff0 + u * bstep) : zero_vec16<T>();
            }
        } else {
#pragma unroll
            for (int u = 0; u < UX; ++u) {
                const int l = xl0 + u * xrpp;
                xv[u] = (xslot && l < rows) ? load_vec16(xb + xoff0 + u * xstep) : zero_vec16<T>();
                wv[u] = wrow[l < Q ? l : 0];
            }
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const int l = bl0 + u * brpp;
                bv[u] = (l < rows) ? load_vec16(bb + boff0 + u * bstep) : zero_vec16<T>();
            }
        }
    };

    // This workgroup's tile list.  Plain mode: (b,c,h) tiles in schedule order.  SCAN mode: the
    // schedule runs over (b,h) sequences and every sequence contributes its nc chunks in order.
    TileSched sched(SCAN ? s.B * s.H : s.B * s.nc * s.H);
    const int nitems = sched.valid() ? (sched.per - sched.pos + sched.step - 1) / sched.step : 0;
    const int ntiles = SCAN ? nitems * s.nc : nitems;
    auto tile_at = [&](int k) {
        if (SCAN) {
            const int seq = sched.base + sched.pos + (k / s.nc) * sched.step;
            Tile t;
            t.b = seq / s.H;
            t.h = seq % s.H;
            t.c = k % s.nc;
            t.g = t.h / (s.H / s.G);
            t.t0 = t.c * Q;
            return t;
        }
        return decode_tile(sched.base + sched.pos + k * sched.step, s);
    };
    if (ntiles > 0) prefetch(tile_at(0), regs[0]);
    if (DEPTH == 2 && ntiles > 1) prefetch(tile_at(1), regs[DEPTH - 1]);
    // zero what no tile write covers (only when N is not a multiple of 32)
    if (N < Npad) {
        if (is_bf16<T>) {
            for (int idx = tid; idx < Q * Npad; idx += nthr) bs[idx] = (T)0.f;
        } else {
            for (int idx = tid; idx < (Npad - N) * ldq; idx += nthr) bs[N * ldq + idx] = (T)0.f;
        }
    }

    // One tile: its inputs are in R; when R has been copied to LDS it is refilled with the tile DEPTH
    // steps ahead.
    f32x16 acc = {0};  // SCAN: the running state block of this wave, carried from chunk to chunk
    auto do_tile = [&](int k, TileRegs &R) {
        const Tile t = tile_at(k);
        const float a_end = R.a_end;
        block_sync_lds();  // the previous tile's operand reads are done (and the zero fill is visible)
        // ---- registers -> LDS: weighted x (hi/lo in bf16 mode), B as is ----
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            const int l = xl0 + u * xrpp;
            if (xrows_exact || l < Q) {
                if constexpr (is_bf16<T>) {
                    Vec16<T> hi, lo;
                    unsigned hw[4], lw[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        split_pair((float)R.xv[u].e[2 * i], R.wv[u], (float)R.xv[u].e[2 * i + 1], R.wv[u], hw[i], lw[i]);
                    hi.u = make_uint4(hw[0], hw[1], hw[2], hw[3]);
                    lo.u = make_uint4(lw[0], lw[1], lw[2], lw[3]);
                    const int o = XT::off(l, xch * VEC);
                    *reinterpret_cast<uint4 *>(xs + o) = hi.u;
                    *reinterpret_cast<uint4 *>(xs + Q * Ppad + o) = lo.u;
                } else {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) xs[(xch * VEC + i) * ldq + l] = R.wv[u] * R.xv[u].e[i];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int l = bl0 + u * brpp;
            if (brows_exact || l < Q) {
                if constexpr (is_bf16<T>) {
                    *reinterpret_cast<uint4 *>(bs + BT::off(l, bch * VEC)) = R.bv[u].u;
                } else {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) bs[(bch * VEC + i) * ldq + l] = R.bv[u].e[i];
                }
            }
        }
        if (k + DEPTH < ntiles) prefetch(tile_at(k + DEPTH), R);
        block_sync_lds();

        // S[p, n] block of this wave: lane r holds column n, sixteen rows p
        const int n = nb * 32 + r;
        const size_t blk = (size_t)(pb * 32 + 4 * half) * N + n;
        const bool p_full = s.P == Ppad;
        auto for_rows = [&](auto &&fn) {  // fn(v, element offset) over the rows this lane holds
            if (n < N) {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (p_full || pb * 32 + 4 * half + 8 * (v / 4) + (v % 4) < s.P) fn(v, (8 * (v / 4) + (v % 4)) * N);
            }
        };
        float *out = states + ((((size_t)t.b * s.nc + t.c) * s.H + t.h) * s.P) * N + blk;
        if constexpr (SCAN) {
            if (t.c == 0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] = 0.f;
                if (init && !(s.fresh != nullptr && s.fresh[(size_t)t.b * s.L] != 0)) {  // (not after a restart at step 0)
                    const float *ib = init + ((size_t)t.b * s.H + t.h) * s.P * N + blk;
                    for_rows([&](int v, int o) { acc[v] = ib[o]; });
                }
            }
            // the state entering chunk 0 is the initial state; later chunks' entering states are
            // written at the end of the tile before (after the MFMAs, when the prefetch has landed)
            if (t.c == 0) for_rows([&](int v, int o) { out[o] = acc[v]; });
            acc = acc * exp2_hw(a_end);
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        }
        if constexpr (is_bf16<T>) {
#pragma unroll 2
            for (int ks = 0; ks < Q; ks += 16) {
                const int k0 = ks + 8 * half;
                const Frag<T> bf = BT::frag(bs, k0, 4, nb * 32, lane);
                acc = mma32(XT::frag(xs, k0, 4, pb * 32, lane), bf, acc);
                acc = mma32(XT::frag(xs + Q * Ppad, k0, 4, pb * 32, lane), bf, acc);
            }
        } else {
            const T *arow_p = xs + (pb * 32 + r) * ldq + half * 8;
            const T *brow_p = bs + (nb * 32 + r) * ldq + half * 8;
            for (int ks = 0; ks < Q; ks += 16) acc = mma32(load_frag(arow_p + ks), load_frag(brow_p + ks), acc);
        }
        if constexpr (SCAN) {
            if (t.c < s.nc - 1) {
                float *nx = out + (size_t)s.H * s.P * N;  // chunk c+1 of the same (b,h)
                for_rows([&](int v, int o) { nx[o] = acc[v]; });
            } else if (final_states) {
                float *fb = final_states + ((size_t)t.b * s.H + t.h) * s.P * N + blk;
                for_rows([&](int v, int o) { fb[o] = acc[v]; });
            }
        } else {
            for_rows([&](int v, int o) { out[o] = acc[v]; });
        }
    };
    for (int k = 0; k < ntiles; k += DEPTH) {
        do_tile(k, regs[0]);
        if (DEPTH == 2 && k + 1 < ntiles) do_tile(k + 1, regs[DEPTH - 1]);
    }
}

// ------------------------------------------------------------------------------------------
// Launchers (one translation unit per mode instantiates state_dispatch)
// ------------------------------------------------------------------------------------------
template <typename T, int PB, int NK, int QB, bool SCAN>
static hipError_t state_launch(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                               const float *init, float *states, float *final_states, hipStream_t st) {
    constexpr int block = 64 * PB * ((NK + 1) / 2);
    const size_t lds = chunk_state_lds_bytes(s, sizeof(T));
    hipError_t e = allow_lds(chunk_state_kernel<T, PB, NK, QB, SCAN>, lds);
    if (e != hipSuccess) return e;
    int grid = 1;
    e = persistent_grid(chunk_state_kernel<T, PB, NK, QB, SCAN>, block, lds, SCAN ? s.B * s.H : s.B * s.nc * s.H,
                        &grid);
    if (e != hipSuccess) return e;
    chunk_state_kernel<T, PB, NK, QB, SCAN><<<dim3(grid), dim3(block), lds, st>>>(
        static_cast<const T *>(x), static_cast<const T *>(Bm), dtcs, init, states, final_states, s);
    return hipGetLastError();
}

template <typename T, int PB, int NK, bool SCAN>
static hipError_t state_dispatch_q(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                                   const float *init, float *states, float *final_states, hipStream_t st) {
    switch (s.Q) {
        case 32: return state_launch<T, PB, NK, 1, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        case 64: return state_launch<T, PB, NK, 2, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        case 128: return state_launch<T, PB, NK, 4, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        case 256: return state_launch<T, PB, NK, 8, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T, int PB, bool SCAN>
static hipError_t state_dispatch_n(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                                   const float *init, float *states, float *final_states, hipStream_t st) {
    switch (s.N) {
        case 16: return state_dispatch_q<T, PB, 1, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        case 32: return state_dispatch_q<T, PB, 2, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        case 64: return state_dispatch_q<T, PB, 4, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        case 128: return state_dispatch_q<T, PB, 8, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
        default: return hipErrorInvalidValue;
    }
}

template <bool SCAN>
hipError_t state_dispatch(const ScanShape &s, int dtype, const void *x, const void *Bm, const float *dtcs,
                          const float *init, float *states, float *final_states, hipStream_t st) {
    if (dtype)
        return (s.P <= 32) ? state_dispatch_n<__bf16, 1, SCAN>(s, x, Bm, dtcs, init, states, final_states, st)
                           : state_dispatch_n<__bf16, 2, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
    return (s.P <= 32) ? state_dispatch_n<float, 1, SCAN>(s, x, Bm, dtcs, init, states, final_states, st)
                       : state_dispatch_n<float, 2, SCAN>(s, x, Bm, dtcs, init, states, final_states, st);
}

}  // namespace ssd
