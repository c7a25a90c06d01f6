// Stage 2 of the SSD forward for gfx950: per-chunk states
//   S[b,c,h] = (w o x)^T [P x Q] . B [Q x N],   w[l] = exp2(alpha[Q-1] - alpha[l]) * dt[l]
// (w is row 3 of the stage-1 output).  One tile per (b,c,h); one wave per 32x32 block of S.
//
// The decay weight goes onto the x side (the smaller tile) in fp32; in bf16 mode the weighted
// x is kept as a hi + lo pair of bf16 (two MFMAs per K step) so that the result carries the
// inputs' precision rather than one extra bf16 rounding.  B enters exactly as given.
// Both operands have K = l as their slow axis in memory: bf16 tiles are stored row-major and
// transposed by the LDS transpose read; float tiles are transposed on their way into LDS.
//
// Persistent and software-pipelined: a workgroup holds the next tile's x, B and w in
// registers while the MFMAs of the current tile run.  Everything that shapes the inner code
// (head-dim blocks, state width, chunk length) is a template parameter, so the tile loop is
// straight-line code with 32-bit offsets from per-tile base pointers.
#include "ssd_device.h"

namespace ssd {

template <typename T, int PB, int NK, int QB>  // Ppad = 32*PB >= P, N = 16*NK, Q = 32*QB
__global__ __launch_bounds__(64 * PB * ((NK + 1) / 2)) void chunk_state_kernel(
    const T *__restrict__ x, const T *__restrict__ Bm, const float *__restrict__ dtcs,
    float *__restrict__ states, ScanShape s) {
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

    Vec16<T> xv[UX], bv[UB];
    float wv[UX];
    auto prefetch = [&](int logical) {
        const Tile t = decode_tile(logical, s);
        const float *wrow = dtcs + ((((size_t)t.b * s.H + t.h) * s.nc + t.c) * 4 + 3) * Q;
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

    TileSched sched(s.B * s.nc * s.H);
    if (sched.valid()) prefetch(sched.logical());
    // zero what no tile write covers (only when N is not a multiple of 32)
    if (N < Npad) {
        if (is_bf16<T>) {
            for (int idx = tid; idx < Q * Npad; idx += nthr) bs[idx] = (T)0.f;
        } else {
            for (int idx = tid; idx < (Npad - N) * ldq; idx += nthr) bs[N * ldq + idx] = (T)0.f;
        }
    }

    for (; sched.valid(); sched.advance()) {
        const Tile t = decode_tile(sched.logical(), s);
        __syncthreads();  // the previous tile's operand reads are done (and the zero fill is visible)
        // ---- registers -> LDS: weighted x (hi/lo in bf16 mode), B as is ----
#pragma unroll
        for (int u = 0; u < UX; ++u) {
            const int l = xl0 + u * xrpp;
            if (xrows_exact || l < Q) {
                if constexpr (is_bf16<T>) {
                    Vec16<T> hi, lo;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) Split<T>::split(wv[u] * (float)xv[u].e[i], hi.e[i], lo.e[i]);
                    const int o = XT::off(l, xch * VEC);
                    *reinterpret_cast<uint4 *>(xs + o) = hi.u;
                    *reinterpret_cast<uint4 *>(xs + Q * Ppad + o) = lo.u;
                } else {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) xs[(xch * VEC + i) * ldq + l] = wv[u] * xv[u].e[i];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int l = bl0 + u * brpp;
            if (brows_exact || l < Q) {
                if constexpr (is_bf16<T>) {
                    *reinterpret_cast<uint4 *>(bs + BT::off(l, bch * VEC)) = bv[u].u;
                } else {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) bs[(bch * VEC + i) * ldq + l] = bv[u].e[i];
                }
            }
        }
        if (sched.has_next()) prefetch(sched.next_logical());
        __syncthreads();

        f32x16 acc = {0};
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
        // S[p, n]: lane r holds column n, sixteen rows p
        const int n = nb * 32 + r;
        float *out = states + ((((size_t)t.b * s.nc + t.c) * s.H + t.h) * s.P) * N + (pb * 32 + 4 * half) * N + n;
        if (n < N) {
            if (s.P == Ppad) {
#pragma unroll
                for (int v = 0; v < 16; ++v) out[(8 * (v / 4) + (v % 4)) * N] = acc[v];
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (pb * 32 + 4 * half + 8 * (v / 4) + (v % 4) < s.P) out[(8 * (v / 4) + (v % 4)) * N] = acc[v];
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------
size_t chunk_state_lds_bytes(const ScanShape &s, int eb) {
    const size_t Ppad = (s.P + 31) & ~31, Npad = (s.N + 31) & ~31;
    if (eb == 2) return ((size_t)2 * s.Q * Ppad + (size_t)s.Q * Npad) * 2;
    return (Ppad + Npad) * (size_t)(s.Q + 4) * 4;
}

template <typename T, int PB, int NK, int QB>
static hipError_t state_launch(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                               float *states, hipStream_t st) {
    constexpr int block = 64 * PB * ((NK + 1) / 2);
    const size_t lds = chunk_state_lds_bytes(s, sizeof(T));
    hipError_t e = allow_lds(chunk_state_kernel<T, PB, NK, QB>, lds);
    if (e != hipSuccess) return e;
    int grid = 1;
    e = persistent_grid(chunk_state_kernel<T, PB, NK, QB>, block, lds, s.B * s.nc * s.H, &grid);
    if (e != hipSuccess) return e;
    chunk_state_kernel<T, PB, NK, QB><<<dim3(grid), dim3(block), lds, st>>>(
        static_cast<const T *>(x), static_cast<const T *>(Bm), dtcs, states, s);
    return hipGetLastError();
}

template <typename T, int PB, int NK>
static hipError_t state_dispatch_q(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                                   float *states, hipStream_t st) {
    switch (s.Q) {
        case 32: return state_launch<T, PB, NK, 1>(s, x, Bm, dtcs, states, st);
        case 64: return state_launch<T, PB, NK, 2>(s, x, Bm, dtcs, states, st);
        case 128: return state_launch<T, PB, NK, 4>(s, x, Bm, dtcs, states, st);
        case 256: return state_launch<T, PB, NK, 8>(s, x, Bm, dtcs, states, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T, int PB>
static hipError_t state_dispatch_n(const ScanShape &s, const void *x, const void *Bm, const float *dtcs,
                                   float *states, hipStream_t st) {
    switch (s.N) {
        case 16: return state_dispatch_q<T, PB, 1>(s, x, Bm, dtcs, states, st);
        case 32: return state_dispatch_q<T, PB, 2>(s, x, Bm, dtcs, states, st);
        case 64: return state_dispatch_q<T, PB, 4>(s, x, Bm, dtcs, states, st);
        case 128: return state_dispatch_q<T, PB, 8>(s, x, Bm, dtcs, states, st);
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

}  // namespace ssd
