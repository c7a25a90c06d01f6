// Backward pass of the SSD scan: the memory-bound kernels around three role-swapped runs of the forward.
//
// With g_t = dLoss/dh_t, the adjoint recurrence g_t = dy_t (x) C_t + a_{t+1} g_{t+1} is the forward recurrence
// run backwards in time with (x, B, C) <- (dy, C, B), unit input weights and the decays shifted by one step.
// The three heavy products of the backward pass are readouts of such recurrences:
//   r_t  = g_t B_t                (x <- dy, B <- C, C <- B; reversed time)            dx  = D dy + dt r
//   yB_t = x_t . g_t              (transposed state: x <- C, B <- dy, C <- x; reversed) dB = sum_heads dt yB
//   yC_t = dy_t . h_t             (transposed state: x <- B, B <- x, C <- dy; forward)  dC = sum_heads yC
// and run on the forward's own stage kernels.  What is left is here: gathering the operands (time reversal,
// one copy of a group's B or C per head), the per-timestep products, the sums over the heads of a group, and
//   ddt_t = x_t . r_t + A q_t,   q_t = a_t <g_t, h_{t-1}>,   dA = sum dt q,   dD = sum dy . x,   dinit = a_0 g_0.
// q obeys q_t = u_t + q_{t+1} with u_t = C_t . yC_t - dt_t x_t . r_t (because a_t <g_t, h_{t-1}> =
// <g_t, h_t> - dt_t <g_t, x_t (x) B_t> and <g_t, h_t> = dy_t . (h_t C_t) + a_{t+1} <g_{t+1}, h_t>), but the u
// are each of the size of q and only their sum telescopes, so summing them over a whole sequence would add up
// their rounding errors (q is small against u where the decay is strong).  q is therefore anchored at the first
// step of every chunk, where it is the inner product of the two transposed scans' chunk states (forward state
// entering the chunk, adjoint state entering it), and at the end of the sequence (<dfinal, final>); the u are
// summed inside a chunk only, and the pass uses chunks of at most 64 steps.  For the two sets of chunk states to
// meet at the same timesteps the reversed sequences are padded in front with no-op steps to whole chunks.
#include "ssd_device.h"
#include "ssd_launch.h"

namespace ssd {

namespace {

template <typename T> struct Row8;  // eight consecutive elements as floats
template <> struct Row8<__bf16> {
    float v[8];
    static __device__ inline Row8 load(const __bf16 *p) {
        const bf16x8 q = *reinterpret_cast<const bf16x8 *>(p);
        Row8 r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r.v[i] = (float)q[i];
        return r;
    }
    __device__ inline void store(__bf16 *p) const {
        bf16x8 q;
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = (__bf16)v[i];
        *reinterpret_cast<bf16x8 *>(p) = q;
    }
};
template <> struct Row8<float> {
    float v[8];
    static __device__ inline Row8 load(const float *p) {
        const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
        Row8 r;
        r.v[0] = a.x; r.v[1] = a.y; r.v[2] = a.z; r.v[3] = a.w;
        r.v[4] = b.x; r.v[5] = b.y; r.v[6] = b.z; r.v[7] = b.w;
        return r;
    }
    __device__ inline void store(float *p) const {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
};

// dst[b, t', (g*rep + k)*W + w] = src[b, t, g*W + w] for k < rep, with t = Ldst-1-t' if reverse else t';
// zero where t >= Lsrc.  One thread per 8 elements of dst (W is a multiple of 8), moved as raw bits.
template <typename T>
__global__ __launch_bounds__(256) void gather_rows_kernel(const T *__restrict__ src, T *__restrict__ dst, int Lsrc,
                                                          int L, int groups, int W, int rep, int reverse,
                                                          long long total) {
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const int w8 = W / 8, per_row = groups * rep * w8;
    const int j = (int)(gid % per_row);
    const long long bt = gid / per_row;
    const int tp = (int)(bt % L);
    const long long b = bt / L;
    const int w = (j % w8) * 8, g = (j / w8) / rep;
    const int t = reverse ? L - 1 - tp : tp;
    typedef __attribute__((ext_vector_type(sizeof(T) * 2))) unsigned piece;  // 8 elements
    piece v = {};
    if (t < Lsrc) v = *reinterpret_cast<const piece *>(src + ((size_t)(b * Lsrc + t) * groups + g) * W + w);
    *reinterpret_cast<piece *>(dst + (size_t)bt * groups * rep * W + (size_t)j * 8) = v;
}

// [.., P, N] -> [.., N, P] for every (b,h): the state of the transposed recurrences
__global__ __launch_bounds__(256) void transpose_state_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                              int P, int N, long long total) {
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const int pn = P * N;
    const long long bh = gid / pn;
    const int i = (int)(gid % pn), n = i / P, p = i % P;  // dst index (n, p)
    dst[gid] = src[bh * pn + (size_t)p * N + n];
}

// Eight lanes per (b, t, h), one 8-element piece of a row each (headdim and dstate are at most 64):
// dx = D dy + dt r, e1 = x . r, dd = dy . x, u = C . yC - dt e1; the three dot products are summed over the
// eight lanes.  r_rev is the reversed scan's float output (row Lrev-1-t of Lrev rows holds timestep t; Lrev = 0:
// already in forward order), yC the forward-time transposed scan's.
// SUMS: the same pass also sums dt yB and yC over the heads of a group into dB and dC (a group's heads are
// adjacent rows, i.e. adjacent blocks of eight lanes of one wave: H/G must be 1, 2, 4 or 8), so that yC is read
// once; otherwise bwd_group_sums_kernel does that.
template <typename T, bool SUMS>
__global__ __launch_bounds__(256) void bwd_rows_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                       const T *__restrict__ dt, const T *__restrict__ Cm,
                                                       const float *__restrict__ D, const float *__restrict__ r_rev,
                                                       const float *__restrict__ yC, const float *__restrict__ yB_rev,
                                                       T *__restrict__ dx, float *__restrict__ e1, float *__restrict__ dd,
                                                       float *__restrict__ u, T *__restrict__ dB, T *__restrict__ dC,
                                                       ScanShape s, int Lrev, int LrevB, long long total) {
    const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long gid = tid >> 3;  // the row; whole groups of eight lanes leave together
    if (gid >= total) return;
    const int piece = (int)(tid & 7) * 8;
    const int h = (int)(gid % s.H);
    const long long bt = gid / s.H;
    const int t = (int)(bt % s.L);
    const long long b = bt / s.L;
    const int g = h / (s.H / s.G);
    const float dtv = (float)dt[gid], dh = D ? D[h] : 0.f;
    float se1 = 0.f, sdd = 0.f, sc = 0.f;
    if (piece < s.P) {
        const size_t row = (size_t)gid * s.P + piece;
        const size_t rrow = (Lrev ? ((size_t)(b * Lrev + (Lrev - 1 - t)) * s.H + h) * s.P : (size_t)gid * s.P) + piece;
        const Row8<T> xv = Row8<T>::load(x + row), dv = Row8<T>::load(dy + row);
        const Row8<float> rv = Row8<float>::load(r_rev + rrow);
        Row8<T> o;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            o.v[i] = dh * dv.v[i] + dtv * rv.v[i];
            se1 += xv.v[i] * rv.v[i];
            sdd += dv.v[i] * xv.v[i];
        }
        o.store(dx + row);
    }
    // the state columns, 64 per pass of the row's eight lanes (dstate 128: two passes)
    for (int n0 = 0; n0 < s.N; n0 += 64) {
        const int np = n0 + piece;
        Row8<float> sb, sy;  // this head's dt yB and yC pieces
#pragma unroll
        for (int i = 0; i < 8; ++i) sb.v[i] = sy.v[i] = 0.f;
        if (np < s.N) {
            const Row8<T> cv = Row8<T>::load(Cm + ((size_t)bt * s.G + g) * s.N + np);
            sy = Row8<float>::load(yC + (size_t)gid * s.N + np);
#pragma unroll
            for (int i = 0; i < 8; ++i) sc += cv.v[i] * sy.v[i];
            if (SUMS) {
                const size_t brow = LrevB ? (size_t)(b * LrevB + (LrevB - 1 - t)) : (size_t)bt;
                sb = Row8<float>::load(yB_rev + (brow * s.H + h) * s.N + np);
#pragma unroll
                for (int i = 0; i < 8; ++i) sb.v[i] *= dtv;
            }
        }
        if (SUMS) {
            const int hpg = s.H / s.G;
            for (int m = 8; m < 8 * hpg; m <<= 1) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    sb.v[i] += __shfl_xor(sb.v[i], m, 64);
                    sy.v[i] += __shfl_xor(sy.v[i], m, 64);
                }
            }
            if (h % hpg == 0 && np < s.N) {
                Row8<T> ob, oc;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    ob.v[i] = sb.v[i];
                    oc.v[i] = sy.v[i];
                }
                ob.store(dB + ((size_t)bt * s.G + g) * s.N + np);
                oc.store(dC + ((size_t)bt * s.G + g) * s.N + np);
            }
        }
    }
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) {
        se1 += __shfl_xor(se1, m, 8);
        sdd += __shfl_xor(sdd, m, 8);
        sc += __shfl_xor(sc, m, 8);
    }
    if (piece == 0) {
        e1[gid] = se1;
        dd[gid] = sdd;
        u[gid] = sc - dtv * se1;
    }
}

// The row products when the transposed scans summed dB and dC themselves: four lanes per (b, t, h) row (headdim 32),
// dx = D dy + dt r, e1 = x . r, dd = dy . x, u = (sum of the parts of C . yC) - dt e1.
template <typename T>
__global__ __launch_bounds__(256) void bwd_rows_parts_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                             const T *__restrict__ dt, const float *__restrict__ D,
                                                             const float *__restrict__ r_rev, const float *__restrict__ parts,
                                                             T *__restrict__ dx, float *__restrict__ e1, float *__restrict__ dd,
                                                             float *__restrict__ u, ScanShape s, int Lrev, int nparts,
                                                             long long total) {
    const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long gid = tid >> 3;
    if (gid >= total) return;
    const int piece = (int)(tid & 7) * 8;
    const int h = (int)(gid % s.H);
    const long long bt = gid / s.H;
    const int t = (int)(bt % s.L);
    const long long b = bt / s.L;
    const float dtv = (float)dt[gid], dh = D ? D[h] : 0.f;
    float se1 = 0.f, sdd = 0.f;
    if (piece < s.P) {
        const size_t row = (size_t)gid * s.P + piece;
        const size_t rrow = (Lrev ? ((size_t)(b * Lrev + (Lrev - 1 - t)) * s.H + h) * s.P : (size_t)gid * s.P) + piece;
        const Row8<T> xv = Row8<T>::load(x + row), dv = Row8<T>::load(dy + row);
        const Row8<float> rv = Row8<float>::load(r_rev + rrow);
        Row8<T> o;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            o.v[i] = dh * dv.v[i] + dtv * rv.v[i];
            se1 += xv.v[i] * rv.v[i];
            sdd += dv.v[i] * xv.v[i];
        }
        o.store(dx + row);
    }
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) {
        se1 += __shfl_xor(se1, m, 8);
        sdd += __shfl_xor(sdd, m, 8);
    }
    if (piece == 0) {
        float sc = 0.f;
        for (int k = 0; k < nparts; ++k) sc += parts[(size_t)gid * nparts + k];
        e1[gid] = se1;
        dd[gid] = sdd;
        u[gid] = sc - dtv * se1;
    }
}

// One thread per (b, t, g, 8 state columns): dB = sum over the group's heads of dt yB, dC = the same of yC.
template <typename T>
__global__ __launch_bounds__(256) void bwd_group_sums_kernel(const T *__restrict__ dt, const float *__restrict__ yB_rev,
                                                             const float *__restrict__ yC, T *__restrict__ dB,
                                                             T *__restrict__ dC, ScanShape s, int Lrev, long long total) {
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const int n8 = s.N / 8, hpg = s.H / s.G;
    const int n = (int)(gid % n8) * 8;
    const long long btg = gid / n8;
    const int g = (int)(btg % s.G);
    const long long bt = btg / s.G;
    const int t = (int)(bt % s.L);
    const long long b = bt / s.L;
    Row8<T> ob, oc;
#pragma unroll
    for (int i = 0; i < 8; ++i) ob.v[i] = oc.v[i] = 0.f;
    for (int k = 0; k < hpg; ++k) {
        const int h = g * hpg + k;
        const float dtv = (float)dt[(size_t)bt * s.H + h];
        const size_t brow = Lrev ? (size_t)(b * Lrev + (Lrev - 1 - t)) : (size_t)bt;
        const Row8<float> vb = Row8<float>::load(yB_rev + (brow * s.H + h) * s.N + n);
        const Row8<float> vc = Row8<float>::load(yC + ((size_t)bt * s.H + h) * s.N + n);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            ob.v[i] += dtv * vb.v[i];
            oc.v[i] += vc.v[i];
        }
    }
    ob.store(dB + (size_t)btg * s.N + n);
    oc.store(dC + (size_t)btg * s.N + n);
}

// One wave per (b, c, h), c = 0 .. nc: anchor[b,c,h] = q at the first step of chunk c = exp(dt A) <adjoint state
// entering chunk c, forward state entering chunk c>, dt the first step's of the chunk.  The reversed scan's chunk
// nc - c begins where forward chunk c does; for c = 0 that is past its last chunk, i.e. its final state, and the
// forward state is the initial one.  c = nc is the end of the sequence: q_L = <dfinal, final> (no decay).
template <typename T>
__global__ __launch_bounds__(256) void bwd_anchor_kernel(const T *__restrict__ dt, const float *__restrict__ A,
                                                         const float *__restrict__ fwd_prev, const float *__restrict__ rev_prev,
                                                         const float *__restrict__ rev_final, const float *__restrict__ init_t,
                                                         const float *__restrict__ fwd_final, const float *__restrict__ dfin_t,
                                                         const unsigned char *__restrict__ reset,
                                                         double *__restrict__ anchor, ScanShape s) {
    const int lane = threadIdx.x & 63;
    const long long id = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (id >= (long long)s.B * (s.nc + 1) * s.H) return;
    const int h = (int)(id % s.H);
    const int c = (int)((id / s.H) % (s.nc + 1));
    const long long b = id / ((long long)s.H * (s.nc + 1));
    const int pn = s.P * s.N;
    const size_t bh = ((size_t)b * s.H + h) * pn;
    const float *f, *g;
    if (c == 0) {
        f = init_t ? init_t + bh : nullptr;
        g = rev_final + bh;
    } else if (c == s.nc) {
        f = dfin_t ? fwd_final + bh : nullptr;
        g = dfin_t ? dfin_t + bh : nullptr;
    } else {
        f = fwd_prev + (((size_t)b * s.nc + c) * s.H + h) * pn;
        g = rev_prev + (((size_t)b * s.nc + (s.nc - c)) * s.H + h) * pn;
    }
    double part = 0.0;
    if (f != nullptr)
        for (int i = lane * 4; i < pn; i += 256) {
            const float4 fv = *reinterpret_cast<const float4 *>(f + i), gv = *reinterpret_cast<const float4 *>(g + i);
            part += (double)fv.x * gv.x + (double)fv.y * gv.y + (double)fv.z * gv.z + (double)fv.w * gv.w;
        }
    const double incl = wave_inclusive_scan(part);
    if (lane == 63) {
        double a = 1.0;
        if (c < s.nc) {  // a restart before the chunk's first step: the state entering it does not reach the loss
            const size_t t = (size_t)b * s.L + (size_t)c * s.Q;
            a = (reset != nullptr && reset[t] != 0) ? 0.0 : exp((double)(float)dt[t * s.H + h] * (double)A[h]);
        }
        anchor[id] = a * incl;
    }
}

// One wave per (b, c, h): a chunk of at most 64 steps.  q is known at both ends of a chunk (the anchors) and obeys
// q_t - q_{t+1} = u_t in between; the computed u do not sum exactly to the difference of the anchors, and the
// mismatch is spread evenly over the chunk's steps:
// q_t = anchor_c - sum_{v < t in the chunk} u_v - mismatch * (steps before t) / (steps of the chunk).
// ddt_t = e1_t + A q_t and this chunk's parts of dA = sum dt_t q_t and of dD = sum dd_t.  Sums in float64.
template <typename T>
__global__ __launch_bounds__(256) void bwd_ddt_kernel(const T *__restrict__ dt, const float *__restrict__ A,
                                                      const float *__restrict__ e1, const float *__restrict__ u,
                                                      const float *__restrict__ dd, const double *__restrict__ anchor,
                                                      T *__restrict__ ddt, double *__restrict__ dA_part,
                                                      double *__restrict__ dD_part, ScanShape s,
                                                      const float *__restrict__ parts, int nparts,
                                                      const unsigned char *__restrict__ reset, int raw_anchors) {
    const int lane = threadIdx.x & 63;
    const long long id = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (id >= (long long)s.B * s.nc * s.H) return;
    const int h = (int)(id % s.H);
    const int c = (int)((id / s.H) % s.nc);
    const long long b = id / ((long long)s.H * s.nc);
    auto last_lane = [](double v) {
        return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), 63),
                                __builtin_amdgcn_readlane(__double2loint(v), 63));
    };
    const double a = (double)A[h];
    // raw_anchors > 0: `anchor` holds that many pieces per (b, c, h) of the inner product of the two states at the
    // chunk's start, still without the first step's decay (zero where the sequence restarts there)
    auto anchor_at = [&](int k) {
        const size_t at = ((size_t)b * (s.nc + 1) + k) * s.H + h;
        if (raw_anchors == 0) return anchor[at];
        double v = 0.0;
        for (int i = 0; i < raw_anchors; ++i) v += anchor[at * raw_anchors + i];
        if (k < s.nc) {
            const size_t t = (size_t)b * s.L + (size_t)k * s.Q;
            v *= (reset != nullptr && reset[t] != 0) ? 0.0 : exp((double)(float)dt[t * s.H + h] * a);
        }
        return v;
    };
    const double q0 = anchor_at(c), q1 = anchor_at(c + 1);
    const int t0 = c * s.Q, len = min(s.Q, s.L - t0);
    const bool ok = lane < len;
    const size_t at = ((size_t)b * s.L + t0 + (ok ? lane : 0)) * s.H + h;
    float e1v = 0.f, ddv = 0.f, dtv = 0.f, uf = 0.f;
    if (ok) {
        dtv = (float)dt[at];
        if (parts != nullptr) {  // (e1, dd) pairs; u from the pieces of C . yC
            const float2 pr = *reinterpret_cast<const float2 *>(e1 + 2 * at);
            e1v = pr.x;
            ddv = pr.y;
            float sc = 0.f;
            for (int k = 0; k < nparts; ++k) sc += parts[at * nparts + k];
            uf = sc - dtv * e1v;
        } else {
            e1v = e1[at];
            ddv = dd[at];
            uf = u[at];
        }
    }
    const double uv = (double)uf;
    const double incl = wave_inclusive_scan(uv);
    const double mismatch = q0 - last_lane(incl) - q1;
    double da = 0.0;
    if (ok) {
        const double q = q0 - (incl - uv) - mismatch * (double)lane / (double)len;
        ddt[at] = (T)(float)((double)e1v + a * q);
        da = (double)dtv * q;
    }
    const double tot = last_lane(wave_inclusive_scan(da)), totd = last_lane(wave_inclusive_scan((double)ddv));
    if (lane == 0) {
        const size_t at_part = (size_t)h * ((size_t)s.B * s.nc) + (size_t)b * s.nc + c;  // [H, B*nc]: a head's parts together
        dA_part[at_part] = tot;
        dD_part[at_part] = totd;
    }
}

// The same for chunks of 64 steps and NH = 4, 8 or 16 heads with one wave per (b, c) and all its heads: lane =
// (step % TL) * NH + head with TL = 64 / NH, register r = step / TL, so that every load and store of the wave is one
// contiguous run of 64 elements of a [B, L, H] array (a wave per head touches a cache line per lane instead).
// NP: the pieces of C . yC per element when they are 1..4 (then e1 holds the (e1, dd) pairs and the loads are
// straight-line code); 0: any other form of the inputs, through conditions uniform over the launch.
// stride (a power of two, at most kDdtMaxStride): the anchors stand at every stride-th chunk boundary and at the end
// of the sequence only.  The chunks between two of them are a run; a run's waves sit in one workgroup (of
// max(4, stride) waves: whole runs), hand each other their chunks' sums of u through LDS, and spread the run's
// mismatch over all of its steps.
constexpr int kDdtMaxStride = 8;
template <typename T, int NH, int NP>
__global__ __launch_bounds__(64 * kDdtMaxStride) void bwd_ddt_heads_kernel(
    const T *__restrict__ dt, const float *__restrict__ A, const float *__restrict__ e1, const float *__restrict__ u,
    const float *__restrict__ dd, const double *__restrict__ anchor, T *__restrict__ ddt, double *__restrict__ dA_part,
    double *__restrict__ dD_part, ScanShape s, const float *__restrict__ parts, int nparts,
    const unsigned char *__restrict__ reset, int raw_anchors, int stride) {
    constexpr int TL = 64 / NH, R = 64 / TL;
    __shared__ double run_sums[kDdtMaxStride][NH];  // [wave of the workgroup][head]: the chunk's sum of u
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int runs = (s.nc + stride - 1) / stride;  // per sequence
    const long long run_id = (long long)blockIdx.x * ((blockDim.x >> 6) / stride) + wave / stride;
    const int cw = wave % stride;  // this wave's chunk of the run
    const int run = (int)(run_id % runs);
    // a wave past the last chunk (of its run, or of the launch) walks the last chunk of its sequence and keeps nothing:
    // every wave of a workgroup reaches the barrier below
    const long long b = min(run_id / runs, (long long)s.B - 1);
    const bool live = run_id < (long long)s.B * runs && run * stride + cw < s.nc;
    const int c = min(run * stride + cw, s.nc - 1);
    const long long id = b * s.nc + c;
    const int h = lane % NH, tl = lane / NH;
    const int t0 = c * 64, len = min(64, s.L - t0);
    const size_t row0 = ((size_t)b * s.L + t0) * NH;  // this chunk's first element of a [B, L, H] array
    // Every load of the wave is requested here, before the first is used, and none stands under a condition (a step
    // past the sequence reads the chunk's last step and counts as zero; a piece past nparts or raw_anchors reads the
    // last piece and counts as zero): under conditions and in loops of unknown length the compiler put a wait behind
    // every one of them.
    constexpr int kMaxPieces = 4;  // pieces per element read without a loop (more take the loops below)
    const size_t last = row0 + (size_t)len * NH - 1;
    T dt_q[R];
    float2 pr_q[R];
    float pk_q[R][kMaxPieces], u_q[R];
    const bool few_parts = NP > 0 || (parts != nullptr && nparts <= kMaxPieces);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const size_t at = min(row0 + (size_t)r * 64 + lane, last);
        dt_q[r] = dt[at];
        if constexpr (NP > 0) {
            pr_q[r] = *reinterpret_cast<const float2 *>(e1 + 2 * at);
#pragma unroll
            for (int k = 0; k < NP; ++k) pk_q[r][k] = parts[at * NP + k];
        } else if (parts != nullptr) {  // (uniform)
            pr_q[r] = *reinterpret_cast<const float2 *>(e1 + 2 * at);
            if (few_parts) {
#pragma unroll
                for (int k = 0; k < kMaxPieces; ++k) pk_q[r][k] = parts[at * nparts + min(k, nparts - 1)];
            }
        } else {
            pr_q[r] = make_float2(e1[at], dd[at]);
            u_q[r] = u[at];
        }
    }
    // the anchors: the inner product of the two states where chunk k starts.  raw_anchors > 0: `anchor` holds that
    // many pieces per (b, k, h), still without the first step's decay (zero where the sequence restarts there)
    const double a = (double)A[h];
    double an_q[2][kMaxPieces];
    T an_dt[2];
    unsigned char an_rs[2];
    const int ra = max(raw_anchors, 1);  // (the launcher keeps raw_anchors within kMaxPieces)
    const unsigned char *rs_or_any = reset != nullptr ? reset : reinterpret_cast<const unsigned char *>(dt);
    const int run_c[2] = {run * stride, min(run * stride + stride, s.nc)};  // the chunk boundaries the run lies between
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const size_t at = ((size_t)b * (s.nc + 1) + run_c[e]) * NH + h;
#pragma unroll
        for (int i = 0; i < kMaxPieces; ++i) an_q[e][i] = anchor[at * ra + min(i, ra - 1)];
        const size_t t = (size_t)b * s.L + (size_t)min(run_c[e], s.nc - 1) * 64;
        an_dt[e] = dt[t * NH + h];
        an_rs[e] = rs_or_any[t];
    }
    auto anchor_at = [&](int e) {
        double v = 0.0;
#pragma unroll
        for (int i = 0; i < kMaxPieces; ++i) v += i < ra ? an_q[e][i] : 0.0;
        const double first = (reset != nullptr && an_rs[e] != 0) ? 0.0 : exp((double)(float)an_dt[e] * a);
        return (raw_anchors != 0 && run_c[e] < s.nc) ? v * first : v;
    };
    const double q0 = anchor_at(0), q1 = anchor_at(1);
    float e1v[R], ddv[R], dtv[R];
    double uv[R], before[R];  // u_t and the sum of u over the chunk's earlier steps
    double carry = 0.0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = r * TL + tl;
        const bool in = t < len;
        dtv[r] = in ? (float)dt_q[r] : 0.f;
        e1v[r] = in ? pr_q[r].x : 0.f;
        ddv[r] = in ? pr_q[r].y : 0.f;
        float uf;
        if constexpr (NP > 0) {
            float sc = 0.f;
#pragma unroll
            for (int k = 0; k < NP; ++k) sc += pk_q[r][k];
            uf = sc - dtv[r] * e1v[r];
        } else if (parts != nullptr) {
            float sc = 0.f;
            if (few_parts) {
#pragma unroll
                for (int k = 0; k < kMaxPieces; ++k) sc += k < nparts ? pk_q[r][k] : 0.f;
            } else {
                const size_t at = min(row0 + (size_t)r * 64 + lane, last);
                for (int k = 0; k < nparts; ++k) sc += parts[at * nparts + k];
            }
            uf = sc - dtv[r] * e1v[r];
        } else {
            uf = u_q[r];
        }
        uv[r] = in ? (double)uf : 0.0;
        double v = uv[r];  // inclusive sum over this register's steps of the same head (lanes NH apart)
#pragma unroll
        for (int d = NH; d < 64; d <<= 1) {
            const double o = __shfl_up(v, d, 64);
            if (lane >= d) v += o;
        }
        before[r] = carry + v - uv[r];
        carry += __shfl(v, 64 - NH + h, 64);
    }
    // the run: the sum of u over its earlier chunks and over all of them, its steps before this chunk and in all
    double run_before = 0.0, run_total = carry;
    int steps_before = 0, run_len = len;
    if (stride > 1) {  // (uniform)
        if (tl == 0) run_sums[wave][h] = live ? carry : 0.0;
        __syncthreads();
        run_total = 0.0;
        for (int k = 0; k < stride; ++k) {
            const double v = run_sums[wave - cw + k][h];
            run_before += k < cw ? v : 0.0;
            run_total += v;
        }
        steps_before = cw * 64;
        run_len = min(stride * 64, s.L - run * stride * 64);
    }
    if (!live) return;
    const double mismatch = q0 - run_total - q1;
    double da = 0.0, sdd = 0.0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = r * TL + tl;
        if (t < len) {
            const double q = q0 - run_before - before[r] - mismatch * (double)(steps_before + t) / (double)run_len;
            ddt[row0 + (size_t)r * 64 + lane] = (T)(float)((double)e1v[r] + a * q);
            da += (double)dtv[r] * q;
            sdd += (double)ddv[r];
        }
    }
#pragma unroll
    for (int d = NH; d < 64; d <<= 1) {
        da += __shfl_xor(da, d, 64);
        sdd += __shfl_xor(sdd, d, 64);
    }
    if (tl == 0) {
        const size_t at_part = (size_t)h * ((size_t)s.B * s.nc) + id;  // [H, B*nc]: a head's parts together
        dA_part[at_part] = da;
        dD_part[at_part] = sdd;
    }
}

// One workgroup per head: dA[h] = the sum over (b, c) of dA_part[h,b,c], dD[h] likewise (float64 sums).
__global__ __launch_bounds__(256) void bwd_head_sums_kernel(const double *__restrict__ dA_part, const double *__restrict__ dD_part,
                                                            float *__restrict__ dA, float *__restrict__ dD, ScanShape s) {
    __shared__ double red[2][256];
    const int h = blockIdx.x;
    double sa = 0.0, sd = 0.0;
    const long long n = (long long)s.B * s.nc;
    const double *pa = dA_part + (size_t)h * (size_t)n, *pd = dD_part + (size_t)h * (size_t)n;
    // eight parts per round, requested together (an index past the end reads the last part and adds zero)
    for (long long i0 = threadIdx.x; i0 < n; i0 += 8LL * blockDim.x) {
        double qa[8], qd[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const long long i = min(i0 + (long long)u * blockDim.x, n - 1);
            qa[u] = pa[i];
            qd[u] = pd[i];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const bool in = i0 + (long long)u * blockDim.x < n;
            sa += in ? qa[u] : 0.0;
            sd += in ? qd[u] : 0.0;
        }
    }
    red[0][threadIdx.x] = sa;
    red[1][threadIdx.x] = sd;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) {
            red[0][threadIdx.x] += red[0][threadIdx.x + w];
            red[1][threadIdx.x] += red[1][threadIdx.x + w];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        dA[h] = (float)red[0][0];
        if (dD != nullptr) dD[h] = (float)red[1][0];
    }
}

// dinit = exp(dt_0 A) g_0, g_0 = the reversed scan's final state; zero for a row that restarts before step 0
template <typename T>
__global__ __launch_bounds__(256) void bwd_dinit_kernel(const T *__restrict__ dt, const float *__restrict__ A,
                                                        const float *__restrict__ gfin, const unsigned char *__restrict__ reset,
                                                        float *__restrict__ dinit, ScanShape s, long long total) {
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const long long bh = gid / (s.P * s.N);
    const int h = (int)(bh % s.H);
    const long long b = bh / s.H;
    const float a0 = (reset != nullptr && reset[(size_t)b * s.L] != 0) ? 0.f : __expf((float)dt[(size_t)b * s.L * s.H + h] * A[h]);
    dinit[gid] = a0 * gfin[gid];
}

inline unsigned blocks_for(long long total) { return (unsigned)((total + 255) / 256); }

template <typename T>
hipError_t gather_t(const void *src, void *dst, int B, int Lsrc, int L, int groups, int W, int rep, bool reverse,
                    hipStream_t st) {
    const long long total = (long long)B * L * groups * rep * (W / 8);
    gather_rows_kernel<T><<<dim3(blocks_for(total)), dim3(256), 0, st>>>(static_cast<const T *>(src), static_cast<T *>(dst), Lsrc,
                                                                         L, groups, W, rep, reverse ? 1 : 0, total);
    return hipGetLastError();
}

// out[row, h * rep + k] = in[row, h] for k < rep: dt (and A, as one row) given once per part of a head whose state
// dimension is scanned in `rep` parts
template <typename T>
__global__ __launch_bounds__(256) void replicate_columns_kernel(const T *__restrict__ in, T *__restrict__ out, int H, int rep,
                                                                long long total) {
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const long long row = gid / (H * rep);
    const int hk = (int)(gid % (H * rep));
    out[gid] = in[row * H + hk / rep];
}

template <typename T>
hipError_t rows_t(const ScanShape &s, int Lrev, const void *x, const void *dy, const void *dt, const void *Cm, const float *D,
                  const float *r_rev, const float *yC, void *dx, float *e1, float *dd, float *u, const float *yB_rev,
                  int LrevB, void *dB, void *dC, hipStream_t st) {
    const long long total = (long long)s.B * s.L * s.H;
    const T *xx = static_cast<const T *>(x), *yy = static_cast<const T *>(dy), *tt = static_cast<const T *>(dt);
    const T *cc = static_cast<const T *>(Cm);
    if (yB_rev != nullptr)
        bwd_rows_kernel<T, true><<<dim3(blocks_for(total * 8)), dim3(256), 0, st>>>(
            xx, yy, tt, cc, D, r_rev, yC, yB_rev, static_cast<T *>(dx), e1, dd, u, static_cast<T *>(dB), static_cast<T *>(dC), s,
            Lrev, LrevB, total);
    else
        bwd_rows_kernel<T, false><<<dim3(blocks_for(total * 8)), dim3(256), 0, st>>>(
            xx, yy, tt, cc, D, r_rev, yC, nullptr, static_cast<T *>(dx), e1, dd, u, nullptr, nullptr, s, Lrev, 0, total);
    return hipGetLastError();
}

template <typename T>
hipError_t group_sums_t(const ScanShape &s, int Lrev, const void *dt, const float *yB_rev, const float *yC, void *dB, void *dC,
                        hipStream_t st) {
    const long long total = (long long)s.B * s.L * s.G * (s.N / 8);
    bwd_group_sums_kernel<T><<<dim3(blocks_for(total)), dim3(256), 0, st>>>(static_cast<const T *>(dt), yB_rev, yC,
                                                                            static_cast<T *>(dB), static_cast<T *>(dC), s, Lrev, total);
    return hipGetLastError();
}

template <typename T>
hipError_t anchors_t(const ScanShape &s, const void *dt, const float *A, const float *fwd_prev, const float *rev_prev,
                     const float *rev_final, const float *init_t, const float *fwd_final, const float *dfin_t,
                     const unsigned char *reset, double *anchor, hipStream_t st) {
    const long long waves = (long long)s.B * (s.nc + 1) * s.H;
    bwd_anchor_kernel<T><<<dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, st>>>(
        static_cast<const T *>(dt), A, fwd_prev, rev_prev, rev_final, init_t, fwd_final, dfin_t, reset, anchor, s);
    return hipGetLastError();
}

template <typename T>
hipError_t ddt_t(const ScanShape &s, const void *dt, const float *A, const float *e1, const float *u, const float *dd,
                 const double *anchor, void *ddt, double *dA_part, double *dD_part, const float *parts, int nparts,
                 const unsigned char *reset, int raw_anchors, int anchor_stride, hipStream_t st) {
    if (s.Q > 64) return hipErrorInvalidValue;  // one pass of the wave per chunk
    if (anchor_stride < 1 || (anchor_stride & (anchor_stride - 1)) != 0 || anchor_stride > kDdtMaxStride ||
        (anchor_stride > 1 && !bwd_ddt_anchor_stride_supported(s, raw_anchors)))
        return hipErrorInvalidValue;
    if (bwd_ddt_anchor_stride_supported(s, raw_anchors)) {
        const int waves = max(4, anchor_stride);  // per workgroup: whole runs
        const long long runs = (long long)s.B * ((s.nc + anchor_stride - 1) / anchor_stride);
        const long long per_group = waves / anchor_stride;
        const dim3 grid((unsigned)((runs + per_group - 1) / per_group)), block(64 * waves);
#define SSD_DDT_HEADS_NP(NH, NP)                                                                                       \
    bwd_ddt_heads_kernel<T, NH, NP><<<grid, block, 0, st>>>(static_cast<const T *>(dt), A, e1, u, dd, anchor,           \
                                                            static_cast<T *>(ddt), dA_part, dD_part, s, parts, nparts,   \
                                                            reset, raw_anchors, anchor_stride)
#define SSD_DDT_HEADS(NH)                                           \
    do {                                                            \
        if (parts != nullptr && nparts == 1) SSD_DDT_HEADS_NP(NH, 1); \
        else if (parts != nullptr && nparts == 2) SSD_DDT_HEADS_NP(NH, 2); \
        else SSD_DDT_HEADS_NP(NH, 0);                               \
    } while (0)
        if (s.H == 4) SSD_DDT_HEADS(4);
        else if (s.H == 8) SSD_DDT_HEADS(8);
        else SSD_DDT_HEADS(16);
#undef SSD_DDT_HEADS
#undef SSD_DDT_HEADS_NP
        return hipGetLastError();
    }
    const long long waves = (long long)s.B * s.nc * s.H;
    bwd_ddt_kernel<T><<<dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, st>>>(static_cast<const T *>(dt), A, e1, u, dd, anchor,
                                                                              static_cast<T *>(ddt), dA_part, dD_part, s, parts,
                                                                              nparts, reset, raw_anchors);
    return hipGetLastError();
}

template <typename T>
hipError_t dinit_t(const ScanShape &s, const void *dt, const float *A, const float *gfin, const unsigned char *reset,
                   float *dinit, hipStream_t st) {
    const long long total = (long long)s.B * s.H * s.P * s.N;
    bwd_dinit_kernel<T><<<dim3(blocks_for(total)), dim3(256), 0, st>>>(static_cast<const T *>(dt), A, gfin, reset, dinit, s, total);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gather_rows(int dtype, const void *src, void *dst, int B, int Lsrc, int Ldst, int groups, int W,
                              int rep, bool reverse, hipStream_t st) {
    return dtype ? gather_t<__bf16>(src, dst, B, Lsrc, Ldst, groups, W, rep, reverse, st)
                 : gather_t<float>(src, dst, B, Lsrc, Ldst, groups, W, rep, reverse, st);
}

hipError_t launch_transpose_state(const float *src, float *dst, long long BH, int P, int N, hipStream_t st) {
    const long long total = BH * P * N;
    transpose_state_kernel<<<dim3(blocks_for(total)), dim3(256), 0, st>>>(src, dst, P, N, total);
    return hipGetLastError();
}

hipError_t launch_bwd_rows_parts(const ScanShape &s, int Lrev, int dtype, const void *x, const void *dy, const void *dt,
                                 const float *D, const float *r_rev, const float *parts, int nparts, void *dx,
                                 float *e1, float *dd, float *u, hipStream_t st) {
    const long long total = (long long)s.B * s.L * s.H;
    if (dtype)
        bwd_rows_parts_kernel<__bf16><<<dim3(blocks_for(total * 8)), dim3(256), 0, st>>>(
            static_cast<const __bf16 *>(x), static_cast<const __bf16 *>(dy), static_cast<const __bf16 *>(dt), D, r_rev, parts,
            static_cast<__bf16 *>(dx), e1, dd, u, s, Lrev, nparts, total);
    else
        bwd_rows_parts_kernel<float><<<dim3(blocks_for(total * 8)), dim3(256), 0, st>>>(
            static_cast<const float *>(x), static_cast<const float *>(dy), static_cast<const float *>(dt), D, r_rev, parts,
            static_cast<float *>(dx), e1, dd, u, s, Lrev, nparts, total);
    return hipGetLastError();
}

bool bwd_rows_can_sum(const ScanShape &s) {
    const int hpg = s.H / s.G;
    return hpg == 1 || hpg == 2 || hpg == 4 || hpg == 8;
}

hipError_t launch_bwd_rows(const ScanShape &s, int Lrev, int dtype, const void *x, const void *dy, const void *dt,
                           const void *Cm, const float *D, const float *r_rev, const float *yC, void *dx, float *e1,
                           float *dd, float *u, hipStream_t st, const float *yB_rev, int LrevB, void *dB, void *dC) {
    if (yB_rev != nullptr && !bwd_rows_can_sum(s)) return hipErrorInvalidValue;
    return dtype ? rows_t<__bf16>(s, Lrev, x, dy, dt, Cm, D, r_rev, yC, dx, e1, dd, u, yB_rev, LrevB, dB, dC, st)
                 : rows_t<float>(s, Lrev, x, dy, dt, Cm, D, r_rev, yC, dx, e1, dd, u, yB_rev, LrevB, dB, dC, st);
}

hipError_t launch_bwd_group_sums(const ScanShape &s, int Lrev, int dtype, const void *dt, const float *yB_rev,
                                 const float *yC, void *dB, void *dC, hipStream_t st) {
    return dtype ? group_sums_t<__bf16>(s, Lrev, dt, yB_rev, yC, dB, dC, st)
                 : group_sums_t<float>(s, Lrev, dt, yB_rev, yC, dB, dC, st);
}

hipError_t launch_bwd_anchors(const ScanShape &s, int dtype, const void *dt, const float *A, const float *fwd_prev,
                              const float *rev_prev, const float *rev_final, const float *init_t, const float *fwd_final,
                              const float *dfin_t, const unsigned char *reset, double *anchor, hipStream_t st) {
    return dtype ? anchors_t<__bf16>(s, dt, A, fwd_prev, rev_prev, rev_final, init_t, fwd_final, dfin_t, reset, anchor, st)
                 : anchors_t<float>(s, dt, A, fwd_prev, rev_prev, rev_final, init_t, fwd_final, dfin_t, reset, anchor, st);
}

bool bwd_ddt_anchor_stride_supported(const ScanShape &s, int raw_anchors) {  // (the kernel with a group's heads per wave)
    return s.Q == 64 && (s.H == 4 || s.H == 8 || s.H == 16) && raw_anchors <= 4;
}

hipError_t launch_bwd_ddt(const ScanShape &s, int dtype, const void *dt, const float *A, const float *e1, const float *u,
                          const float *dd, const double *anchor, void *ddt, double *dA_part, double *dD_part,
                          hipStream_t st, const float *parts, int nparts, const unsigned char *reset, int raw_anchors,
                          int anchor_stride) {
    return dtype ? ddt_t<__bf16>(s, dt, A, e1, u, dd, anchor, ddt, dA_part, dD_part, parts, nparts, reset, raw_anchors,
                                 anchor_stride, st)
                 : ddt_t<float>(s, dt, A, e1, u, dd, anchor, ddt, dA_part, dD_part, parts, nparts, reset, raw_anchors,
                                anchor_stride, st);
}

hipError_t launch_bwd_head_sums(const ScanShape &s, const double *dA_part, const double *dD_part, float *dA, float *dD,
                                hipStream_t st) {
    bwd_head_sums_kernel<<<dim3(s.H), dim3(256), 0, st>>>(dA_part, dD_part, dA, dD, s);
    return hipGetLastError();
}

hipError_t launch_bwd_dinit(const ScanShape &s, int dtype, const void *dt, const float *A, const float *gfin,
                            const unsigned char *reset, float *dinit, hipStream_t st) {
    return dtype ? dinit_t<__bf16>(s, dt, A, gfin, reset, dinit, st) : dinit_t<float>(s, dt, A, gfin, reset, dinit, st);
}

hipError_t launch_replicate_columns(int dtype, const void *in, void *out, long long rows, int H, int rep, hipStream_t st) {
    const long long total = rows * H * rep;
    if (dtype == 0)
        replicate_columns_kernel<float><<<dim3(blocks_for(total)), dim3(256), 0, st>>>(static_cast<const float *>(in),
                                                                                     static_cast<float *>(out), H, rep, total);
    else
        replicate_columns_kernel<__bf16><<<dim3(blocks_for(total)), dim3(256), 0, st>>>(static_cast<const __bf16 *>(in),
                                                                                      static_cast<__bf16 *>(out), H, rep, total);
    return hipGetLastError();
}

}  // namespace ssd
