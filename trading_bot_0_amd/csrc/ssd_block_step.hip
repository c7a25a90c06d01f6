// One timestep of the whole Mamba-2 block for a few streams, as ONE launch (gfx950):
//   in-projection (a matrix-vector product per stream) -> conv window update + SiLU, softplus(dt) -> SSM state
//   update and readout -> gate + RMSNorm -> out-projection.
// At a handful of streams the step's cost is the host's time to issue its launches (five kernels and two library
// products take about 0.1 ms of issue time for 0.01 ms of work); here a workgroup of 1 024 threads owns one stream
// and walks the five stages with workgroup barriers between them, every intermediate in LDS.  The two weight
// matrices come through L2 (0.33 MB and 0.13 MB in bf16 at 256 channels: every workgroup reads them whole), which is
// what bounds the launch -- so this entry point is for small batches; large ones keep the stage kernels, where the
// projections are matrix-matrix products.
//
// Rounding: every tensor the stage kernels would write to memory in the activation type (zxbcdt, x, B, C, dt, y, the
// normalised row) is rounded to that type here at the same point, so that a stream advanced by this kernel and one
// advanced by the stage kernels see the same numbers up to the order of the float32 sums.
#include "ssd_block_common.h"

namespace ssd {

namespace {

constexpr int kStepThreads = 1024;

template <typename T> __device__ inline float round_to(float v) { return (float)(T)v; }

// rows [0, rows) of w [rows, K] (K-contiguous) times vec (K floats in LDS) -> out (LDS floats), one row per group of
// K/8 lanes, eight rows of a group in flight at once
template <typename T, int K>
__device__ inline void gemv_rows(const T *__restrict__ w, int rows, const float *vec, float *out, int tid, bool round_out) {
    constexpr int G = K / 8;                       // lanes per row: 16 bytes (bf16) or 32 bytes (float) each
    constexpr int NG = kStepThreads / G;           // rows per pass of the workgroup
    constexpr int UN = 8;
    const int gl = tid % G, grp = tid / G;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = vec[gl * 8 + i];
    for (int r0 = grp; r0 < rows; r0 += NG * UN) {
        Pack8<T> q[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) q[u] = Pack8<T>::load(w + (size_t)min(r0 + u * NG, rows - 1) * K + gl * 8);
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            float a = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) a += q[u].get(i) * v[i];
#pragma unroll
            for (int m = G / 2; m >= 1; m >>= 1) a += __shfl_xor(a, m, 64);
            const int row = r0 + u * NG;
            if (gl == 0 && row < rows) out[row] = round_out ? round_to<T>(a) : a;
        }
    }
}

template <typename T, int DM, int DI, int DCONV>
__global__ __launch_bounds__(kStepThreads) void block_step_kernel(
    const T *__restrict__ u, const T *__restrict__ w_in, const float *__restrict__ conv_w, const float *__restrict__ conv_b,
    const float *__restrict__ dt_bias, const float *__restrict__ A, const float *__restrict__ D,
    const float *__restrict__ norm_w, float eps, const T *__restrict__ w_out, T *conv_state, float *ssm_state,
    T *__restrict__ out, BlockShape s) {
    const int tid = threadIdx.x, b = blockIdx.x;
    const int H = s.H, P = s.P, N = s.N, GN = s.G * s.N, C = DI + 2 * GN, E = 2 * DI + 2 * GN + H;
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float *u_s = sm;              // [DM]
    float *zx_s = u_s + DM;       // [E]    z | x | B | C | dt_raw, as the in-projection leaves them
    float *act_s = zx_s + E;      // [C]    x | B | C after conv + SiLU
    float *dt_s = act_s + C;      // [H]
    float *y_s = dt_s + ((H + 3) & ~3);  // [DI]   y, then the gated, normalised row
    float *red_s = y_s + DI;      // [kStepThreads / 64]

    for (int i = tid; i < DM; i += kStepThreads) u_s[i] = (float)u[(size_t)b * DM + i];
    __syncthreads();
    gemv_rows<T, DM>(w_in, E, u_s, zx_s, tid, true);
    __syncthreads();

    // conv window: the stream's last DCONV-1 inputs, then this step's; the state moves up by one row
    for (int c = tid; c < C; c += kStepThreads) {
        T *cs = conv_state + (size_t)b * (DCONV - 1) * C + c;
        float win[DCONV];
#pragma unroll
        for (int k = 0; k < DCONV - 1; ++k) win[k] = (float)cs[(size_t)k * C];
        win[DCONV - 1] = zx_s[DI + c];
        float a = conv_b[c];
#pragma unroll
        for (int k = 0; k < DCONV; ++k) a += conv_w[(size_t)c * DCONV + k] * win[k];
        act_s[c] = round_to<T>(silu(a));
#pragma unroll
        for (int k = 0; k < DCONV - 1; ++k) cs[(size_t)k * C] = (T)win[k + 1];
    }
    for (int h = tid; h < H; h += kStepThreads) dt_s[h] = round_to<T>(softplus(zx_s[DI + C + h] + dt_bias[h]));
    __syncthreads();

    // SSM step: four lanes per (head, row p), a quarter of the row's N columns each (float4 pieces, strided so that
    // the four lanes of a row read 64 consecutive bytes at a time)
    {
        const int HG = H / s.G, NQ = N / 4;  // float4 pieces per row
        for (int row = tid / 4; row < H * P; row += kStepThreads / 4) {
            const int h = row / P, q = tid & 3;
            const int g = h / HG;
            const float dtv = dt_s[h], xv = act_s[row];
            const float decay = __expf(dtv * A[h]), dx = dtv * xv;
            float4 *st = reinterpret_cast<float4 *>(ssm_state + ((size_t)b * H * P + row) * N);
            const float *Bv = act_s + DI + g * N, *Cv = act_s + DI + GN + g * N;
            float acc = 0.f;
            for (int j = q; j < NQ; j += 4) {
                float4 hv = st[j];
                const float4 bb = *reinterpret_cast<const float4 *>(Bv + 4 * j), cc = *reinterpret_cast<const float4 *>(Cv + 4 * j);
                hv.x = decay * hv.x + dx * bb.x;
                hv.y = decay * hv.y + dx * bb.y;
                hv.z = decay * hv.z + dx * bb.z;
                hv.w = decay * hv.w + dx * bb.w;
                acc += hv.x * cc.x + hv.y * cc.y + hv.z * cc.z + hv.w * cc.w;
                st[j] = hv;
            }
            acc += __shfl_xor(acc, 1, 64);
            acc += __shfl_xor(acc, 2, 64);
            if (q == 0) y_s[row] = round_to<T>(acc + (D != nullptr ? D[h] : 0.f) * xv);
        }
    }
    __syncthreads();

    // gate + RMSNorm over the DI channels
    {
        float ss = 0.f;
        for (int c = tid; c < DI; c += kStepThreads) {
            const float v = y_s[c] * silu(zx_s[c]);
            y_s[c] = v;
            ss += v * v;
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
        if ((tid & 63) == 0) red_s[tid >> 6] = ss;
        __syncthreads();
        float tot = 0.f;
        for (int i = 0; i < kStepThreads / 64; ++i) tot += red_s[i];
        const float scale = rsqrtf(tot / (float)DI + eps);
        for (int c = tid; c < DI; c += kStepThreads) y_s[c] = round_to<T>(y_s[c] * scale * norm_w[c]);
    }
    __syncthreads();
    gemv_rows<T, DI>(w_out, DM, y_s, zx_s, tid, false);
    __syncthreads();
    for (int i = tid; i < DM; i += kStepThreads) out[(size_t)b * DM + i] = (T)zx_s[i];
}

}  // namespace

bool block_step_supported(const BlockShape &s, int d_model) {
    const int DI = s.H * s.P;
    return s.L == 1 && (d_model == 128 || d_model == 256) && (DI == 128 || DI == 256) && s.N % 16 == 0 && s.P % 4 == 0 &&
           s.d_conv >= 2 && s.d_conv <= 4 && s.H % s.G == 0;
}

template <typename T, int DM, int DI>
static hipError_t step_dispatch(const BlockShape &s, const void *u, const void *w_in, const float *conv_w, const float *conv_b,
                                const float *dt_bias, const float *A, const float *D, const float *norm_w, float eps,
                                const void *w_out, void *conv_state, float *ssm_state, void *out, hipStream_t st) {
    const int GN = s.G * s.N, C = DI + 2 * GN, E = 2 * DI + 2 * GN + s.H;
    const size_t lds = sizeof(float) * ((size_t)DM + E + C + ((s.H + 3) & ~3) + DI + kStepThreads / 64);
    if (lds > 64 * 1024) return hipErrorInvalidValue;
    const T *uu = static_cast<const T *>(u), *wi = static_cast<const T *>(w_in), *wo = static_cast<const T *>(w_out);
    T *cs = static_cast<T *>(conv_state), *oo = static_cast<T *>(out);
    const dim3 grid(s.B), block(kStepThreads);
    switch (s.d_conv) {
        case 2: block_step_kernel<T, DM, DI, 2><<<grid, block, lds, st>>>(uu, wi, conv_w, conv_b, dt_bias, A, D, norm_w, eps, wo, cs, ssm_state, oo, s); break;
        case 3: block_step_kernel<T, DM, DI, 3><<<grid, block, lds, st>>>(uu, wi, conv_w, conv_b, dt_bias, A, D, norm_w, eps, wo, cs, ssm_state, oo, s); break;
        case 4: block_step_kernel<T, DM, DI, 4><<<grid, block, lds, st>>>(uu, wi, conv_w, conv_b, dt_bias, A, D, norm_w, eps, wo, cs, ssm_state, oo, s); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// u [B, d_model], w_in [E, d_model], w_out [d_model, H*P] in the activation type (dtype 0 float32, else bf16);
// conv_state [B, d_conv-1, C] (activation type) and ssm_state [B, H, P, N] (float32) advance in place; out [B, d_model].
hipError_t launch_block_step(const BlockShape &s, int dtype, int d_model, const void *u, const void *w_in, const float *conv_w,
                             const float *conv_b, const float *dt_bias, const float *A, const float *D, const float *norm_w,
                             float eps, const void *w_out, void *conv_state, float *ssm_state, void *out, hipStream_t st) {
    if (!block_step_supported(s, d_model)) return hipErrorInvalidValue;
    const int DI = s.H * s.P;
#define SSD_STEP_CASE(Tv, DMv, DIv)                                                                                     \
    if (d_model == DMv && DI == DIv)                                                                                    \
        return step_dispatch<Tv, DMv, DIv>(s, u, w_in, conv_w, conv_b, dt_bias, A, D, norm_w, eps, w_out, conv_state,   \
                                           ssm_state, out, st);
    if (dtype == 0) {
        SSD_STEP_CASE(float, 128, 128) SSD_STEP_CASE(float, 128, 256) SSD_STEP_CASE(float, 256, 128) SSD_STEP_CASE(float, 256, 256)
    } else {
        SSD_STEP_CASE(__bf16, 128, 128) SSD_STEP_CASE(__bf16, 128, 256) SSD_STEP_CASE(__bf16, 256, 128) SSD_STEP_CASE(__bf16, 256, 256)
    }
#undef SSD_STEP_CASE
    return hipErrorInvalidValue;
}

}  // namespace ssd
