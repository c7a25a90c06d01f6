/*
 * CPU oracle (plain C) for the Mamba-2 SSD forward: the definitional sequential recurrence
 * and the single-timestep update.  TEST INFRASTRUCTURE ONLY -- the shipped library never
 * links or calls this file; it exists as the checker for the HIP kernels at sizes where a
 * Python time loop is too slow, and as the timed CPU baseline of the benchmark.
 *
 * The reference tree holds no SSD source to restate (only the benchmark row names at
 * benchmark_results/bench_20260112_070055.json:7,16,25,34 and the encoder slot at
 * trading_bots/src/torch/model/trading_model.rs:589-606), so this follows the published
 * Mamba-2 recurrence under the task's conventions:
 *
 *   h_t = exp(dt_t*A_h) h_{t-1} + dt_t * x_t (outer) B_t ;  y_t = h_t . C_t + D_h x_t
 *
 * Layouts (row-major, contiguous): x,y [B,L,H,P]; dt [B,L,H]; A,D [H]; Bm,Cm [B,L,G,N];
 * init,final [B,H,P,N].  D and init may be NULL.  Pinned against oracle/ssd_oracle.py
 * (itself pinned by closed forms) in tests/test_oracle.py.
 *
 * Two precisions are generated from one body: *_f64 (ground truth) and *_f32 (the CPU
 * baseline; same arithmetic type as the reference's CPU dtype policy,
 * trading_bots/src/torch/model/trading_model.rs:140-146).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DEFINE_SEQ(NAME, T, EXPF)                                                             \
    int NAME(int64_t Bsz, int64_t L, int64_t H, int64_t P, int64_t N, int64_t G, const T *x,  \
             const T *dt, const T *A, const T *Bm, const T *Cm, const T *D, const T *init,    \
             T *y, T *final_state, int nthreads)                                              \
    {                                                                                         \
        if (H % G != 0) return 1;                                                             \
        const int64_t hpg = H / G;                                                            \
        int failed = 0;                                                                       \
        (void)nthreads;                                                                       \
        _Pragma("omp parallel for collapse(2) schedule(static) num_threads(nthreads)")        \
        for (int64_t b = 0; b < Bsz; ++b) {                                                   \
            for (int64_t h = 0; h < H; ++h) {                                                 \
                T *st = (T *)malloc(sizeof(T) * (size_t)(P * N));                             \
                if (!st) { failed = 1; continue; }                                            \
                if (init) memcpy(st, init + ((b * H + h) * P) * N, sizeof(T) * (size_t)(P * N)); \
                else memset(st, 0, sizeof(T) * (size_t)(P * N));                              \
                const int64_t g = h / hpg;                                                    \
                const T a_h = A[h];                                                           \
                const T d_h = D ? D[h] : (T)0;                                                \
                for (int64_t t = 0; t < L; ++t) {                                             \
                    const T dtv = dt[(b * L + t) * H + h];                                    \
                    const T decay = EXPF(dtv * a_h);                                          \
                    const T *xr = x + ((b * L + t) * H + h) * P;                              \
                    const T *br = Bm + ((b * L + t) * G + g) * N;                             \
                    const T *cr = Cm + ((b * L + t) * G + g) * N;                             \
                    T *yr = y + ((b * L + t) * H + h) * P;                                    \
                    for (int64_t p = 0; p < P; ++p) {                                         \
                        const T dx = dtv * xr[p];                                             \
                        T *row = st + p * N;                                                  \
                        T acc = (T)0;                                                         \
                        for (int64_t n = 0; n < N; ++n) {                                     \
                            const T v = decay * row[n] + dx * br[n];                          \
                            row[n] = v;                                                       \
                            acc += v * cr[n];                                                 \
                        }                                                                     \
                        yr[p] = acc + d_h * xr[p];                                            \
                    }                                                                         \
                }                                                                             \
                if (final_state)                                                              \
                    memcpy(final_state + ((b * H + h) * P) * N, st, sizeof(T) * (size_t)(P * N)); \
                free(st);                                                                     \
            }                                                                                 \
        }                                                                                     \
        return failed;                                                                        \
    }

DEFINE_SEQ(ssd_oracle_seq_f64, double, exp)
DEFINE_SEQ(ssd_oracle_seq_f32, float, expf)

/* One recurrent update in place: state [B,H,P,N]; x,y [B,H,P]; dt [B,H]; Bm,Cm [B,G,N]. */
int ssd_oracle_step_f64(int64_t Bsz, int64_t H, int64_t P, int64_t N, int64_t G, double *state,
                        const double *x, const double *dt, const double *A, const double *Bm,
                        const double *Cm, const double *D, double *y)
{
    if (H % G != 0) return 1;
    const int64_t hpg = H / G;
    for (int64_t b = 0; b < Bsz; ++b)
        for (int64_t h = 0; h < H; ++h) {
            const int64_t g = h / hpg;
            const double dtv = dt[b * H + h];
            const double decay = exp(dtv * A[h]);
            const double *br = Bm + (b * G + g) * N;
            const double *cr = Cm + (b * G + g) * N;
            for (int64_t p = 0; p < P; ++p) {
                const double xv = x[(b * H + h) * P + p];
                double *row = state + ((b * H + h) * P + p) * N;
                double acc = 0.0;
                for (int64_t n = 0; n < N; ++n) {
                    row[n] = decay * row[n] + dtv * xv * br[n];
                    acc += row[n] * cr[n];
                }
                y[(b * H + h) * P + p] = acc + (D ? D[h] * xv : 0.0);
            }
        }
    return 0;
}
