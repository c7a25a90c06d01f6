// The backward pass's adjoint scan with the row products in its epilogue: dx written directly in bf16, and per
// (b, t, h) the pair (x . r, dy . x), instead of a float r that a row kernel reads back.
#include "ssd_fused_scan.h"

namespace ssd {

bool adjoint_rows_scan_supported(const ScanShape &s) {
    return s.P == 32 && (s.N == 32 || s.N == 64) && s.Q == kOnePassTile && (s.H / s.G) % 8 == 0;
}

hipError_t launch_adjoint_rows_scan(const ScanShape &sR, const void *dy, const void *dt, const float *A, const void *Cm,
                                    const void *Bm, const float *D, const void *x, const float *dfinal,
                                    const unsigned char *reset, void *dx, float *g0, float *pairs, hipStream_t st) {
    if (!adjoint_rows_scan_supported(sR)) return hipErrorInvalidValue;
    // the recurrence's roles: x <- dy, B <- C, C <- B
    return sR.N == 32 ? fused_launch_adjoint_rows<2>(sR, dy, dt, A, Cm, Bm, D, x, dfinal, reset, dx, g0, pairs, st)
                      : fused_launch_adjoint_rows<4>(sR, dy, dt, A, Cm, Bm, D, x, dfinal, reset, dx, g0, pairs, st);
}

}  // namespace ssd
