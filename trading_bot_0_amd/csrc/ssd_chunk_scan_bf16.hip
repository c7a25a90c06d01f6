// Stage 4 (chunk_scan) instantiations for __bf16 inputs and __bf16 output.
#include "ssd_chunk_scan.h"

namespace ssd {

hipError_t launch_chunk_scan_bf16(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                                  const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    return scan_dispatch<__bf16, __bf16>(s, x, Bm, Cm, dtcs, prev, D, y, st);
}

size_t chunk_scan_lds_bytes(const ScanShape &s, int eb) {
    const size_t Ppad = (s.P + 31) & ~31;
    const size_t ldb = s.N + 16 / eb, parts = eb == 2 ? 2 : 1;
    const size_t xs = eb == 2 ? (size_t)s.Q * Ppad : Ppad * (size_t)(s.Q + 4);
    return (size_t)s.Q * 12 + (size_t)(s.Q / 32) * s.Q * 4 + ((size_t)s.Q * ldb + parts * Ppad * ldb + xs) * eb;
}

hipError_t launch_chunk_scan_f32(const ScanShape &, const void *, const void *, const void *, const float *,
                                 const float *, const float *, void *, hipStream_t);
hipError_t launch_chunk_scan_bf16_y32(const ScanShape &, const void *, const void *, const void *, const float *,
                                      const float *, const float *, void *, hipStream_t);

hipError_t launch_chunk_scan(const ScanShape &s, int dtype, const void *x, const void *Bm, const void *Cm,
                             const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    switch (dtype) {
        case 0: return launch_chunk_scan_f32(s, x, Bm, Cm, dtcs, prev, D, y, st);
        case 1: return launch_chunk_scan_bf16(s, x, Bm, Cm, dtcs, prev, D, y, st);
        default: return launch_chunk_scan_bf16_y32(s, x, Bm, Cm, dtcs, prev, D, y, st);
    }
}

}  // namespace ssd
