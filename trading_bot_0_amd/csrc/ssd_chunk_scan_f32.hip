// Stage 4 (chunk_scan) instantiations for float inputs and float output.
#include "ssd_chunk_scan.h"

namespace ssd {

hipError_t launch_chunk_scan_f32(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                                  const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    return scan_dispatch<float, float>(s, x, Bm, Cm, dtcs, prev, D, y, st);
}

}  // namespace ssd
