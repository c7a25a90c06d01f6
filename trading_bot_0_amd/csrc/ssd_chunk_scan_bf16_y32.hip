// Stage 4 (chunk_scan) instantiations for __bf16 inputs and float output.
#include "ssd_chunk_scan.h"

namespace ssd {

hipError_t launch_chunk_scan_bf16_y32(const ScanShape &s, const void *x, const void *Bm, const void *Cm,
                                  const float *dtcs, const float *prev, const float *D, void *y, hipStream_t st) {
    return scan_dispatch<__bf16, float>(s, x, Bm, Cm, dtcs, prev, D, y, st);
}

}  // namespace ssd
