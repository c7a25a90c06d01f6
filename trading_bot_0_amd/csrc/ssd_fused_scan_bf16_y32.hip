// One-pass forward, bf16 inputs and float32 y.
#include "ssd_fused_scan.h"

namespace ssd {

hipError_t launch_fused_scan_y32(const ScanShape &s, int waves, const void *x, const void *dt, const float *A,
                                 const void *Bm, const void *Cm, const float *D, const float *init,
                                 const unsigned char *reset, void *y, float *final_states, float *tile_states,
                                 hipStream_t st) {
    return fused_dispatch<float>(s, waves, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
}

}  // namespace ssd
