// Stages 2+3 in one pass (chunk_state with the running state carried in the accumulators).
#include "ssd_chunk_state.h"

namespace ssd {

hipError_t launch_chunk_state_scan(const ScanShape &s, int dtype, const void *x, const void *Bm, const float *dtcs,
                                   const float *init, float *prev, float *final_states, hipStream_t st) {
    return state_dispatch<true>(s, dtype, x, Bm, dtcs, init, prev, final_states, st);
}

}  // namespace ssd
