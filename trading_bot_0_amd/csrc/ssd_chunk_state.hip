// Stage 2 (chunk_state) instantiations: per-chunk states, one tile per (b,c,h).
#include "ssd_chunk_state.h"

namespace ssd {

size_t chunk_state_lds_bytes(const ScanShape &s, int eb) {
    const size_t Ppad = (s.P + 31) & ~31, Npad = (s.N + 31) & ~31;
    if (eb == 2) return ((size_t)2 * s.Q * Ppad + (size_t)s.Q * Npad) * 2;
    return (Ppad + Npad) * (size_t)(s.Q + 4) * 4;
}

hipError_t launch_chunk_state(const ScanShape &s, int dtype, const void *x, const void *Bm, const float *dtcs,
                              float *states, hipStream_t st) {
    return state_dispatch<false>(s, dtype, x, Bm, dtcs, nullptr, states, nullptr, st);
}

}  // namespace ssd
