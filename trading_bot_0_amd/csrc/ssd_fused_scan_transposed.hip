// The backward pass's two scans of the transposed state on the one-pass kernel's transposed kinds: eight heads
// per workgroup, the sum over a group's heads taken in LDS, bf16 gradients written directly.
#include "ssd_fused_scan.h"

namespace ssd {

bool transposed_scan_supported(const ScanShape &sT, int x_groups) {
    return sT.N == 32 && sT.G == sT.H && x_groups > 0 && sT.H == 8 * x_groups && sT.P % 32 == 0 && sT.P <= 64 &&
           sT.Q == kOnePassTile;
}

namespace {
// a 64-wide state with both slices in one wave where that still leaves enough workgroups for the chip
bool wide(const ScanShape &sT) {
    constexpr int kWideMinWorkgroups = 96;
    return sT.P == 64 && (long long)sT.B * (sT.H / 8) >= kWideMinWorkgroups;
}
}  // namespace

// The wide kinds take the anchors in the adjoint scan (the forward one already carries the parts of C . y and has
// no registers left for them), the narrow ones in the forward scan.
bool transposed_scan_anchors_in_adjoint(const ScanShape &sT) { return wide(sT); }

hipError_t launch_transposed_scan(const ScanShape &sT, bool adjoint, const void *x, const void *dt, const float *A,
                                  const void *Bm, const void *Cm, const void *aux, const float *init,
                                  const unsigned char *reset, void *out, float *final_states, float *tile_states,
                                  float *parts, const ScanAnchors &an, hipStream_t st) {
    ScanShape t = sT;
    t.Q = kOnePassTile;
    t.nc = (sT.L + kOnePassTile - 1) / kOnePassTile;
    if (an.out != nullptr && adjoint != wide(sT)) return hipErrorInvalidValue;
    if (an.out != nullptr && an.other_tiles == nullptr) return hipErrorInvalidValue;  // (the kernel reads it without asking)
    if (an.stride < 1 || an.phase < 0 || an.phase >= an.stride) return hipErrorInvalidValue;
    ScanAnchors keep;  // the scan that runs first: which of its tile states it keeps
    keep.stride = an.stride;
    keep.phase = an.phase;
    if (wide(sT))
        return adjoint ? fused_launch_transposed<__bf16, 7>(t, x, dt, A, Bm, Cm, nullptr, init, reset, out, final_states,
                                                            tile_states, nullptr, an, st)
                       : fused_launch_transposed<__bf16, 6>(t, x, dt, A, Bm, Cm, aux, init, reset, out, final_states,
                                                            tile_states, parts, keep, st);
    return adjoint ? fused_launch_transposed<__bf16, 4>(t, x, dt, A, Bm, Cm, nullptr, init, reset, out, final_states,
                                                        tile_states, nullptr, keep, st)
                   : fused_launch_transposed<__bf16, 3>(t, x, dt, A, Bm, Cm, aux, init, reset, out, final_states,
                                                        tile_states, parts, an, st);
}

}  // namespace ssd
