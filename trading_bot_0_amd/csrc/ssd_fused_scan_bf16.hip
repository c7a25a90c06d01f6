// One-pass forward, bf16 inputs and bf16 y; also the shape test and the entry the C ABI calls.
#include "ssd_fused_scan.h"

namespace ssd {

hipError_t launch_fused_scan_y32(const ScanShape &, int, const void *, const void *, const float *, const void *,
                                 const void *, const float *, const float *, const unsigned char *, void *, float *,
                                 float *, hipStream_t);

bool fused_scan_wide_supported(const ScanShape &);
hipError_t launch_fused_scan_wide(const ScanShape &, int, const void *, const void *, const float *, const void *,
                                  const void *, const float *, const float *, const unsigned char *, void *, float *,
                                  hipStream_t);

int fused_scan_waves(const ScanShape &s, int dtype) {
    if (dtype == 0) return 0;                         // float inputs take the staged kernels
    if (s.P % 32 != 0) return 0;
    if (s.N != 32 && s.N != 64 && s.N != 128) return 0;
    const int units = (s.H / s.G) * (s.P / 32);
    int waves = (units % 8 == 0) ? 8 : ((units % 4 == 0) ? 4 : 0);
    // a 128-wide state takes a wave's whole register file: four waves per workgroup, one per SIMD
    if (s.N == 128) waves = (units % 4 == 0) ? 4 : 0;
    if (waves == 0 && units % 2 == 0 && s.N == 32 && dtype == 2) waves = 2;  // float y only: the backward's scans
    if (waves == 0 || fused_scan_lds_bytes(s.N, kOnePassTile, waves) > kLdsLimitBytes) return 0;
    // the kernel writes a batch row's y through a 32-bit-offset buffer descriptor
    if ((long long)(s.L > s.dt_len ? s.L : s.dt_len) * s.H * s.P * 4 >= (1LL << 31)) return 0;
    return waves;
}

hipError_t launch_fused_scan(const ScanShape &s, int dtype, const void *x, const void *dt, const float *A,
                             const void *Bm, const void *Cm, const float *D, const float *init,
                             const unsigned char *reset, void *y, float *final_states, hipStream_t st,
                             float *tile_states) {
    if (dtype == 0) {
        if (tile_states != nullptr) return hipErrorInvalidValue;
        return launch_fused_scan_f32(s, x, dt, A, Bm, Cm, D, init, reset, y, final_states, st);
    }
    const int waves = fused_scan_waves(s, dtype);
    if (waves == 0) return hipErrorInvalidValue;
    if (s.x_groups != 0 && (s.G != s.H || s.H % s.x_groups != 0 || (s.P / 32) % waves != 0)) return hipErrorInvalidValue;
    ScanShape t = s;  // the kernel's own tiling of time; the caller's chunk length does not enter
    t.Q = kOnePassTile;
    t.nc = (s.L + kOnePassTile - 1) / kOnePassTile;
    // a 128-wide state: two waves per unit (the one-wave-per-unit instance stays for callers that want the state
    // entering every tile, which that kernel can write)
    if (tile_states == nullptr && fused_scan_wide_supported(t))
        return launch_fused_scan_wide(t, dtype, x, dt, A, Bm, Cm, D, init, reset, y, final_states, st);
    if (dtype == 2)
        return launch_fused_scan_y32(t, waves, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
    return fused_dispatch<__bf16>(t, waves, x, dt, A, Bm, Cm, D, init, reset, y, final_states, tile_states, st);
}

}  // namespace ssd
