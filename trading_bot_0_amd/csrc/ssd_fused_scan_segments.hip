// One-pass forward for batches too small to fill the chip with one workgroup per 8 units: the sequence is cut
// into segments that different workgroups walk side by side.
//   1. states only (no y, no C): what every segment adds to the state, from a zero state, and its total decay;
//   2. the forward proper per segment; each workgroup first runs the recurrence over the states of the segments
//      before its own (a few fused multiply-adds per state element), which gives the state entering its segment.
// Step 1 costs about 0.4 of step 2 (staging, scan and the state update, without the output phase); the two
// together run S times as many workgroups as the uncut kernel.
#include "ssd_fused_scan.h"

namespace ssd {

namespace {

constexpr int kSegmentMinTiles = 4;        // shorter segments are mostly prologue
constexpr int kSegmentTargetGroups = 192;  // workgroups to aim for (256 CUs; the last quarter gains little)

constexpr double kFloatTileUs = 7.5;

int tiles_of(const ScanShape &s) { return (s.L + kOnePassTile - 1) / kOnePassTile; }

}  // namespace

// Which way a forward runs fastest: 0 = staged kernels, 1 = the one-pass kernel, 2 = the one-pass kernel on
// *segments segments.  Estimates in microseconds from measurements on MI355X: a workgroup walks a tile of 64 steps
// in about 6.5 (states only: 0.4 of that) and a CU holds one workgroup, so the one-pass kernel takes that times
// the tiles of a sequence (or segment) times the rounds of 256 workgroups; the staged kernels run every tile of
// every sequence side by side, about 510 per 2048 units x 32 tiles; a launch costs about 5.
int fused_scan_plan(const ScanShape &s, int dtype, int *segments) {
    *segments = 1;
    if (dtype == 0) {
        // float inputs: the one-pass kernel on three bf16 terms per operand walks a tile of 32 steps in about
        // kFloatTileUs (states only: 0.45 of that); the staged float kernels take about 1345 per 2048 units x 32
        // tiles of 64
        if (fused_scan_f32_waves(s) == 0) return 0;
        const long long groups = (long long)s.B * s.G * ((s.H / s.G) * (s.P / 32) / 8);
        const int nc = (s.L + fused_scan_f32_tile() - 1) / fused_scan_f32_tile();
        const double staged = 20.0 + 1345.0 * ((double)groups * 8 * tiles_of(s)) / (2048.0 * 32.0);
        const double whole = 5.0 + kFloatTileUs * nc * (double)((groups + 255) / 256);
        double cut = 1e30;
        int S = 1;
        while (groups * S < kSegmentTargetGroups && nc / (2 * S) >= 2 * kSegmentMinTiles) S *= 2;
        if (S >= 2) {
            const int seg_tiles = (nc + S - 1) / S;
            S = (nc + seg_tiles - 1) / seg_tiles;
            cut = 10.0 + 1.45 * kFloatTileUs * seg_tiles * (double)((groups * S + 255) / 256);
        }
        if (cut < whole && cut < staged) {
            *segments = S;
            return 2;
        }
        return whole < staged ? 1 : 0;
    }
    const int waves = fused_scan_waves(s, dtype);
    if (waves == 4 && s.N != 128) {
        // groups of four units (four heads of 32, two of 64 ...): workgroups of four waves, two to a CU.  A workgroup
        // alone on its CU walks a tile in about 4.2 (one wave per SIMD), two sharing it in about 7.0 each; a round is 512
        // workgroups.  Measured at 2 048 steps, 4 heads of 32, state 64: 256 sequences 144 (staged 263), 512 221
        // (503), 1 024 459 (1 010); 128 sequences 125 against 124, below that the staged kernels win.  Not cut into
        // segments (the states-only instance is the eight-wave one).
        const long long groups = (long long)s.B * s.G * ((s.H / s.G) * (s.P / 32) / 4);
        const int nc = tiles_of(s);
        const double staged = 20.0 + 510.0 * ((double)groups * 4 * nc) / (2048.0 * 32.0);
        const long long rounds = groups / 512, rest = groups % 512;
        const double per_tile = 7.0 * rounds + (rest == 0 ? 0.0 : rest <= 256 ? 4.2 : 4.2 + 2.8 * (double)(rest - 256) / 256.0);
        return 5.0 + per_tile * nc < staged ? 1 : 0;
    }
    const int full = s.N == 128 ? 4 : 8;  // waves of a workgroup that fills a CU
    if (waves != full) return 0;
    const long long groups = (long long)s.B * s.G * ((s.H / s.G) * (s.P / 32) / full);
    const int nc = tiles_of(s);
    const double staged = 20.0 + 510.0 * ((double)groups * full * nc) / (2048.0 * 32.0) * (s.N == 128 ? 2.0 : 1.0);
    const double whole = 5.0 + 6.5 * nc * (double)((groups + 255) / 256);
    double cut = 1e30;
    int S = 1;
    if (s.N != 128) {
        while (groups * S < kSegmentTargetGroups && nc / (2 * S) >= kSegmentMinTiles) S *= 2;
        if (S >= 2) {
            const int seg_tiles = (nc + S - 1) / S;
            S = (nc + seg_tiles - 1) / seg_tiles;
            cut = 15.0 + 1.4 * 6.5 * seg_tiles * (double)((groups * S + 255) / 256);
        }
    }
    if (cut < whole && cut < staged) {
        *segments = S;
        return 2;
    }
    return whole < staged ? 1 : 0;
}

// A batch whose workgroups fill the chip k >= 1 whole times plus a remainder that would be cheaper as a batch of
// its own (by the plan's estimates) than as one more round: the rows of that remainder, else 0.
int fused_scan_tail_rows(const ScanShape &s, int dtype) {
    int segments;
    if (fused_scan_plan(s, dtype, &segments) != 1) return 0;
    if (dtype != 0 && s.N != 128 && fused_scan_waves(s, dtype) == 4) return 0;  // (four-wave workgroups: whole rounds only)
    const int full = (dtype != 0 && s.N == 128) ? 4 : 8;
    const int per_row = s.G * ((s.H / s.G) * (s.P / 32) / full);  // workgroups per batch row
    const long long groups = (long long)s.B * per_row;
    if (groups <= 256 || 256 % per_row != 0) return 0;
    const int rest = (int)(groups % 256);
    if (rest == 0) return 0;
    ScanShape tail = s;
    tail.B = rest / per_row;
    const int tail_plan = fused_scan_plan(tail, dtype, &segments);
    if (tail_plan == 1) return 0;  // it would run as a round of the one-pass kernel anyway
    double cost, round;  // of the remainder as its own batch, as fused_scan_plan estimates it; of one more round
    if (dtype == 0) {
        const int nc = (s.L + fused_scan_f32_tile() - 1) / fused_scan_f32_tile();
        round = kFloatTileUs * nc;
        if (tail_plan == 2) {
            const int seg_tiles = (nc + segments - 1) / segments;
            cost = 10.0 + 1.45 * kFloatTileUs * seg_tiles * (double)(((long long)rest * segments + 255) / 256);
        } else {
            cost = 20.0 + 1345.0 * ((double)rest * 8 * tiles_of(s)) / (2048.0 * 32.0);
        }
    } else {
        const int nc = tiles_of(s);
        round = 6.5 * nc;
        if (tail_plan == 2) {
            const int seg_tiles = (nc + segments - 1) / segments;
            cost = 15.0 + 1.4 * 6.5 * seg_tiles * (double)(((long long)rest * segments + 255) / 256);
        } else {
            cost = 20.0 + 510.0 * ((double)rest * full * nc) / (2048.0 * 32.0) * (s.N == 128 ? 2.0 : 1.0);
        }
    }
    return cost < round ? tail.B : 0;
}

hipError_t launch_fused_scan_segmented(const ScanShape &s, int dtype, int segments, const void *x, const void *dt,
                                       const float *A, const void *Bm, const void *Cm, const float *D, const float *init,
                                       const unsigned char *reset, void *y, float *final_states, float *seg_states,
                                       float *seg_decay, hipStream_t st) {
    if (dtype == 0)
        return launch_fused_scan_f32_segmented(s, segments, x, dt, A, Bm, Cm, D, init, reset, y, final_states, seg_states,
                                               seg_decay, st);
    if (segments < 2 || fused_scan_waves(s, dtype) != 8 || s.N == 128) return hipErrorInvalidValue;
    ScanShape t = s;
    t.Q = kOnePassTile;
    t.nc = tiles_of(s);
    t.seg_tiles = (t.nc + segments - 1) / segments;
    if ((t.nc + t.seg_tiles - 1) / t.seg_tiles != segments) return hipErrorInvalidValue;
    hipError_t e = t.N == 32 ? fused_launch_states<2, kOnePassTile / 32, 8>(t, x, dt, A, Bm, nullptr, reset, seg_states, seg_decay, st)
                             : fused_launch_states<4, kOnePassTile / 32, 8>(t, x, dt, A, Bm, nullptr, reset, seg_states, seg_decay, st);
    if (e != hipSuccess) return e;
    // the forward per segment; its prologue runs the recurrence over the segment states
    ScanShape f = s;
    f.seg_tiles = t.seg_tiles;
    f.seg_local = seg_states;
    f.seg_local_decay = seg_decay;
    return launch_fused_scan(f, dtype, x, dt, A, Bm, Cm, D, init, reset, y, final_states, st);
}

}  // namespace ssd
