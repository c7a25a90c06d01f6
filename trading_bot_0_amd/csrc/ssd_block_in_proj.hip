// The block's in-projection with the pre-scan stage in its epilogue (gfx950, bf16): zxbcdt = u . w^T, and from the
// x | B | C | dt channels of every row, before they leave the chip, the tensors the scan takes --
// x, B, C = silu(causal depthwise conv over time + bias), dt = softplus(dt_raw + dt_bias).  Run as two kernels those
// channels are written by the projection and read straight back by the pre-scan stage (0.8 GB of the block's 3.8 GB at
// 524 288 rows of 256 -> 648 channels); here only z goes to zxbcdt (and, for a caller that will run the backward pass,
// the raw x | B | C | dt channels it needs), and x, B, C, dt are written once.
//
// The product is block_proj_kernel's: a workgroup owns a block of 128 (the last: up to 160) output columns and 2 048
// rows, its rows of w in LDS, eight waves without a barrier, a wave's rows of u straight into MFMA operand fragments,
// two chunks of 32 columns collected in an LDS tile of the wave's own.  What differs:
//  * a wave's eight tiles of 32 rows are CONSECUTIVE rows (a run of 256 timesteps of one sequence: seqlen must be a
//    multiple of 256), so that the conv's window carries over from tile to tile: the last three rows of a tile stay
//    in a small ring in LDS (one per pair of column chunks) for the next tile of the run;
//  * before its first tile a wave fills the rings -- from conv_state_in (or zeros) where the run starts a sequence,
//    else with one more tile of products over the 32 rows in front of its run, of which the last three are kept;
//  * the tile is rounded to bf16 when it goes to LDS, exactly as zxbcdt's rows are, and the conv, SiLU and softplus
//    are block_pre_kernel's expressions, so that the results equal the two kernels' bit for bit.
// The conv's taps are zero-padded to four per channel (a shorter filter's leading taps are zeros: adding 0 * x
// changes no sum), so the filter length is not a template parameter.
#include <algorithm>

#include "ssd_block_common.h"

namespace ssd {

namespace {

constexpr int kInWaves = 8;
constexpr int kInChunk = 32;
constexpr int kInTiles = 8;           // tiles of 32 rows per wave: a run of 256 consecutive rows
constexpr int kInRun = 32 * kInTiles;
constexpr int kInBlockCols = 128;     // columns per workgroup; the last block takes up to 160
constexpr int kInMaxCols = 160;
constexpr int kHalo = 3;              // rows of history a tile needs (filter length 4; shorter filters use fewer)

// element i (a compile-time index) of eight bf16 values held in a uint4, as a float
__device__ inline float bf16_at(const uint4 &q, int i) {
    const unsigned w = (i >> 1) == 0 ? q.x : (i >> 1) == 1 ? q.y : (i >> 1) == 2 ? q.z : q.w;
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
}

struct InProjArgs {
    const __bf16 *u, *w;
    const float *conv_w, *conv_b, *dt_bias;
    const __bf16 *state_in;
    __bf16 *state_out, *zx, *x, *Bm, *Cm, *dt;
    long long M;
    int N, ldo, col_blocks, L, DI, GN, H, d_conv, write_raw;
};

template <int KS, int CH>  // K = 16 * KS, CH chunks of 32 columns in the widest block
__global__ __launch_bounds__(64 * kInWaves) void block_in_proj_pre_kernel(const InProjArgs a) {
    constexpr int K = 16 * KS, NTHR = 64 * kInWaves;
    constexpr int ROWB = K * 2 + 16;
    constexpr int kTileRowB = 64 * 2 + 16;
    constexpr int PAIRS = (CH + 1) / 2;
    __shared__ __attribute__((aligned(16))) unsigned char wsm[CH * kInChunk * ROWB];
    __shared__ __attribute__((aligned(16))) unsigned char otile[kInWaves][32 * kTileRowB];
    __shared__ __attribute__((aligned(16))) unsigned char ring[kInWaves][PAIRS][kHalo * 128];
    __shared__ __attribute__((aligned(16))) float taps[CH * kInChunk][4];  // per column of the block: four taps
    __shared__ __attribute__((aligned(16))) float biases[CH * kInChunk];   // conv bias, or dt_bias for the dt columns
    const int tid = threadIdx.x, lane = tid & 63;
    // (in a scalar register: the wave's buffer descriptors below are built from it, and a descriptor the compiler cannot
    // prove uniform is stored through a loop over its distinct values)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int xcd = blockIdx.x % 8, within = blockIdx.x / 8;
    const int cb = within % a.col_blocks;
    const long long rg = (long long)(within / a.col_blocks) * 8 + xcd;
    const int N = a.N, DI = a.DI, C = DI + 2 * a.GN;
    const int n0 = cb * kInBlockCols;
    const int ncols = cb == a.col_blocks - 1 ? N - n0 : kInBlockCols;
    const long long row0 = rg * kInWaves * (long long)kInRun;
    if (row0 >= a.M) return;  // the grid is padded to whole rounds of XCDs

    {   // this block's rows of w (as block_proj_kernel stages them)
        constexpr int PIECES = CH * kInChunk * (K / 8);
        constexpr int FILL = (PIECES + NTHR - 1) / NTHR;
        uint4 q[FILL];
#pragma unroll
        for (int i = 0; i < FILL; ++i) {
            const int p = min(tid + i * NTHR, PIECES - 1);
            q[i] = *reinterpret_cast<const uint4 *>(a.w + (size_t)min(n0 + p / (K / 8), N - 1) * K + (p % (K / 8)) * 8);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < FILL; ++i) {
            const int p = min(tid + i * NTHR, PIECES - 1);
            *reinterpret_cast<uint4 *>(wsm + (p / (K / 8)) * ROWB + (p % (K / 8)) * 16) = q[i];
        }
        // the conv's taps (zero-padded in front to four) and biases of this block's columns
        for (int c = tid; c < CH * kInChunk; c += NTHR) {
            const int col = n0 + c;
            float t4[4] = {0.f, 0.f, 0.f, 0.f}, bias = 0.f;
            if (col >= DI && col < DI + C) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {  // tap k of four is tap k - (4 - d_conv) of the filter
                    const int kk = k - (4 - a.d_conv);
                    t4[k] = kk >= 0 ? a.conv_w[(size_t)(col - DI) * a.d_conv + kk] : 0.f;
                }
                bias = a.conv_b[col - DI];
            } else if (col >= DI + C && col < N) {
                bias = a.dt_bias[col - DI - C];
            }
            taps[c][0] = t4[0];
            taps[c][1] = t4[1];
            taps[c][2] = t4[2];
            taps[c][3] = t4[3];
            biases[c] = bias;
        }
    }
    __syncthreads();

    const int r = lane & 31, half = lane >> 5;
    unsigned char *tile = otile[wave];
    const long long run0 = row0 + (long long)wave * kInRun;  // this wave's first row
    if (run0 >= a.M) return;                                 // (no barrier follows)
    const int t_run = (int)(run0 % a.L);                     // its timestep: runs never straddle sequences
    const long long bidx = run0 / a.L;
    const bool block_has_conv = n0 + ncols > DI;             // anything but z in this block
    // the wave's rows of every output as range-checked buffers (stores to rows past M are dropped by the hardware)
    const unsigned run_rows = (unsigned)min((long long)kInRun, a.M - run0);
    const __amdgpu_buffer_rsrc_t zbuf = make_buffer(a.zx + (size_t)run0 * a.ldo, run_rows * (unsigned)a.ldo * 2u);
    const __amdgpu_buffer_rsrc_t xbuf = make_buffer(a.x + (size_t)run0 * DI, run_rows * (unsigned)DI * 2u);
    const __amdgpu_buffer_rsrc_t bbuf = make_buffer(a.Bm + (size_t)run0 * a.GN, run_rows * (unsigned)a.GN * 2u);
    const __amdgpu_buffer_rsrc_t cbuf = make_buffer(a.Cm + (size_t)run0 * a.GN, run_rows * (unsigned)a.GN * 2u);
    const __amdgpu_buffer_rsrc_t dbuf = make_buffer(a.dt + (size_t)run0 * a.H, run_rows * (unsigned)a.H * 2u);

    auto load_rows = [&](long long first, Frag<__bf16>(&uf)[KS]) __attribute__((always_inline)) {  // rows first .. first + 31 (clamped into u)
        const __bf16 *ur = a.u + (size_t)min(max(first + r, 0LL), a.M - 1) * K + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) uf[ks].v = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(ur + 16 * ks));
    };
    const bool last_chunk = ncols > (CH - 1) * kInChunk;
    // products of one pair of column chunks into the wave's tile (bf16, as zxbcdt holds them)
    auto pair_products = [&](int c0, const Frag<__bf16>(&uf)[KS], f32x16 (&acc)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            const int c = c0 + sub;
            acc[sub] = f32x16{0};
            if (c >= CH) break;  // (a block narrower than CH chunks computes columns it never stores)
            const unsigned char *wb = wsm + (c * kInChunk + r) * ROWB + half * 16;
            f32x16 acc_odd = {0};
#pragma unroll
            for (int ks = 0; ks < KS; ks += 2) {
                Frag<__bf16> wf0, wf1;
                wf0.v = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(wb + ks * 32));
                wf1.v = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(wb + ks * 32 + 32));
                acc[sub] = mma32(wf0, uf[ks], acc[sub]);
                acc_odd = mma32(wf1, uf[ks + 1], acc_odd);
            }
            acc[sub] = acc[sub] + acc_odd;
        }
    };

    // ---- the rings before the run's first tile ----
    if (block_has_conv) {
        if (t_run == 0) {
            // the sequence starts here: its history is conv_state_in's rows (the last d_conv-1 of them; the ring's
            // older rows meet zero taps) or zeros
#pragma unroll
            for (int pr = 0; pr < PAIRS; ++pr) {
                for (int i = lane; i < kHalo * 8; i += 64) {
                    const int hr = i / 8, col = n0 + pr * 64 + (i % 8) * 8;  // ring row hr is timestep hr - 3
                    uint4 v = make_uint4(0, 0, 0, 0);
                    const int sr = hr - (kHalo - (a.d_conv - 1));            // its row of conv_state_in
                    if (a.state_in != nullptr && sr >= 0 && col >= DI && col < DI + C)
                        v = *reinterpret_cast<const uint4 *>(a.state_in + ((size_t)bidx * (a.d_conv - 1) + sr) * C + (col - DI));
                    *reinterpret_cast<uint4 *>(ring[wave][pr] + hr * 128 + (i % 8) * 16) = v;
                }
            }
        } else {
            // one more tile of products over the 32 rows in front of the run; rows 29 .. 31 of it are the history
            Frag<__bf16> uh[KS];
            load_rows(run0 - 32, uh);
#pragma unroll
            for (int c0 = 0; c0 < CH; c0 += 2) {
                if (c0 == CH - 1 && !last_chunk) break;
                f32x16 acc[2];
                pair_products(c0, uh, acc);
                if (r >= 32 - kHalo) {
#pragma unroll
                    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
                        for (int vg = 0; vg < 4; ++vg)
                            *reinterpret_cast<uint2 *>(ring[wave][c0 / 2] + (r - (32 - kHalo)) * 128 + (sub * 32 + 8 * vg + 4 * half) * 2) =
                                make_uint2(pack_bf16x2(acc[sub][4 * vg], acc[sub][4 * vg + 1]), pack_bf16x2(acc[sub][4 * vg + 2], acc[sub][4 * vg + 3]));
                    }
                }
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
    }

    // where the run ends a sequence its last d_conv-1 raw rows are the conv state the call returns
    const bool ends_sequence = a.state_out != nullptr && t_run + kInRun == a.L;

    // One tile.  The pairs of column chunks go in a fixed order that ends with a pair every block has (an odd last
    // chunk, which only the widest block has, goes first): behind that pair's products the fragments of u are dead and
    // take the next tile's rows, which are then in flight during the pair's epilogue and stores -- requested behind the
    // stores they would wait for those to reach memory (loads and stores complete in order per wave), and a second set
    // of fragments, which would let them start a tile earlier, does not fit the registers beside the epilogue.
    auto tile_product = [&](int t, Frag<__bf16>(&uf)[KS]) __attribute__((always_inline)) {
        const unsigned trow = (unsigned)(t * 32);  // the tile's first row within the run
#pragma unroll
        for (int ci = 0; ci < PAIRS; ++ci) {
            const int c0 = (CH % 2) ? (ci == 0 ? CH - 1 : 2 * (ci - 1)) : 2 * ci;
            if (c0 == CH - 1 && !last_chunk) continue;
            f32x16 acc[2];
            pair_products(c0, uf, acc);
            if (ci == PAIRS - 1 && t + 1 < kInTiles) {
                // (the products above have read the fragments: the loads may overwrite them)
#pragma unroll
                for (int sub = 0; sub < 2; ++sub) asm volatile("" : "+v"(acc[sub]));
                load_rows(run0 + (t + 1) * 32, uf);
            }
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
                for (int vg = 0; vg < 4; ++vg)
                    *reinterpret_cast<uint2 *>(tile + r * kTileRowB + (sub * 32 + 8 * vg + 4 * half) * 2) = make_uint2(
                        pack_bf16x2(acc[sub][4 * vg], acc[sub][4 * vg + 1]), pack_bf16x2(acc[sub][4 * vg + 2], acc[sub][4 * vg + 3]));
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();
            const int pcol = c0 * kInChunk + (lane & 7) * 8;  // this lane's piece of eight columns, within the block
            const int col = n0 + pcol;
            if (n0 + c0 * kInChunk + 64 <= DI) {
                // a pair of chunks inside z: the rows go out as they are
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) {
                    const int row = pass * 8 + (lane >> 3);
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(tile + row * kTileRowB + (lane & 7) * 16);
                    const unsigned off = ((trow + (unsigned)row) * (unsigned)a.ldo + (unsigned)col) * 2u;
                    __builtin_amdgcn_raw_buffer_store_b128(v, zbuf, pcol < ncols ? off : kBufferDropOffset, 0, 0);
                }
            } else {
                // this lane: rows 4 rq .. 4 rq + 3 of its piece, with the three rows before them (of the tile, or of
                // the ring: the last rows of the tile before)
                const int rq = lane >> 3;
                const unsigned char *rg_base = ring[wave][c0 / 2] + (lane & 7) * 16;
                uint4 raw[4 + kHalo];
#pragma unroll
                for (int j = 0; j < 4 + kHalo; ++j) {
                    const int row = 4 * rq - kHalo + j;
                    const unsigned char *src = row >= 0 ? tile + row * kTileRowB + (lane & 7) * 16 : rg_base + (row + kHalo) * 128;
                    raw[j] = *reinterpret_cast<const uint4 *>(src);
                }
                // the ring takes this tile's last three rows (every lane has read what it needs of the ring: LDS works
                // a wave's requests off in order)
                if (rq == 7) {
#pragma unroll
                    for (int j = 0; j < kHalo; ++j)
                        *reinterpret_cast<uint4 *>(ring[wave][c0 / 2] + j * 128 + (lane & 7) * 16) = raw[4 + j];
                }
                // Where the pair's results go: H*P and G*N are multiples of 64 and so is the pair's first column, so a
                // pair lies in ONE tensor -- x, B, C or dt -- and its buffer is the same for every lane (a descriptor
                // that differed from lane to lane would be stored through a loop over its distinct values, at which the
                // compiler waits for everything outstanding).
                const int pair_col = n0 + c0 * kInChunk;   // (uniform)
                const bool in_block = pcol < ncols && col < N;
                const bool is_z = false, is_dt = pair_col >= DI + C;
                const int cc = pair_col - DI;
                const __amdgpu_buffer_rsrc_t obuf = is_dt ? dbuf : cc < DI ? xbuf : cc < DI + a.GN ? bbuf : cbuf;
                const unsigned old = (unsigned)(is_dt ? a.H : cc < DI ? DI : a.GN);
                const unsigned ocol = (unsigned)(col - (is_dt ? DI + C : cc < DI ? DI : cc < DI + a.GN ? 2 * DI : 2 * DI + a.GN));
                const bool is_conv = !is_dt;
                // (every store below is issued by every lane, its offset put out of range where the lane has nothing to
                // write: a store under a condition is a branch, and the compiler then waits for the next tile's rows of u
                // together with every store in front of them)
                // one channel at a time (its taps, its seven rows), so that few values are live beside the rows of u;
                // the dt pair (one per projection) and the conv pairs are two straight-line paths under a uniform branch
                unsigned opk[4][4];  // the four rows' results, packed in pairs of channels
                // (pieces past the widest block's chunks -- the missing half of an odd last pair -- read the tables'
                // last entries; nothing of them is stored)
                const int tc0 = min(pcol, CH * kInChunk - 8);
                if (is_dt) {
#pragma unroll
                    for (int ip = 0; ip < 4; ++ip) {
                        const float b0 = biases[tc0 + 2 * ip], b1 = biases[tc0 + 2 * ip + 1];
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj)
                            opk[jj][ip] = pack_bf16x2(softplus(bf16_at(raw[jj + kHalo], 2 * ip) + b0),
                                                      softplus(bf16_at(raw[jj + kHalo], 2 * ip + 1) + b1));
                    }
                } else {
#pragma unroll
                    for (int ip = 0; ip < 4; ++ip) {
                        float o2[2][4];
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            const int i = 2 * ip + e;
                            const float4 t4 = *reinterpret_cast<const float4 *>(taps[tc0 + i]);
                            const float bias = biases[tc0 + i];
                            const float tp[4] = {t4.x, t4.y, t4.z, t4.w};
                            float win[4 + kHalo];
#pragma unroll
                            for (int j = 0; j < 4 + kHalo; ++j) win[j] = bf16_at(raw[j], i);
#pragma unroll
                            for (int jj = 0; jj < 4; ++jj) {
                                float sc = bias;
#pragma unroll
                                for (int k = 0; k < 4; ++k) sc += tp[k] * win[jj + k];
                                o2[e][jj] = silu(sc);
                            }
                        }
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) opk[jj][ip] = pack_bf16x2(o2[0][jj], o2[1][jj]);
                    }
                }
                const bool raw_out = in_block && (is_z || a.write_raw != 0), act_out = in_block && !is_z;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const unsigned row = trow + 4u * (unsigned)rq + (unsigned)jj;
                    const uint4 cur = raw[jj + kHalo];
                    __builtin_amdgcn_raw_buffer_store_b128(u32x4{cur.x, cur.y, cur.z, cur.w}, zbuf,
                                                           raw_out ? (row * (unsigned)a.ldo + (unsigned)col) * 2u : kBufferDropOffset, 0, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(u32x4{opk[jj][0], opk[jj][1], opk[jj][2], opk[jj][3]}, obuf,
                                                           act_out ? (row * old + ocol) * 2u : kBufferDropOffset, 0, 0);
                }
                if (ends_sequence && t == kInTiles - 1 && rq == 7 && is_conv && in_block) {
                    // rows 29 .. 31 of the run's last tile (raw[4 .. 6]): the last d_conv-1 of them are the new state
#pragma unroll
                    for (int j = 0; j < kHalo; ++j) {
                        const int k = j - (kHalo - (a.d_conv - 1));
                        if (k >= 0)
                            *reinterpret_cast<uint4 *>(a.state_out + ((size_t)bidx * (a.d_conv - 1) + k) * C + (col - DI)) = raw[4 + j];
                    }
                }
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();
        }
    };
    Frag<__bf16> uf[KS];
    load_rows(run0, uf);
#pragma unroll
    for (int t = 0; t < kInTiles; ++t) tile_product(t, uf);
}

}  // namespace

// Whether the fused kernel takes the shape: bf16, 128 or 256 input channels, sequences of whole runs of 256 steps, a
// channel layout whose pairs of column chunks never straddle two tensors (H*P and G*N multiples of 64), and an output
// wide enough for blocks of 128 columns.
bool block_in_proj_pre_supported(const BlockShape &s, int d_model) {
    const int DI = s.H * s.P, GN = s.G * s.N, E = 2 * DI + 2 * GN + s.H;
    // (H*P and G*N multiples of 64: a pair of column chunks then never straddles two of x | B | C | dt)
    if (!(d_model == 128 || d_model == 256) || s.L % kInRun != 0 || s.H % 8 != 0 || DI % 64 != 0 || GN % 64 != 0) return false;
    if (s.d_conv < 2 || s.d_conv > 4 || E <= kInMaxCols) return false;
    const int blocks = (E - kInMaxCols + kInBlockCols - 1) / kInBlockCols + 1;
    const int last = E - (blocks - 1) * kInBlockCols;
    return last > 0 && last <= kInMaxCols && s.ld % 8 == 0 && s.ld >= E;
}

// zx [B*L, s.ld]: z channels always, the raw x | B | C | dt channels too when write_raw; x [B*L, H*P], Bm, Cm
// [B*L, G*N], dt [B*L, H]; conv_state_in / conv_state_out [B, d_conv-1, C] or NULL.
hipError_t launch_block_in_proj_pre(const BlockShape &s, int d_model, const void *u, const void *w, const float *conv_w,
                                    const float *conv_b, const float *dt_bias, const void *state_in, void *state_out,
                                    int write_raw, void *zx, void *x, void *Bm, void *Cm, void *dt, hipStream_t st) {
    if (!block_in_proj_pre_supported(s, d_model)) return hipErrorInvalidValue;
    const int DI = s.H * s.P, GN = s.G * s.N, E = 2 * DI + 2 * GN + s.H;
    const long long rows = (long long)s.B * s.L;
    const int col_blocks = (E - kInMaxCols + kInBlockCols - 1) / kInBlockCols + 1;
    const int widest = std::max(kInBlockCols, E - (col_blocks - 1) * kInBlockCols);
    const int ch = (widest + kInChunk - 1) / kInChunk;
    const long long rows_per_group = (long long)kInWaves * kInRun;
    const long long groups = ((rows + rows_per_group - 1) / rows_per_group + 7) / 8 * 8 * col_blocks;
    if (groups > 0x7fffffffLL || (unsigned long long)kInRun * s.ld * 2 > 0x7fffffffULL) return hipErrorInvalidValue;
    InProjArgs a{static_cast<const __bf16 *>(u), static_cast<const __bf16 *>(w), conv_w, conv_b, dt_bias,
                 static_cast<const __bf16 *>(state_in), static_cast<__bf16 *>(state_out), static_cast<__bf16 *>(zx),
                 static_cast<__bf16 *>(x), static_cast<__bf16 *>(Bm), static_cast<__bf16 *>(Cm), static_cast<__bf16 *>(dt),
                 rows, E, s.ld, col_blocks, s.L, DI, GN, s.H, s.d_conv, write_raw};
    const dim3 grid((unsigned)groups), block(64 * kInWaves);
#define SSD_IN_PROJ_CASE(KSv, CHv)                                             \
    if (d_model == 16 * KSv && ch == CHv) {                                    \
        block_in_proj_pre_kernel<KSv, CHv><<<grid, block, 0, st>>>(a);         \
        return hipGetLastError();                                              \
    }
    SSD_IN_PROJ_CASE(8, 4) SSD_IN_PROJ_CASE(8, 5) SSD_IN_PROJ_CASE(16, 4) SSD_IN_PROJ_CASE(16, 5)
#undef SSD_IN_PROJ_CASE
    return hipErrorInvalidValue;
}

}  // namespace ssd
