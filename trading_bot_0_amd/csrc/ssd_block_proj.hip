// The block's projections: out[m, n] = sum_k u[m, k] w[n, k] for a tall u (rows = batch * seqlen, 128 or 256
// columns) and a small weight matrix, bf16 in and out, float32 accumulation (gfx950).
//
// With K of a few hundred the product is bound by memory, not by the matrix cores: u is read once, out written once
// (0.95 GB for 524 288 rows, 256 -> 648).  A workgroup owns a block of at most 160 output columns and a range of
// rows: it puts its rows of w into LDS once (84 KB), and from then on its eight waves run without a barrier -- each
// takes tiles of 32 rows, loads its rows of u straight into MFMA operand fragments (u and w are both contiguous
// along K, so a lane's eight K elements are one 16-byte load; the next tile's rows are in flight during this
// tile's products), and walks the block's columns in chunks of 32 with the w fragments read from LDS.  The MFMA's
// first operand is w, so that a lane ends up with one row m and runs of four consecutive columns n; two chunks are
// collected in an LDS tile of the wave's own and written out with adjacent lanes on adjacent 16-byte pieces of a
// row (stores scattered over 32 rows straight from the accumulators' layout run at a fraction of the memory
// system's rate).
#include <algorithm>

#include "ssd_block_common.h"
#include "ssd_device.h"

namespace ssd {

namespace {

constexpr int kProjWaves = 8;         // waves per workgroup: two per SIMD, 256 registers each
constexpr int kProjBlockCols = 160;   // most output columns per workgroup (their rows of w stay in LDS)
constexpr int kProjChunk = 32;        // output columns per MFMA tile
constexpr int kProjTiles = 8;         // tiles of 32 rows per wave

// CH: 32-column chunks of the widest block of columns (1..5; a block takes CH or CH - 1 chunks, and its last chunk
// may hold fewer columns than it covers).  The chunk count is a template parameter and every store goes out without a condition -- a
// buffer store whose offset is put out of range for rows past M and columns past the block, which the hardware then
// drops -- because loads and stores share one counter per wave, in order: only in straight-line code with every
// store counted does the compiler wait for a tile's rows of u by their exact position in that order.  With a loop of
// unknown length or a guarded store in between it waits for everything outstanding -- the next tile's rows, requested
// a moment ago, and the last stores -- and the tile's loads, products and stores ran one after the other.
template <int KS, int CH>  // K = 16 * KS
__global__ __launch_bounds__(64 * kProjWaves) void block_proj_kernel(const __bf16 *__restrict__ u,
                                                                      const __bf16 *__restrict__ w,
                                                                      __bf16 *__restrict__ out, long long M, int N,
                                                                      int ldo, int col_blocks, int block_cols) {
    constexpr int K = 16 * KS, NTHR = 64 * kProjWaves;
    constexpr int ROWB = K * 2 + 16;        // bytes of a staged row of w: 16 bytes of padding shift the banks
    constexpr int kTileRowB = 64 * 2 + 16;  // a row of a wave's output tile: 64 columns and 16 bytes of padding
    __shared__ __attribute__((aligned(16))) unsigned char wsm[CH * kProjChunk * ROWB];
    __shared__ __attribute__((aligned(16))) unsigned char otile[kProjWaves][32 * kTileRowB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Workgroups go to the eight XCDs in turn, each XCD with an L2 of its own: the column blocks of a range of rows
    // are consecutive workgroups of ONE XCD, so that they run at the same time and all but the first find those
    // rows of u in its L2.
    const int xcd = blockIdx.x % 8, within = blockIdx.x / 8;
    const int cb = within % col_blocks;
    const long long rg = (long long)(within / col_blocks) * 8 + xcd;
    const int n0 = cb * block_cols;                 // this workgroup's first column
    const int ncols = cb == col_blocks - 1 ? N - n0 : block_cols;  // a multiple of 8; the last block takes the rest
    const long long row0 = rg * kProjTiles * (32LL * kProjWaves);
    if (row0 >= M) return;  // the grid is padded to whole rounds of XCDs

    {   // rows n0 .. n0 + 32 * CH - 1 of w, all requested before the first is written to LDS (rows past N repeat the
        // last one, and pieces past the block are the block's last piece once more: neither loads nor writes stand
        // under a condition; the surplus columns are never stored)
        constexpr int PIECES = CH * kProjChunk * (K / 8);
        constexpr int FILL = (PIECES + NTHR - 1) / NTHR;
        uint4 q[FILL];
#pragma unroll
        for (int i = 0; i < FILL; ++i) {
            const int p = min(tid + i * NTHR, PIECES - 1);
            q[i] = *reinterpret_cast<const uint4 *>(w + (size_t)min(n0 + p / (K / 8), N - 1) * K + (p % (K / 8)) * 8);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < FILL; ++i) {
            const int p = min(tid + i * NTHR, PIECES - 1);
            *reinterpret_cast<uint4 *>(wsm + (p / (K / 8)) * ROWB + (p % (K / 8)) * 16) = q[i];
        }
    }
    __syncthreads();

    const int r = lane & 31, half = lane >> 5;
    unsigned char *tile = otile[wave];
    // the workgroup's rows of `out` as a range-checked buffer: 2 048 rows of at most ldo elements
    const __amdgpu_buffer_rsrc_t obuf = make_buffer(out + (size_t)row0 * ldo, (unsigned)min((long long)kProjTiles * 32 * kProjWaves, M - row0) * (unsigned)ldo * 2u);
    auto tile_row0 = [&](int t) { return row0 + (long long)t * (32 * kProjWaves) + wave * 32; };
    // this lane's part of its row of u: K elements 16 ks + 8 half .. + 7 for every K step (rows past M repeat the
    // last row; they are never stored)
    auto load_rows = [&](int t, Frag<__bf16>(&uf)[KS]) {
        const __bf16 *ur = u + (size_t)min(tile_row0(t) + r, M - 1) * K + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) uf[ks].v = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(ur + 16 * ks));
    };
    // (a block takes CH chunks or one fewer -- 648 columns are 4 x 128 + 136 -- and the last chunk is the only piece
    // of a tile's work under a condition, a uniform one)
    const bool last_chunk = ncols > (CH - 1) * kProjChunk;
    constexpr int kRing = KS < 8 ? KS : 8;
    uint4 wq[kRing];  // the next kRing fragments of w
#pragma unroll
    for (int ks = 0; ks < kRing; ++ks) wq[ks] = *reinterpret_cast<const uint4 *>(wsm + r * ROWB + half * 16 + ks * 32);
    auto tile_product = [&](int t, const Frag<__bf16>(&uf)[KS]) {
        const unsigned trow = (unsigned)(t * (32 * kProjWaves) + wave * 32);  // the tile's first row within the workgroup's
        const long long m0 = tile_row0(t);
#pragma unroll
        for (int c0 = 0; c0 < CH; c0 += 2) {
            if (c0 == CH - 1 && !last_chunk) break;  // (an odd CH: the last pair is the last chunk alone)
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                const int c = c0 + sub;
                if (c >= CH || (c == CH - 1 && !last_chunk)) break;
                // the chunk that follows this one (the next tile's first after the last)
                const int cn = (c + 1 < CH && (c + 1 < CH - 1 || last_chunk)) ? c + 1 : 0;
                const unsigned char *wb = wsm + (c * kProjChunk + r) * ROWB + half * 16;
                const unsigned char *wn = wsm + (cn * kProjChunk + r) * ROWB + half * 16;
                f32x16 acc = {0}, acc_odd = {0};  // two chains of dependent MFMAs instead of one
#pragma unroll
                for (int ks = 0; ks < KS; ks += 2) {
                    Frag<__bf16> wf0, wf1;
                    wf0.v = __builtin_bit_cast(bf16x8, wq[ks % kRing]);
                    wf1.v = __builtin_bit_cast(bf16x8, wq[(ks + 1) % kRing]);
                    acc = mma32(wf0, uf[ks], acc);
                    acc_odd = mma32(wf1, uf[ks + 1], acc_odd);
                    // ... and the fragments of w kRing K steps further on (in this chunk or the next), each requested
                    // into the registers of the one just used: kRing / 2 pairs of products lie between a request and
                    // its use (requested right in front of its use, as the compiler orders them when left alone, every
                    // pair of products waits out the LDS latency)
                    const unsigned char *wa = ks + kRing < KS ? wb + kRing * 32 : wn + (kRing - KS) * 32;
                    wq[ks % kRing] = *reinterpret_cast<const uint4 *>(wa + ks * 32);
                    wq[(ks + 1) % kRing] = *reinterpret_cast<const uint4 *>(wa + ks * 32 + 32);
                    __builtin_amdgcn_sched_barrier(0);
                }
                acc = acc + acc_odd;
                // acc[4 vg + i] = out[m, n0 + 32 c + 8 vg + 4 half + i]
#pragma unroll
                for (int vg = 0; vg < 4; ++vg)
                    // (rows 8 .. 15 and 24 .. 31 keep the 8-byte halves of every 16-byte piece the other way round: rows
                    // are 144 bytes apart, so that rows r and r + 8, served together, would otherwise share their banks)
                    *reinterpret_cast<uint2 *>(tile + r * kTileRowB + (sub * 32 + 8 * vg + 4 * (half ^ ((r >> 3) & 1))) * 2) = make_uint2(
                        pack_bf16x2(acc[4 * vg], acc[4 * vg + 1]), pack_bf16x2(acc[4 * vg + 2], acc[4 * vg + 3]));
            }
            // The tile was written by this wave's other lanes: LDS works a wave's requests off in order, so all that
            // is needed is that the compiler keeps the order (a fence would also wait for the stores to memory).
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int pass = 0; pass < 4; ++pass) {
                const int row = pass * 8 + (lane >> 3), col = c0 * kProjChunk + (lane & 7) * 8;
                const u32x4 q = *reinterpret_cast<const u32x4 *>(tile + row * kTileRowB + (lane & 7) * 16);
                const u32x4 v = (pass & 1) ? u32x4{q.z, q.w, q.x, q.y} : q;
                const bool ok = m0 + row < M && col < ncols;
                const unsigned off = ((trow + (unsigned)row) * (unsigned)ldo + (unsigned)(n0 + col)) * 2u;
                __builtin_amdgcn_raw_buffer_store_b128(v, obuf, ok ? off : kBufferDropOffset, 0, 0);
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();
        }
    };
    // Two sets of row fragments: the next tile's rows are requested before this tile's products, because loads and
    // stores complete in order per wave -- requested after, they would wait for this tile's stores to reach memory.
    // (Tiles past M load the last row and store nothing, so that the loop has no exit in its middle.)
    Frag<__bf16> ua[KS], ub[KS];
    load_rows(0, ua);
#pragma unroll
    for (int t = 0; t < kProjTiles; t += 2) {
        load_rows(t + 1, ub);
        tile_product(t, ua);
        if (t + 2 < kProjTiles) load_rows(t + 2, ua);
        tile_product(t + 1, ub);
    }
}


// ------------------------------------------------------------------------------------------------------------------
// Gate + RMSNorm + out-projection in one pass: out[m, n] = sum_k yn[m, k] w[n, k] with
// yn[m, k] = v[m, k] rsqrt(mean_k v[m, k]^2 + eps) norm_w[k], v = y silu(z) -- the normalised row never reaches
// memory (it would be written by one kernel and read back by the next: two thirds of the bytes of a row's y and z).
// A row of the inner width K (128 or 256 channels) is exactly the MFMA's K axis, which a lane pair (r, r + 32) holds
// entirely in its operand fragments: the prologue turns a tile's rows of y and z into fragments of bf16(v) and the
// pair's sum of squares; the norm's weights are folded into the staged matrix (w[n, k] norm_w[k], rounded to bf16)
// and the row's rsqrt factor scales the accumulators, whose lanes hold one row each.  One workgroup takes all
// out_features (at most 256) columns, so that the prologue runs once per row: its rows of w fill 132 KB of LDS, and a
// wave's output tile covers 16 rows at a time to fit beside them.
// ------------------------------------------------------------------------------------------------------------------
constexpr int kPostProjMaxCols = 256;

template <int KS, int CH>  // K = 16 * KS inner channels, CH chunks of 32 output columns
__global__ __launch_bounds__(64 * kProjWaves) void block_post_proj_kernel(
    const __bf16 *__restrict__ y, const __bf16 *__restrict__ zxbcdt, const float *__restrict__ norm_w, float eps,
    const __bf16 *__restrict__ w, __bf16 *__restrict__ out, long long M, int N, int ld_z, int ldo, int tiles) {
    constexpr int K = 16 * KS, NTHR = 64 * kProjWaves, PPR = K / 8;  // 16-byte pieces per row of w
    constexpr int ROWB = K * 2 + 16;  // a staged row of w: 16 bytes of padding shift the banks from row to row
    constexpr int kTileRowB = 64 * 2 + 16;
    __shared__ __attribute__((aligned(16))) unsigned char wsm[CH * kProjChunk * ROWB];
    __shared__ __attribute__((aligned(16))) unsigned char otile[kProjWaves][16 * kTileRowB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long long row0 = (long long)blockIdx.x * tiles * (32LL * kProjWaves);  // tiles: 32-row tiles per wave, 1 .. kProjTiles
    const int r = lane & 31, half = lane >> 5;
    // this lane's K elements are 16 ks + 8 half .. + 7 for every K step
    auto tile_row0 = [&](int t) { return row0 + (long long)t * (32 * kProjWaves) + wave * 32; };
    // A tile's rows of y are requested one tile ahead (they are in flight during the products and stores of the tile
    // before); its rows of z only at the top of the tile: both sets a tile ahead would not fit the registers beside
    // the operand fragments, and the workgroup's other waves fill the SIMD during the wait.
    uint4 yq[KS], zq[KS];
    auto tile_row = [&](int t) { return min(tile_row0(t) + r, M - 1); };  // rows past M repeat the last row; never stored
    auto load_y = [&](int t) {
        const __bf16 *yr = y + (size_t)tile_row(t) * K + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) yq[ks] = *reinterpret_cast<const uint4 *>(yr + 16 * ks);
    };
    auto load_z = [&](int t) {
        const __bf16 *zr = zxbcdt + (size_t)tile_row(t) * ld_z + 8 * half;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) zq[ks] = *reinterpret_cast<const uint4 *>(zr + 16 * ks);
    };
    load_y(0);  // in flight while w is staged
    {   // rows 0 .. 32 CH - 1 of w times norm_w, rounded to bf16 (rows past N repeat the last one: never stored)
        constexpr int PIECES = CH * kProjChunk * PPR;
        constexpr int FILL = (PIECES + NTHR - 1) / NTHR;
#pragma unroll 4
        for (int i = 0; i < FILL; ++i) {
            const int p = min(tid + i * NTHR, PIECES - 1);
            const int row = p / PPR, piece = p % PPR;
            const Pack8<__bf16> q = Pack8<__bf16>::load(w + (size_t)min(row, N - 1) * K + piece * 8);
            const float4 na = *reinterpret_cast<const float4 *>(norm_w + piece * 8);
            const float4 nb = *reinterpret_cast<const float4 *>(norm_w + piece * 8 + 4);
            uint4 o;
            o.x = pack_bf16x2(q.get(0) * na.x, q.get(1) * na.y);
            o.y = pack_bf16x2(q.get(2) * na.z, q.get(3) * na.w);
            o.z = pack_bf16x2(q.get(4) * nb.x, q.get(5) * nb.y);
            o.w = pack_bf16x2(q.get(6) * nb.z, q.get(7) * nb.w);
            *reinterpret_cast<uint4 *>(wsm + row * ROWB + piece * 16) = o;
        }
    }
    __syncthreads();
    if (row0 >= M) return;
    unsigned char *tile = otile[wave];
    const __amdgpu_buffer_rsrc_t obuf = make_buffer(out + (size_t)row0 * ldo, (unsigned)min((long long)tiles * 32 * kProjWaves, M - row0) * (unsigned)ldo * 2u);
    const float inv_k = 1.f / (float)K;
#pragma unroll 1
    for (int t = 0; t < tiles; ++t) {
        // ---- prologue: this tile's rows of y and z -> fragments of bf16(y silu(z)) and the rows' rsqrt factor ----
        load_z(t);
        Frag<__bf16> uf[KS];
        float ss = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const Pack8<__bf16> yy{yq[ks]}, zz{zq[ks]};
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[i] = yy.get(i) * silu(zz.get(i));
                ss += v[i] * v[i];
            }
            uint4 o;
            o.x = pack_bf16x2(v[0], v[1]);
            o.y = pack_bf16x2(v[2], v[3]);
            o.z = pack_bf16x2(v[4], v[5]);
            o.w = pack_bf16x2(v[6], v[7]);
            uf[ks].v = __builtin_bit_cast(bf16x8, o);
        }
        ss += __shfl_xor(ss, 32, 64);
        const float rstd = rsqrtf(ss * inv_k + eps);
        // the next tile's rows of y: requested before this tile's products and stores (loads and stores complete in
        // order per wave: requested behind the stores they would wait for those to reach memory)
        if (t + 1 < tiles) load_y(t + 1);
        const unsigned trow = (unsigned)(t * (32 * kProjWaves) + wave * 32);
        const long long m0 = tile_row0(t);
#pragma unroll
        for (int c0 = 0; c0 < CH; c0 += 2) {
            f32x16 acc[2];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                const int c = c0 + sub;
                acc[sub] = f32x16{0};
                if (c >= CH) break;
                const unsigned char *wb = wsm + (c * kProjChunk + r) * ROWB + half * 16;
                f32x16 acc_odd = {0};
#pragma unroll
                for (int ks = 0; ks < KS; ks += 2) {
                    Frag<__bf16> wf0, wf1;
                    wf0.v = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(wb + ks * 32));
                    wf1.v = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(wb + ks * 32 + 32));
                    acc[sub] = mma32(wf0, uf[ks], acc[sub]);
                    acc_odd = mma32(wf1, uf[ks + 1], acc_odd);
                }
                acc[sub] = (acc[sub] + acc_odd) * rstd;
            }
            // acc[sub][4 vg + i] = out[m0 + r, 32 (c0 + sub) + 8 vg + 4 half + i]; the wave's tile holds 16 rows, so
            // the rows go out in two halves (rows r < 16, then the others)
#pragma unroll
            for (int rh = 0; rh < 2; ++rh) {
                if ((r >> 4) == rh) {
#pragma unroll
                    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
                        for (int vg = 0; vg < 4; ++vg)
                            *reinterpret_cast<uint2 *>(tile + (r & 15) * kTileRowB + (sub * 32 + 8 * vg + 4 * (half ^ ((r >> 3) & 1))) * 2) = make_uint2(
                                pack_bf16x2(acc[sub][4 * vg], acc[sub][4 * vg + 1]), pack_bf16x2(acc[sub][4 * vg + 2], acc[sub][4 * vg + 3]));
                    }
                }
                asm volatile("" ::: "memory");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int pass = 0; pass < 2; ++pass) {
                    const int trw = pass * 8 + (lane >> 3), row = rh * 16 + trw, col = c0 * kProjChunk + (lane & 7) * 8;
                    const u32x4 q = *reinterpret_cast<const u32x4 *>(tile + trw * kTileRowB + (lane & 7) * 16);
                    const u32x4 v = (pass & 1) ? u32x4{q.z, q.w, q.x, q.y} : q;  // (halves swapped in rows 8 .. 15)
                    const bool ok = m0 + row < M && col < N;
                    const unsigned off = ((trow + (unsigned)row) * (unsigned)ldo + (unsigned)col) * 2u;
                    __builtin_amdgcn_raw_buffer_store_b128(v, obuf, ok ? off : kBufferDropOffset, 0, 0);
                }
                asm volatile("" ::: "memory");
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
}

}  // namespace

bool block_proj_supported(long long rows, int in_features, int out_features) {
    return rows > 0 && (in_features == 128 || in_features == 256) && out_features > 0 && out_features % 8 == 0;
}

// Column blocks: equal blocks of at most kProjBlockCols columns (a multiple of 8) -- or, where that takes no more
// workgroups, blocks of 128 with the last one taking the rest (up to kProjBlockCols): every block then starts on a
// multiple of 64 columns, so that with rows a multiple of 128 bytes apart every 128-byte piece a wave writes is one
// whole line of the memory system (648 columns: 4 x 128 + 136 instead of 4 x 136 + 104, 21 column chunks instead of 25).
static void proj_col_blocks(int out_features, int *col_blocks, int *block_cols) {
    const int equal = (out_features + kProjBlockCols - 1) / kProjBlockCols;
    const int by128 = out_features <= kProjBlockCols ? 1 : (out_features - kProjBlockCols + 127) / 128 + 1;
    if (by128 == equal) {
        *col_blocks = by128;
        *block_cols = by128 == 1 ? (out_features + 7) / 8 * 8 : 128;
    } else {
        *col_blocks = equal;
        *block_cols = ((out_features + equal - 1) / equal + 7) / 8 * 8;
    }
}

hipError_t launch_block_proj(long long rows, int in_features, int out_features, int out_ld, const void *u, const void *w,
                             void *out, hipStream_t st) {
    if (!block_proj_supported(rows, in_features, out_features) || out_ld < out_features || out_ld % 8 != 0)
        return hipErrorInvalidValue;
    int col_blocks, block_cols;
    proj_col_blocks(out_features, &col_blocks, &block_cols);
    const long long rows_per_group = 32LL * kProjWaves * kProjTiles;
    const long long groups = ((rows + rows_per_group - 1) / rows_per_group + 7) / 8 * 8 * col_blocks;
    if (groups > 0x7fffffffLL || out_features - (col_blocks - 1) * block_cols > kProjBlockCols ||
        out_features - (col_blocks - 1) * block_cols <= 0)
        return hipErrorInvalidValue;
    const dim3 grid((unsigned)groups), block(64 * kProjWaves);
    const __bf16 *uu = static_cast<const __bf16 *>(u), *ww = static_cast<const __bf16 *>(w);
    __bf16 *oo = static_cast<__bf16 *>(out);
    // the chunks of 32 columns the widest block takes
    const int widest = std::max(block_cols, out_features - (col_blocks - 1) * block_cols);
    const int ch = (widest + kProjChunk - 1) / kProjChunk;
#define SSD_PROJ_CASE(KSv, CHv)                                                                                        \
    if (in_features == 16 * KSv && ch == CHv) {                                                                        \
        block_proj_kernel<KSv, CHv><<<grid, block, 0, st>>>(uu, ww, oo, rows, out_features, out_ld, col_blocks, block_cols); \
        return hipGetLastError();                                                                                      \
    }
    SSD_PROJ_CASE(8, 1) SSD_PROJ_CASE(8, 2) SSD_PROJ_CASE(8, 3) SSD_PROJ_CASE(8, 4) SSD_PROJ_CASE(8, 5)
    SSD_PROJ_CASE(16, 1) SSD_PROJ_CASE(16, 2) SSD_PROJ_CASE(16, 3) SSD_PROJ_CASE(16, 4) SSD_PROJ_CASE(16, 5)
#undef SSD_PROJ_CASE
    return hipErrorInvalidValue;
}

bool block_post_proj_supported(const BlockShape &s, int out_features) {
    const int DI = s.H * s.P;
    return (DI == 128 || DI == 256) && out_features > 0 && out_features <= kPostProjMaxCols && out_features % 8 == 0;
}

// out [B*L, out_features] (row stride out_ld) = rmsnorm(y silu(z)) norm_w . w^T; y [B*L, H*P] bf16, z the first H*P
// channels of zxbcdt's rows (stride s.ld), w [out_features, H*P] bf16.
hipError_t launch_block_post_proj(const BlockShape &s, const void *y, const void *zxbcdt, const float *norm_w, float eps,
                                  const void *w, int out_features, int out_ld, void *out, hipStream_t st) {
    if (!block_post_proj_supported(s, out_features) || out_ld < out_features || out_ld % 8 != 0) return hipErrorInvalidValue;
    const int K = s.H * s.P;
    const long long rows = (long long)s.B * s.L;
    // rows per workgroup: up to kProjTiles tiles of 32 rows per wave, fewer when that would leave CUs without a
    // workgroup (each workgroup stages all of w, as much as 256 of its rows, so more than one tile where rows allow)
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = device_cu_count(dev, &cus);
    if (e != hipSuccess) return e;
    const long long per_tile = 32LL * kProjWaves;
    const int tiles = (int)std::max<long long>(1, std::min<long long>(kProjTiles, rows / (per_tile * cus)));
    const long long rows_per_group = per_tile * tiles;
    const long long groups = (rows + rows_per_group - 1) / rows_per_group;
    if (groups > 0x7fffffffLL || (unsigned long long)rows_per_group * out_ld * 2 > 0x7fffffffULL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)groups), block(64 * kProjWaves);
    const __bf16 *yy = static_cast<const __bf16 *>(y), *zz = static_cast<const __bf16 *>(zxbcdt), *ww = static_cast<const __bf16 *>(w);
    __bf16 *oo = static_cast<__bf16 *>(out);
    const int ch = (out_features + kProjChunk - 1) / kProjChunk;
#define SSD_POST_PROJ_CASE(KSv, CHv)                                                                                   \
    if (K == 16 * KSv && ch == CHv) {                                                                                  \
        block_post_proj_kernel<KSv, CHv><<<grid, block, 0, st>>>(yy, zz, norm_w, eps, ww, oo, rows, out_features, s.ld, out_ld, tiles); \
        return hipGetLastError();                                                                                      \
    }
    SSD_POST_PROJ_CASE(8, 1) SSD_POST_PROJ_CASE(8, 2) SSD_POST_PROJ_CASE(8, 3) SSD_POST_PROJ_CASE(8, 4)
    SSD_POST_PROJ_CASE(8, 5) SSD_POST_PROJ_CASE(8, 6) SSD_POST_PROJ_CASE(8, 7) SSD_POST_PROJ_CASE(8, 8)
    SSD_POST_PROJ_CASE(16, 1) SSD_POST_PROJ_CASE(16, 2) SSD_POST_PROJ_CASE(16, 3) SSD_POST_PROJ_CASE(16, 4)
    SSD_POST_PROJ_CASE(16, 5) SSD_POST_PROJ_CASE(16, 6) SSD_POST_PROJ_CASE(16, 7) SSD_POST_PROJ_CASE(16, 8)
#undef SSD_POST_PROJ_CASE
    return hipErrorInvalidValue;
}

}  // namespace ssd
