// Internal interface between the C ABI (ssd_api.cpp) and the gfx950 kernels (ssd_kernels.hip).
// Shapes arrive here already validated; launchers only pick a template instance and a grid.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace ssd {

struct ScanShape {
    int B, L, H, P, N, G, Q, nc;
    // The one-pass kernel only (the staged path takes these as arguments of launch_chunk_cumsum): decays and input
    // weights of the time-reversed adjoint recurrence.  All tensors are then the forward sequence's, dt_len <= L
    // rows per batch row: the kernel reads x, B, C at row L-1-t for its step t and writes y there (rows outside
    // the tensors are no-op steps), dt and the reset mask at row L-t.
    int mode = 0, dt_len = 0;
    // The one-pass kernel only, shapes with B and C per head (G == H): x is given once per x_groups groups of
    // heads, as a [B, L, x_groups, P] tensor, instead of once per head (0 = per head, [B, L, H, P]).
    int x_groups = 0;
    // The one-pass kernel only: the sequence cut into segments of seg_tiles tiles of 64 steps (0 = not cut) that
    // different workgroups walk; initial states are then given per segment, [B, segments, H, P, N].
    int seg_tiles = 0;
    // The forward on segments: what the states-only pass left, per segment but the last, [B, segments, H, P, N] (the
    // state a segment adds from zero) and [B, segments, H] (its total decay).  A workgroup's prologue runs the
    // recurrence over the segments before its own, from the true initial state [B, H, P, N].
    const float *seg_local = nullptr, *seg_local_decay = nullptr;
    // The staged kernels that read the initial state only: the restart mask [B, L] (or NULL).  A sequence that
    // restarts before its first step does not read its initial state at all, whatever that holds.
    const unsigned char *fresh = nullptr;
};

struct StepShape {
    int B, H, P, N, G;
};

struct BlockShape {  // a Mamba-2 block around the scan: conv width d_conv over the x | B | C channels
    int B, L, H, P, N, G, d_conv;
    int ld;  // elements from one timestep's row of zxbcdt to the next (at least its channel count)
};

constexpr size_t kLdsLimitBytes = 160 * 1024;  // LDS per workgroup on gfx950

// Dynamic LDS the stage-2 / stage-4 workgroup needs (elem_bytes = 2 for bf16, 4 for float).
// (stage 1 transposes a [chunk, nheads] tile of dt through LDS)
inline size_t chunk_cumsum_lds_bytes(const ScanShape &s) { return ((size_t)s.H * (s.Q + 1) + s.Q) * sizeof(float); }
size_t chunk_state_lds_bytes(const ScanShape &s, int elem_bytes);
size_t chunk_scan_lds_bytes(const ScanShape &s, int elem_bytes);

// dtype: 0 = float32, 1 = bf16, 2 = bf16 inputs with float32 y (stage 4 only; stages 1-2 treat it as 1).
// dtcs is the stage-1 output [B,H,nc,4,Q] float32: log2(e) * cumulative dt*A as a hi/lo pair, dt, and
// the stage-2 weight exp2(alpha[Q-1] - alpha[l]) * dt[l].
// reset: [B,L] bytes or NULL; a non-zero entry restarts the state from zero before that timestep
// mode 0: decays exp(dt_t A) and input weights dt_t (the forward).  mode 1: the time-reversed adjoint
// recurrence of the backward pass: step t decays by exp(dt_{L-t} A) and every step weighs one; dt then has
// dt_len <= L rows per batch row (0 = L) and steps whose L-t falls outside 1..dt_len-1 do not decay, so a
// reversed sequence can carry L - dt_len leading no-op steps that pad it to whole chunks.  reset is then the
// forward sequence's mask ([B,dt_len]): a restart before forward step L-t cuts the adjoint at reversed step t.
hipError_t launch_chunk_cumsum(const ScanShape &s, int dtype, const void *dt, const float *A,
                               const unsigned char *reset, float *dtcs, hipStream_t stream, int mode = 0,
                               int dt_len = 0);
hipError_t launch_chunk_state(const ScanShape &s, int dtype, const void *x, const void *Bm,
                              const float *dtcs, float *states, hipStream_t stream);
// stages 2+3 in one pass: writes the state entering each chunk into `prev` and the final state
hipError_t launch_chunk_state_scan(const ScanShape &s, int dtype, const void *x, const void *Bm,
                                   const float *dtcs, const float *init, float *prev, float *final_states,
                                   hipStream_t stream);
hipError_t launch_state_passing(const ScanShape &s, const float *states, const float *dtcs,
                                const float *init, float *prev, float *final_states,
                                hipStream_t stream);
hipError_t launch_chunk_scan(const ScanShape &s, int dtype, const void *x, const void *Bm,
                             const void *Cm, const float *dtcs, const float *prev, const float *D,
                             void *y, hipStream_t stream);
// The whole forward in one pass (bf16 inputs): no workspace, nothing but x, dt, B, C read and y, final written.
// fused_scan_waves is 0 when the shape cannot run there, else the waves per workgroup it would use.
// tile_states (optional, [B, ceil(L/64), H, P, N]): the state entering every tile of 64 steps.
int fused_scan_waves(const ScanShape &s, int dtype);
hipError_t launch_fused_scan(const ScanShape &s, int dtype, const void *x, const void *dt, const float *A,
                             const void *Bm, const void *Cm, const float *D, const float *init,
                             const unsigned char *reset, void *y, float *final_states, hipStream_t stream,
                             float *tile_states = nullptr);
// The one-pass forward with the sequence cut into segments that run side by side (bf16 inputs, dstate 32 or 64):
// first every segment's own contribution to the state and its total decay (states only, no y, no C), then the
// state entering every segment by a recurrence over the segments, then the forward proper per segment.
// seg_states [B, segments, H, P, N] and seg_decay [B, segments, H] are scratch of the caller.
// Float inputs on the one-pass kernel (three bf16 terms per operand): fused_scan_f32_waves is 0 when the shape
// cannot run there, else the waves per workgroup (8).
int fused_scan_f32_waves(const ScanShape &s);
hipError_t launch_fused_scan_f32(const ScanShape &s, const void *x, const void *dt, const float *A, const void *Bm,
                                 const void *Cm, const float *D, const float *init, const unsigned char *reset, void *y,
                                 float *final_states, hipStream_t st);
int fused_scan_f32_tile();  // time steps per tile of the float one-pass kernel
hipError_t launch_fused_scan_f32_segmented(const ScanShape &s, int segments, const void *x, const void *dt, const float *A,
                                           const void *Bm, const void *Cm, const float *D, const float *init,
                                           const unsigned char *reset, void *y, float *final_states, float *seg_states,
                                           float *seg_decay, hipStream_t st);
// fused_scan_plan: which way a forward of this shape runs fastest by the library's cost estimates: 0 = the
// staged kernels, 1 = the one-pass kernel, 2 = the one-pass kernel on *segments segments.
int fused_scan_plan(const ScanShape &s, int dtype, int *segments);
// fused_scan_tail_rows: for a batch that fills the chip a whole number of times and a bit, the batch rows of
// that bit when it is cheaper run as a batch of its own than as one more round of the one-pass kernel; else 0.
int fused_scan_tail_rows(const ScanShape &s, int dtype);
hipError_t launch_fused_scan_segmented(const ScanShape &s, int dtype, int segments, const void *x, const void *dt,
                                       const float *A, const void *Bm, const void *Cm, const float *D, const float *init,
                                       const unsigned char *reset, void *y, float *final_states, float *seg_states,
                                       float *seg_decay, hipStream_t stream);
hipError_t launch_step(const StepShape &s, int dtype, float *state, const void *x, const void *dt,
                       const float *A, const void *Bm, const void *Cm, const float *D, void *y,
                       hipStream_t stream);

// nsteps consecutive single-timestep updates in one launch (state in registers), reset [B,nsteps] bytes or NULL:
// a non-zero entry zeroes that batch row before the step.  Tensors as for the scan: x,y [B,T,H,P], dt [B,T,H],
// Bm,Cm [B,T,G,N].  steps_supported: headdim 16, 32 or 64.
bool steps_supported(const StepShape &s);
hipError_t launch_steps(const StepShape &s, int nsteps, int dtype, float *state, const unsigned char *reset,
                        const void *x, const void *dt, const float *A, const void *Bm, const void *Cm,
                        const float *D, void *y, hipStream_t stream);

// The memory-bound stages of a Mamba-2 block around the scan.  zxbcdt [B,L,E], E = 2*H*P + 2*G*N + H, laid out
// per timestep as [ z | x | B | C | dt_raw ].  pre: conv1d + bias + SiLU over x|B|C into the scan's tensors and
// dt = softplus(dt_raw + dt_bias); conv state [B, d_conv-1, H*P + 2*G*N] in the activation dtype (both optional);
// reset [B,L] bytes or NULL: a non-zero entry cuts the filter's history before that timestep.
// post: out [B,L,H*P] = rmsnorm(y * silu(z)) * norm_w.  dtype 2 = bf16 activations with float32 y.
bool block_supported(const BlockShape &s);
// The block's projections in bf16: out [rows, out_features] = u [rows, in_features] . w [out_features, in_features]^T,
// float32 accumulation.  in_features 128 or 256, out_features a multiple of 8.
bool block_proj_supported(long long rows, int in_features, int out_features);
hipError_t launch_block_proj(long long rows, int in_features, int out_features, int out_ld, const void *u, const void *w,
                             void *out, hipStream_t st);
hipError_t launch_block_pre(const BlockShape &s, int dtype, const void *zxbcdt, const float *conv_w,
                            const float *conv_b, const float *dt_bias, const void *state_in, void *state_out,
                            const unsigned char *reset, void *x, void *Bm, void *Cm, void *dt, hipStream_t stream);
bool block_step_supported(const BlockShape &s, int d_model);
hipError_t launch_block_step(const BlockShape &s, int dtype, int d_model, const void *u, const void *w_in, const float *conv_w,
                             const float *conv_b, const float *dt_bias, const float *A, const float *D, const float *norm_w,
                             float eps, const void *w_out, void *conv_state, float *ssm_state, void *out, hipStream_t st);
bool block_post_proj_supported(const BlockShape &s, int out_features);
hipError_t launch_block_post_proj(const BlockShape &s, const void *y, const void *zxbcdt, const float *norm_w, float eps,
                                  const void *w, int out_features, int out_ld, void *out, hipStream_t st);
hipError_t launch_block_post(const BlockShape &s, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                             float eps, void *out, hipStream_t stream);

// Backward of the two stages (dtype as the forward's; dtype 2 = bf16 activations with the scan's float32 y in
// post_bwd).  dzxbcdt [B,L,ld] is the gradient of zxbcdt: post_bwd writes its z channels, pre_bwd its x | B | C | dt
// channels.  workspace: block_bwd_workspace_bytes (partial sums of the parameter gradients).  With yn given
// ([B,L,H*P], the activation type) post_bwd also writes the forward's normalised rows, bit for bit what
// launch_block_post writes, for a forward that did not keep them.
size_t block_bwd_workspace_bytes(const BlockShape &s);
hipError_t launch_block_post_bwd(const BlockShape &s, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                                 float eps, const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, void *workspace,
                                 hipStream_t stream, void *yn = nullptr);
hipError_t launch_block_pre_bwd(const BlockShape &s, int dtype, const void *zxbcdt, const float *conv_w, const float *conv_b,
                                const float *dt_bias, const void *state_in, const unsigned char *reset, const void *dx,
                                const void *dB, const void *dC, const void *ddt, const void *dstate_out, void *dzxbcdt,
                                float *dconv_w, float *dconv_b, float *ddt_bias, void *dstate_in, void *workspace,
                                hipStream_t stream);

// The backward pass's two scans of the transposed state with the sum over a group's heads taken on chip (bf16,
// headdim 32, eight heads per group; sT is the transposed shape: P = dstate, N = 32, G = H; sT.mode / dt_len as
// for the one-pass kernel when adjoint).  x [B,L,x_groups,P] is the operand a group's heads share, Bm and Cm
// [B,L,H,32] are per head.  out [B,L,x_groups,P] (bf16) = the sum over each group's heads of the per-head
// outputs, weighted by the heads' dt when adjoint.  Forward in time it also writes parts [B,L,H,P/32]: per head
// and 32-column slice, aux_t . y_t (aux [B,L,x_groups,P]).  tile_states / final_states as for the one-pass kernel.
// With `an.out` given, the scan that runs second (transposed_scan_anchors_in_adjoint says which takes them) also
// writes, per (b, k, h) for k = 0 .. nc in forward time and per 32-column slice, the inner product of the two scans'
// states at the start of forward tile k (k = nc: the end of the sequence): its own state entering its tile j with
// other_tiles[b, nc - j, h] for 0 < j < nc, its initial state with other_final (zero without an initial state), its
// final state with other_init (zero when NULL).  out [B, nc+1, H, P/32], float64.
// stride > 1: the two scans meet at every stride-th tile boundary of forward time only (k = 0, stride, 2 stride, ..
// and nc); the other entries of `out` are left alone.  The scan that runs first then keeps only the states entering
// its tiles c = phase, phase + stride, .. in tile_states [B, (nc - 1 - phase) / stride + 1, H, P, N] (phase = 0 for
// the forward scan, nc % stride for the adjoint one, whose tile c starts where forward tile nc - c ends), and is
// given stride and phase in `an` as well (its `out` stays NULL).
struct ScanAnchors {
    const float *other_tiles = nullptr, *other_final = nullptr, *other_init = nullptr;
    double *out = nullptr;
    int stride = 1, phase = 0;
};
bool transposed_scan_anchors_in_adjoint(const ScanShape &sT);
bool transposed_scan_supported(const ScanShape &sT, int x_groups);
hipError_t launch_transposed_scan(const ScanShape &sT, bool adjoint, const void *x, const void *dt, const float *A,
                                  const void *Bm, const void *Cm, const void *aux, const float *init,
                                  const unsigned char *reset, void *out, float *final_states, float *tile_states,
                                  float *parts, const ScanAnchors &an, hipStream_t stream);

// The backward pass's reversed-adjoint scan with the row products in its epilogue (bf16, headdim 32, heads per
// group a multiple of eight, dstate 32 or 64).  sR is the forward shape with L padded to whole tiles, mode 1 and
// dt_len = the true length; all tensors are the forward sequence's.  Writes dx = dt r + D dy [B,L,H,32] (bf16), the
// adjoint state at step 0 into g0 [B,H,32,N], and per (b,t,h) the pair (x . r, dy . x) into pairs, float2 [B,L,H].
bool adjoint_rows_scan_supported(const ScanShape &sR);
hipError_t launch_adjoint_rows_scan(const ScanShape &sR, const void *dy, const void *dt, const float *A, const void *Cm,
                                    const void *Bm, const float *D, const void *x, const float *dfinal,
                                    const unsigned char *reset, void *dx, float *g0, float *pairs, hipStream_t stream);

// The memory-bound kernels of the backward pass (its three heavy products run on the stage launchers above with
// the operands' roles swapped).  dtype: 0 = float32, 1 = bf16 activations and gradients.
// gather_rows: dst[b, t', (g*rep + k)*W + w] = src[b, t, g*W + w] for t' < Ldst, with t = Ldst-1-t' if reverse
// else t'; rows with t >= Lsrc are zero.  W a multiple of 8.
hipError_t launch_gather_rows(int dtype, const void *src, void *dst, int B, int Lsrc, int Ldst, int groups, int W,
                              int rep, bool reverse, hipStream_t stream);
// out [rows, H*rep] = in [rows, H] with every column repeated rep times (dtype: 0 = float32, 1 = bf16)
hipError_t launch_replicate_columns(int dtype, const void *in, void *out, long long rows, int H, int rep, hipStream_t stream);
// [BH, P, N] -> [BH, N, P]
hipError_t launch_transpose_state(const float *src, float *dst, long long BH, int P, int N, hipStream_t stream);
// per (b,t,h): dx = D dy + dt r, e1 = x . r, dd = dy . x, u = C . yC - dt e1.  r_rev (and yB_rev below) hold
// Lrev >= L rows per batch row, row Lrev-1-t for timestep t; Lrev = 0: L rows in forward order.
// With yB_rev (LrevB rows, as Lrev) the same pass also writes dB and dC, the sums over a group's heads of dt yB
// and yC (what launch_bwd_group_sums does otherwise); bwd_rows_can_sum: nheads/ngroups is 1, 2, 4 or 8.
bool bwd_rows_can_sum(const ScanShape &s);
hipError_t launch_bwd_rows(const ScanShape &s, int Lrev, int dtype, const void *x, const void *dy, const void *dt, const void *Cm,
                           const float *D, const float *r_rev, const float *yC, void *dx, float *e1, float *dd,
                           float *u, hipStream_t stream, const float *yB_rev = nullptr, int LrevB = 0,
                           void *dB = nullptr, void *dC = nullptr);
// The same without the transposed scans' per-head outputs: C . yC comes as parts [B,L,H,nparts] to add up
// (launch_transposed_scan wrote them, and dB and dC).
hipError_t launch_bwd_rows_parts(const ScanShape &s, int Lrev, int dtype, const void *x, const void *dy, const void *dt,
                                 const float *D, const float *r_rev, const float *parts, int nparts, void *dx,
                                 float *e1, float *dd, float *u, hipStream_t stream);
// dB = sum over a group's heads of dt yB (yB_rev time-reversed), dC = the same of yC
hipError_t launch_bwd_group_sums(const ScanShape &s, int Lrev, int dtype, const void *dt, const float *yB_rev, const float *yC,
                                 void *dB, void *dC, hipStream_t stream);
// anchor [B,nc+1,H]: q at the first step of chunk c = exp(dt A) <adjoint state, forward state> entering the chunk:
// fwd_prev [B,nc,H,N,P] are the forward-time transposed scan's chunk states, rev_prev those of the reversed one
// (chunk nc-c there), rev_final its final state and init_t the transposed initial state (NULL = zero) for c = 0;
// c = nc is the end of the sequence, <dfin_t, fwd_final> (zero when dfin_t is NULL).  reset [B,L] or NULL: an
// anchor is zero where the sequence restarts before the chunk's first step.
hipError_t launch_bwd_anchors(const ScanShape &s, int dtype, const void *dt, const float *A, const float *fwd_prev,
                              const float *rev_prev, const float *rev_final, const float *init_t, const float *fwd_final,
                              const float *dfin_t, const unsigned char *reset, double *anchor, hipStream_t stream);
// q_t between the anchors of its chunk (chunk <= 64 steps); ddt = e1 + A q; dA_part[h,b,c] = the chunk's sum of
// dt q, dD_part[h,b,c] = its sum of dd.  With parts given ([B,L,H,nparts], the pieces of C . yC), e1 holds the
// pairs (e1, dd) of the adjoint scan with row products and u = sum of the parts - dt e1 is formed here (u and dd
// unused).
// With raw_anchors > 0, anchor holds that many pieces per (b, c, h) ([B, nc+1, H, raw_anchors], as ScanAnchors
// writes them) of the two states' inner product, and the first step's decay exp(dt A) -- zero where `reset` marks
// the chunk's first step -- is applied here.
// anchor_stride > 1 (a power of two up to 8, where bwd_ddt_anchor_stride_supported): q is known only at every
// anchor_stride-th chunk boundary and at the end of the sequence, the u are summed over the chunks in between and
// their mismatch is spread over all of those steps.
bool bwd_ddt_anchor_stride_supported(const ScanShape &s, int raw_anchors);
hipError_t launch_bwd_ddt(const ScanShape &s, int dtype, const void *dt, const float *A, const float *e1, const float *u,
                          const float *dd, const double *anchor, void *ddt, double *dA_part, double *dD_part,
                          hipStream_t stream, const float *parts = nullptr, int nparts = 0,
                          const unsigned char *reset = nullptr, int raw_anchors = 0, int anchor_stride = 1);
// dA[h], dD[h] (NULL allowed) = the sums over batch and chunks of the parts
hipError_t launch_bwd_head_sums(const ScanShape &s, const double *dA_part, const double *dD_part, float *dA, float *dD,
                                hipStream_t stream);
hipError_t launch_bwd_dinit(const ScanShape &s, int dtype, const void *dt, const float *A, const float *gfin,
                            const unsigned char *reset, float *dinit, hipStream_t stream);

}  // namespace ssd
