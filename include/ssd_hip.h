/*
 * libssd_hip -- C ABI of the MI355X (gfx950) Mamba-2 SSD chunk-scan forward and the
 * single-timestep streaming update.
 *
 * What each entry point replaces in CarsonBurke/trading_bot_0: the SSD op itself is no longer
 * in that tree (only its benchmark rows survive, benchmark_results/bench_20260112_070055.json:
 * 7,16,25,34), so the citations name the slot each call fills and the FFI conventions it
 * follows.  Conventions are those of the tree's own extern "C" boundary, the vendored
 * torch-sys shim:
 *   - errors never cross the ABI as exceptions; a failing call returns non-zero and leaves a
 *     malloc'd message in a thread-local slot fetched (and cleared) by
 *     ssd_get_and_reset_last_err(), which the caller frees with free()
 *     (vendor/torch-sys-0.25.0/libtch/torch_api.h:18-24,33; torch_api.cpp:32,84-88;
 *     polled from Rust at trading_bots/src/torch/cuda/graph.rs:107-119);
 *   - tensors stay owned by the caller and arrive as raw device pointers, the value of
 *     Tensor::data_ptr() (vendor/torch-sys-0.25.0/src/lib.rs:38, libtch/torch_api.cpp:180);
 *     the library retains nothing between calls;
 *   - all work is enqueued on the stream handed in (NULL = the legacy default stream), with no
 *     allocation and no synchronisation, so a call can sit inside the reference's captured
 *     update (trading_bots/src/torch/train/update.rs:206-330; torch_api.cpp:408-464);
 *   - every entry point is re-entrant: no global mutable state, unlike the FA4 bridge that
 *     needs a process-wide lock (trading_bots/src/torch/fa4.rs:11,50-55).
 *
 * Tensor layouts (all contiguous row-major, last stride 1; every pointer 16-byte aligned):
 *   x, y        [batch, seqlen, nheads, headdim]      element type = dtype
 *   dt          [batch, seqlen, nheads]               dtype; already positive, no softplus/bias
 *   A, D        [nheads]                              float32; A < 0; D may be NULL
 *   Bm, Cm      [batch, seqlen, ngroups, dstate]      dtype; head h uses group h/(nheads/ngroups)
 *   states      [batch, nheads, headdim, dstate]      float32 (initial, final, streaming)
 *   dtcs        [batch, nheads, nchunks, 4, chunk]    float32 (stage 1 output): rows 0 and 1 are
 *               log2(e) times the per-chunk inclusive cumulative sum of dt*A, as an unevaluated
 *               pair hi + lo (later stages only use differences of it, which the pair keeps
 *               exact to the difference's own rounding, and turn them into decays with one
 *               exp2), row 2 is dt, row 3 is the decay from each step to the end of its chunk
 *               times dt (the weight stage 2 applies to x)
 *   chunk states[batch, nchunks, nheads, headdim, dstate] float32 (stages 2-4)
 * Recurrence: h_t = exp(dt_t A_h) h_{t-1} + dt_t x_t (outer) B_t ; y_t = h_t . C_t + D_h x_t.
 *
 * Supported shapes: dstate in {16,32,64,128}; headdim a multiple of 8, <= 64; chunk in
 * {32,64,128,256}; nheads % ngroups == 0; the LDS tile of stage 4 must fit 160 KiB (all bf16
 * shapes do; float32 up to headdim 64 / dstate 64 / chunk 256 or dstate 128 / chunk 128).
 * seqlen need not be a multiple of chunk: the ragged tail behaves as dt = 0 padding.
 */
#ifndef SSD_HIP_H
#define SSD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SSD_DTYPE_F32 0  /* all tensors float32 */
#define SSD_DTYPE_BF16 1 /* x, dt, Bm, Cm, y bfloat16; A, D, states, accumulators float32 */
#define SSD_DTYPE_BF16_Y32 2 /* as 1, but y is written as float32 (no output rounding) */

#define SSD_OK 0
#define SSD_ERR_INVALID 1     /* NULL/misaligned pointer, non-positive or inconsistent dims */
#define SSD_ERR_UNSUPPORTED 2 /* shape outside the kernels' tile set */
#define SSD_ERR_WORKSPACE 3   /* workspace smaller than ssd_workspace_bytes() */
#define SSD_ERR_RUNTIME 4     /* the HIP runtime rejected a launch */

typedef struct ssd_dims {
    int64_t batch, seqlen, nheads, headdim, dstate, ngroups, chunk;
} ssd_dims;

typedef struct ssd_step_dims {
    int64_t batch, nheads, headdim, dstate, ngroups;
} ssd_step_dims;

/* Library version (major*10000 + minor*100 + patch). */
int ssd_version(void);

/* Thread-local last error, malloc'd; NULL when none.  Same contract as get_and_reset_last_err
 * (vendor/torch-sys-0.25.0/libtch/torch_api.h:33, torch_api.cpp:84-88). */
char *ssd_get_and_reset_last_err(void);

/* Bytes of scratch ssd_chunk_scan_fwd needs for these dims.  The reference lets ATen allocate
 * op temporaries; a capturable op cannot, so the caller owns the buffer (the Rust side would
 * hold it as a Tensor::empty, cf. the persistent rollout buffers at
 * trading_bots/src/torch/train/trainer.rs:622-944). */
int ssd_workspace_bytes(const ssd_dims *dims, size_t *out_bytes);

/* Whole forward: stages 1-4 on one stream.  Fills y and, when non-NULL, final_states.
 * Slot: the temporal encoder's sequence mixer, TradingModel::patch_trunk
 * (trading_bots/src/torch/model/trading_model.rs:589-606), reached from the batched replay
 * forward (trading_bots/src/torch/model/stream/replay.rs:83-114) and from prefix
 * initialisation of a stream (trading_bots/src/torch/model/stream/live.rs:322-360);
 * historical benchmark rows mamba2_forward_train / mamba2_infer_prefill
 * (benchmark_results/bench_20260112_070055.json:7,25). */
int ssd_chunk_scan_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt,
                       const float *A, const void *Bm, const void *Cm, const float *D,
                       const float *initial_states, void *y, float *final_states,
                       void *workspace, size_t workspace_bytes, void *hip_stream);

/* Stage 1: per-chunk inclusive cumulative sum of dt*A (times log2 e, hi/lo pair) and dt as float32
 * -> dtcs. */
int ssd_chunk_cumsum_fwd(const ssd_dims *dims, int dtype, const void *dt, const float *A, float *dtcs,
                         void *hip_stream);

/* Stage 2: per-chunk states S[b,c,h,p,n] = sum_l exp(cs[Q-1]-cs[l]) dt[l] x[l,p] B[l,n], cs the
 * cumulative sum of dt*A inside chunk c. */
int ssd_chunk_state_fwd(const ssd_dims *dims, int dtype, const void *x, const void *Bm,
                        const float *dtcs, float *chunk_states, void *hip_stream);

/* Stages 2 and 3 in one pass: prev_states[c] receives the state entering chunk c, final_states the state
 * after the last chunk; the per-chunk states stay on chip.  Parallel over (batch, head) sequences only;
 * ssd_chunk_scan_fwd uses it when there are enough of them.  initial_states / final_states may be NULL
 * and may alias each other. */
int ssd_chunk_state_passing_fwd(const ssd_dims *dims, int dtype, const void *x, const void *Bm,
                                const float *dtcs, const float *initial_states, float *prev_states,
                                float *final_states, void *hip_stream);

/* The whole forward in one kernel and one pass over the inputs: a wave keeps the running
 * state of 32 head-dim columns of one (batch, head) in registers while it walks the chunks, so no workspace
 * is needed and nothing but x, dt, B, C is read and y, final_states written.  Same arguments (with the
 * optional reset mask of ssd_chunk_scan_reset_fwd) and results as ssd_chunk_scan_fwd.  Parallel over
 * (batch, head) sequences only; ssd_chunk_scan_fwd takes this path by itself when there are enough of them (groups of
 * eight such units in workgroups of eight waves; groups of four in workgroups of four waves, two to a CU; a 128-wide
 * state with two waves per unit, half of the state each).  SSD_ERR_UNSUPPORTED unless headdim is a
 * multiple of 32 and, for bf16 inputs (dtype 1 or 2), dstate is 32, 64 or 128 and (nheads/ngroups)*(headdim/32) a
 * multiple of 4; for float32 inputs (every operand enters the matrix cores as three bf16 terms, six products per
 * multiplication: float accuracy at three eighths of the float instruction's cost), dstate is 32 or 64 and
 * (nheads/ngroups)*(headdim/32) a multiple of 8.  dims->chunk must
 * be a valid chunk length but does not enter: with no workspace layout to honour, the kernel tiles time by
 * its own block (64 steps, float32 inputs 32; results agree with every chunk length to rounding).  Replaces the same slot as ssd_chunk_scan_fwd (model/trading_model.rs:589-606). */
int ssd_chunk_scan_onepass_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                               const void *Bm, const void *Cm, const float *D, const float *initial_states,
                               const uint8_t *reset, void *y, float *final_states, void *hip_stream);

/* ssd_chunk_scan_fwd with restarts inside the sequences: reset [B,L] bytes or NULL; a non-zero reset[b,t]
 * sets the state of batch row b to zero before timestep t, i.e. y[b,t..] and the final state see nothing
 * from before t (an episode boundary inside a replayed window: the reset slots of
 * trading_bots/src/torch/train/rollout.rs:130-135 landing inside the chunks that
 * trading_bots/src/torch/model/stream/replay.rs:83-114 replays).  reset[b,0] != 0 discards
 * initial_states[b].  Implemented as a drop of the cumulative log-decay at t, so it costs nothing beyond
 * reading the mask.  ssd_chunk_scan_fwd is this function with reset = NULL. */
int ssd_chunk_scan_reset_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                             const void *Bm, const void *Cm, const float *D, const float *initial_states,
                             const uint8_t *reset, void *y, float *final_states, void *workspace,
                             size_t workspace_bytes, void *hip_stream);

/* ssd_chunk_scan_reset_fwd for callers that cannot allocate device memory at all -- code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc -- and so cannot bring a workspace: the scratch the staged and
 * segmented paths need comes from an array of SSD_STATIC_SCRATCH_BYTES (64 MiB) that is part of the library's device
 * code (each GPU the library runs on holds it until the process ends).  No counterpart in the reference.  Same
 * arguments and results as ssd_chunk_scan_reset_fwd minus the workspace.  SSD_ERR_WORKSPACE when the scratch that the
 * shape's own path uses exceeds the array: all of ssd_workspace_bytes on the staged kernels, the segment states and
 * decays (batch * segments * nheads * (headdim * dstate + 1) floats) when the sequences run cut into segments
 * (ssd_chunk_scan_segments > 1), nothing when the shape runs as one launch of the one-pass kernel
 * (ssd_chunk_scan_is_onepass), at any size.  Calls no hipMalloc/hipFree or any other allocating
 * routine.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (different streams or
 * threads) race on it; calls on one stream are ordered and safe.  Nothing in the array has to start at zero (every
 * kernel writes what it later reads), so it is not cleared between calls.
 * Under graph capture: the first call on a device places the array there and looks its address up, and the first call
 * for a shape asks the runtime for occupancy figures and raises LDS limits -- none of that may run inside a capture.
 * Make one call per device and shape outside the capture first; every later call of that shape issues kernel launches
 * only and can be captured and replayed. */
#define SSD_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int ssd_chunk_scan_noalloc_fwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A,
                               const void *Bm, const void *Cm, const float *D, const float *initial_states,
                               const uint8_t *reset, void *y, float *final_states, void *hip_stream);

/* *is_onepass = 1 if ssd_chunk_scan_fwd runs these dims as one launch of the one-pass kernel (its workspace is
 * then not touched), 0 otherwise (staged kernels, the one-pass kernel on segments, or a batch whose partial
 * last round of workgroups runs as a batch of its own).  A plan query like ssd_workspace_bytes; no reference counterpart. */
int ssd_chunk_scan_is_onepass(const ssd_dims *dims, int dtype, int *is_onepass);

/* *segments > 1 if ssd_chunk_scan_fwd runs these dims as the one-pass kernel on that many segments of the
 * sequence side by side (batches too small to fill the chip with whole sequences, long enough to be worth
 * cutting: a states-only pass per segment, a recurrence over the segments, then the forward per segment; the
 * segment states live in the workspace).  1 otherwise.  A plan query; no reference counterpart. */
int ssd_chunk_scan_segments(const ssd_dims *dims, int dtype, int *segments);

/* Stage 3: sequential recurrence over chunks.  prev_states[c] receives the state entering
 * chunk c and may alias chunk_states (in place); final_states and initial_states may be NULL
 * and may alias each other. */
int ssd_state_passing_fwd(const ssd_dims *dims, const float *chunk_states, const float *dtcs,
                          const float *initial_states, float *prev_states, float *final_states,
                          void *hip_stream);

/* Stage 4: intra-chunk masked (C B^T o decay) x plus the C.h readout of the entering state
 * plus D x. */
int ssd_chunk_scan_stage_fwd(const ssd_dims *dims, int dtype, const void *x, const void *Bm,
                             const void *Cm, const float *dtcs, const float *prev_states,
                             const float *D, void *y, void *hip_stream);

/* One recurrent update, in place on state [B,H,P,N]:  x,y [B,H,P]; dt [B,H]; Bm,Cm [B,G,N].
 * Slot: the per-bar streaming step step_uniform_stream_state_on_device
 * (trading_bots/src/torch/model/stream/live.rs:228-244), called per bar from
 * trading_bots/src/torch/infer/offline.rs:124-125 and per rollout step from
 * trading_bots/src/torch/train/rollout.rs:209-235; historical row mamba2_infer_step
 * (benchmark_results/bench_20260112_070055.json:34). */
int ssd_step_fwd(const ssd_step_dims *dims, int dtype, float *state, const void *x,
                 const void *dt, const float *A, const void *Bm, const void *Cm, const float *D,
                 void *y, void *hip_stream);

/* nsteps consecutive recurrent updates in ONE launch, in place on state [B,H,P,N], with per-row resets:
 * x,y [B,T,H,P]; dt [B,T,H]; Bm,Cm [B,T,G,N] (T = nsteps; the layout of the scan's tensors, so slices of a
 * sequence can be passed); reset [B,T] bytes or NULL: a non-zero reset[b,t] zeroes batch row b of the state
 * before step t.  The state stays in registers between the steps, so it crosses HBM once per launch instead
 * of once per step, and T launches become one.  nsteps = 1 with a mask is the fused "reset some rows, then
 * step" of a rollout (advance -> reset slots -> forward: trading_bots/src/torch/train/rollout.rs:130-135,
 * 209-235; trading_bots/src/torch/model/stream/state.rs:10-21 for what a reset is).  headdim 16, 32 or 64;
 * other head sizes return SSD_ERR_UNSUPPORTED (call ssd_step_fwd per step instead).  Results are those of
 * ssd_step_fwd applied nsteps times; for bf16 inputs and 16 steps or more, shapes the one-pass scan takes run on
 * it (the state as its initial and final state, the mask as its restarts), which is several times faster and
 * agrees with the step-by-step results to rounding. */
int ssd_steps_fwd(const ssd_step_dims *dims, int64_t nsteps, int dtype, float *state, const uint8_t *reset,
                  const void *x, const void *dt, const float *A, const void *Bm, const void *Cm, const float *D,
                  void *y, void *hip_stream);

/* ---- Backward pass of the scan ("next" after the forward) ------------------------------------------------
 * Gradients of ssd_chunk_scan_fwd's outputs with respect to all of its inputs, so that a trainer can replay a
 * window through the scan and update through it (trading_bots/src/torch/train/update.rs:206-330 is the captured
 * update this would run in; the reference's historical benchmark case is mamba2_fwd_bwd_train,
 * benchmark_results/bench_20260112_070055.json:16-23).  dtype 0 = float32, 1 = bf16 (activations and their
 * gradients in that type; A, D, states and their gradients float32).
 * In: the forward's inputs (reset [B,L] as for ssd_chunk_scan_reset_fwd, NULL = none), dy [B,L,H,P], and
 * optionally dfinal_states [B,H,P,N] (NULL if the final state does not reach the loss).
 * Out: dx [B,L,H,P], ddt [B,L,H], dA [H], dB, dC [B,L,G,N], dD [H] (NULL allowed; must be NULL without D),
 * dinitial_states [B,H,P,N] (NULL allowed; defined also when the forward had no initial state).
 * headdim 16, 32 or 64 (the pass runs the forward's kernels on the transposed state, a 128-wide state in two parts of
 * 64 rows); other shapes return SSD_ERR_UNSUPPORTED.  Workspace size from ssd_chunk_scan_bwd_workspace_bytes. */
int ssd_chunk_scan_bwd_workspace_bytes(const ssd_dims *dims, int dtype, size_t *out_bytes);
int ssd_chunk_scan_bwd(const ssd_dims *dims, int dtype, const void *x, const void *dt, const float *A, const void *Bm,
                       const void *Cm, const float *D, const float *initial_states, const uint8_t *reset, const void *dy,
                       const float *dfinal_states, void *dx, void *ddt, float *dA, void *dB, void *dC, float *dD,
                       float *dinitial_states, void *workspace, size_t workspace_bytes, void *hip_stream);

/* ---- The memory-bound stages of a Mamba-2 block around the scan ("next" after the scan itself) ----------
 * The layer that would take GqaBlock's place in patch_trunk (trading_bots/src/torch/model/trading_model.rs:
 * 589-606, trading_bots/src/torch/model/blocks/gqa.rs:82-109; the reference already mixes with a causal
 * depthwise filter, gqa.rs:172-178): in-projection -> [pre] -> SSD scan -> [post] -> out-projection.  The two
 * projections are plain GEMMs and stay with the caller's BLAS; pre and post are these two kernels.
 * zxbcdt [B,L,E] is the in-projection's output, E = 2*H*P + 2*G*N + H channels per timestep laid out as
 * [ z | x | B | C | dt_raw ]; activations are float32 (dtype 0) or bf16 (dtype 1; dtype 2 = bf16 with the
 * scan's float32 y as the input of post); parameters are float32. */
typedef struct {
    int64_t batch, seqlen, nheads, headdim, dstate, ngroups, d_conv;
    /* elements from one timestep's row of zxbcdt to the next: 0 = E (dense), else at least E and a whole number of
     * 16-byte pieces.  Rows a multiple of 128 bytes apart (704 for E = 648 in bf16) keep every row's lines of the
     * memory system whole, which the in-projection's stores gain most from. */
    int64_t zxbcdt_ld;
} ssd_block_dims;

/* x [B,L,H,P], Bm, Cm [B,L,G,N] = silu(causal depthwise conv1d of width d_conv (2..4) over the x | B | C
 * channels + conv_b) and dt [B,L,H] = softplus(dt_raw + dt_bias): exactly the tensors ssd_chunk_scan_fwd takes.
 * conv_w [H*P + 2*G*N, d_conv] (tap d_conv-1 multiplies the current timestep), conv_b [H*P + 2*G*N].
 * conv_state_in [B, d_conv-1, H*P + 2*G*N] (activation dtype) holds the x | B | C inputs of the d_conv-1
 * timesteps before the first one (NULL = zeros); conv_state_out (nullable) receives those of the last d_conv-1
 * timesteps: the conv's streaming state, carried next to the SSM state (cf. StreamState,
 * trading_bots/src/torch/model/trading_model.rs:56-75).  The two may alias only for seqlen 1. */
int ssd_block_pre_fwd(const ssd_block_dims *dims, int dtype, const void *zxbcdt, const float *conv_w,
                      const float *conv_b, const float *dt_bias, const void *conv_state_in, void *conv_state_out,
                      void *x, void *Bm, void *Cm, void *dt, void *hip_stream);

/* ssd_block_pre_fwd with episode boundaries inside the window: reset [B,L] bytes or NULL (the mask
 * ssd_chunk_scan_reset_fwd takes); a non-zero reset[b,t] cuts the filter's history before timestep t -- the inputs
 * of earlier timesteps (and conv_state_in) count as zeros from t on, in the outputs and in conv_state_out -- so that
 * a replayed window with reset slots (trading_bots/src/torch/train/rollout.rs:130-135) equals the rollout that
 * zeroed the conv state between steps (trading_bots/src/torch/model/stream/state.rs:10-21).  ssd_block_pre_fwd is
 * this function with reset = NULL. */
int ssd_block_pre_reset_fwd(const ssd_block_dims *dims, int dtype, const void *zxbcdt, const float *conv_w,
                            const float *conv_b, const float *dt_bias, const void *conv_state_in, void *conv_state_out,
                            const uint8_t *reset, void *x, void *Bm, void *Cm, void *dt, void *hip_stream);

/* The block's two projections (the reference's equivalents are the linear layers around its temporal mixer,
 * trading_bots/src/torch/model/blocks/gqa.rs:82-109): out [rows, out_features] = u [rows, in_features] .
 * w [out_features, in_features]^T, bfloat16 in and out (dtype 1), float32 accumulation; rows = batch * seqlen.
 * in_features must be 128 or 256 and out_features a multiple of 8 (SSD_ERR_UNSUPPORTED otherwise: use the
 * caller's BLAS).  out_ld = elements from one row of out to the next (0 = out_features; else at least that and a
 * multiple of 8): the padding columns are not written.  No bias. */
int ssd_block_proj_fwd(int64_t rows, int64_t in_features, int64_t out_features, int64_t out_ld, int dtype, const void *u,
                       const void *w, void *out, void *hip_stream);

/* out [B,L,H*P] = rmsnorm(y * silu(z)) * norm_w over the H*P channels of a timestep (z from zxbcdt). */
int ssd_block_post_fwd(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt,
                       const float *norm_w, float eps, void *out, void *hip_stream);

/* ssd_block_post_fwd and the out-projection behind it as one kernel: out [B*L, out_features] (row stride out_ld
 * elements, 0 = out_features) = rmsnorm(y * silu(z)) * norm_w . w [out_features, H*P]^T, so that the normalised rows
 * never reach memory (the reference's counterpart is the output linear layer of its temporal mixer,
 * trading_bots/src/torch/model/blocks/gqa.rs:82-109).  bfloat16 only (dtype 1: y, zxbcdt, w and out bf16, float32
 * accumulation), H*P 128 or 256, out_features a multiple of 8 up to 256; SSD_ERR_UNSUPPORTED otherwise (run the two
 * stages).  Rounding differs from the two stages' by where it happens: the gated row and the weights times norm_w
 * are rounded to bf16 once each, the row's rsqrt factor is applied to the float32 sums. */
int ssd_block_post_proj_fwd(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                            float eps, const void *w, int64_t out_features, int64_t out_ld, void *out, void *hip_stream);

/* One timestep of the whole block for every stream as ONE launch: in-projection, conv window update + SiLU,
 * softplus(dt), SSM state update and readout, gate + RMSNorm, out-projection (the per-bar update of
 * trading_bots/src/torch/model/stream/live.rs:228-244, called from trading_bots/src/torch/infer/offline.rs:124-125:
 * at a few streams the step's cost is the host's time to issue launches, so the chain of stage kernels and library
 * products is one kernel here).  dims->seqlen must be 1.  u [B,d_model], w_in [2*H*P+2*G*N+H, d_model] and w_out
 * [d_model, H*P] in the activation type (dtype 0: float32, 1: bfloat16), conv_w [C,d_conv], conv_b [C], dt_bias [H],
 * A [H], D [H] or NULL, norm_w [H*P] float32; conv_state [B,d_conv-1,C] (activation type) and ssm_state [B,H,P,N]
 * (float32) advance in place; out [B,d_model].  d_model and H*P must each be 128 or 256 and dstate a multiple of 16
 * (SSD_ERR_UNSUPPORTED otherwise: run the stages).  A workgroup per stream reads both weight matrices whole, so the
 * call is meant for small batches (up to a few dozen streams); large ones are faster through the stage kernels. */
int ssd_block_step_fwd(const ssd_block_dims *dims, int dtype, int64_t d_model, const void *u, const void *w_in,
                       const float *conv_w, const float *conv_b, const float *dt_bias, const float *A, const float *D,
                       const float *norm_w, float eps, const void *w_out, void *conv_state, float *ssm_state, void *out,
                       void *hip_stream);

/* ---- Backward pass of the block's two stages -------------------------------------------------------------------
 * With ssd_chunk_scan_bwd between them and two GEMMs per projection (the caller's BLAS), these make the block
 * trainable: the reference's historical benchmark case for it is mamba2_fwd_bwd_train
 * (benchmark_results/bench_20260112_070055.json:16-23), the update they would run in is
 * trading_bots/src/torch/train/update.rs:206-330.  dzxbcdt [B,L,zxbcdt_ld] is the gradient of zxbcdt, laid out like it:
 * ssd_block_post_bwd writes its z channels, ssd_block_pre_bwd its x | B | C | dt channels (padding columns are not
 * touched).  Parameter gradients are float32 and are summed in a fixed order (same bits on every run); the partial
 * sums live in a workspace of ssd_block_bwd_workspace_bytes, which the two calls of one backward pass may share. */
int ssd_block_bwd_workspace_bytes(const ssd_block_dims *dims, int dtype, size_t *out_bytes);

/* Gradients of ssd_block_post_fwd: dout [B,L,H*P] -> dy [B,L,H,P] (activation dtype), dz into dzxbcdt, dnorm_w [H*P].
 * y is the scan's output as the forward took it (dtype 2: float32 y with bf16 activations). */
int ssd_block_post_bwd(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                       float eps, const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, void *workspace,
                       size_t workspace_bytes, void *hip_stream);
/* The same, and with yn_out [B,L,H*P] (activation dtype; NULL allowed) also the forward's normalised rows, bit for bit
 * what ssd_block_post_fwd writes: a training forward can then run gate, norm and out-projection as one kernel
 * (ssd_block_post_proj_fwd, which never writes those rows) and the backward still has them for the out-projection's
 * weight gradient dout^T yn, which is the only thing that reads them.  No counterpart in the reference, whose
 * autograd keeps such tensors itself (trading_bots/src/torch/model/blocks/gqa.rs:172-178 is where its norm sits). */
int ssd_block_post_bwd_yn(const ssd_block_dims *dims, int dtype, const void *y, const void *zxbcdt, const float *norm_w,
                          float eps, const void *dout, void *dy, void *dzxbcdt, float *dnorm_w, void *yn_out,
                          void *workspace, size_t workspace_bytes, void *hip_stream);

/* Gradients of ssd_block_pre_reset_fwd: from dx [B,L,H,P], dB, dC [B,L,G,N], ddt [B,L,H] (what ssd_chunk_scan_bwd
 * returns) and, optionally, dconv_state_out [B,d_conv-1,C] (a gradient on the conv state the forward returned) to
 * the x | B | C | dt channels of dzxbcdt, dconv_w [C,d_conv], dconv_b [C], ddt_bias [H] and, when asked for,
 * dconv_state_in [B,d_conv-1,C].  conv_state_in and reset are the forward's (NULL allowed). */
int ssd_block_pre_bwd(const ssd_block_dims *dims, int dtype, const void *zxbcdt, const float *conv_w, const float *conv_b,
                      const float *dt_bias, const void *conv_state_in, const uint8_t *reset, const void *dx, const void *dB,
                      const void *dC, const void *ddt, const void *dconv_state_out, void *dzxbcdt, float *dconv_w,
                      float *dconv_b, float *ddt_bias, void *dconv_state_in, void *workspace, size_t workspace_bytes,
                      void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* SSD_HIP_H */
