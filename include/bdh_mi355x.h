/*
 * bdh_mi355x.h — C ABI of libbdh_mi355x.so: the BDH (Dragon Hatchling) cached-inference
 * hot path of mosure/burn_dragon, hand-written for AMD MI355X (gfx950, CDNA4).
 *
 * The reference has no FFI of its own: the path sits behind generic Rust functions over
 * burn::tensor::Tensor (src/lib.rs:8,31-38).  Each entry point below names the reference
 * function it replaces (paths relative to the reference tree); a Rust `-sys` crate or any
 * other FFI binds exactly these symbols.
 *
 * Conventions
 *   - All `const float*` / `void*` data arguments are caller-owned DEVICE pointers unless
 *     the parameter name ends in `_host`.  Tensors are row-major contiguous, last index
 *     fastest, in the reference's layouts.
 *   - Calls are asynchronous: work is enqueued on the context's HIP stream and the call
 *     returns; the caller synchronises the stream before reading results on the host.
 *   - Every function returns 0 (BDH_OK) or a negative bdh_status.  Nothing aborts or throws
 *     across this boundary (the reference panics on contract violations:
 *     src/model/bdh.rs:314-318, src/model/config.rs:143-153).  bdh_last_error() gives the
 *     text of the last failure on a context.
 *   - A context is not re-entrant; independent contexts may be used from different threads.
 *   - A context belongs to the device it was created on; the caller keeps that device current
 *     (hipSetDevice) on the calling thread for every call that takes the context or a model of it.
 *   - Entry points may grow the context's workspace (hipMalloc) the first time a shape is seen: run a
 *     step of each shape once before capturing calls in a HIP graph.
 *   - There is no CPU fallback: without a HIP device every compute entry point fails.
 *   - State (`rho`) and output (`out`) buffers are ordinary device memory (hipMalloc: coarse-grained).  Calls
 *     of many tokens add their products into them with the L2's no-return f32 adder (one add per element and call,
 *     so no ordering question); fine-grained or host-coherent allocations may not perform such an add and would
 *     lose updates silently.  Sums of that path below the smallest normal float are flushed to zero.
 *   - bdh_ctx_set_stream only swaps the stream: the context's workspace is shared by all of its calls, so the
 *     caller orders the old stream's queued work before the new stream's (an event), or uses one context per stream.
 */
#ifndef BDH_MI355X_H
#define BDH_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct bdh_ctx bdh_ctx;     /* opaque: device, stream, workspace */
typedef struct bdh_model bdh_model; /* opaque: weights view + per-model tables */

enum bdh_status {
  BDH_OK = 0,
  BDH_E_INVAL = -1,       /* null pointer / bad enum / bad scalar */
  BDH_E_SHAPE = -2,       /* dimension not supported (e.g. odd latent with RoPE) */
  BDH_E_ALIGN = -3,       /* pointer not aligned as required */
  BDH_E_HIP = -4,         /* a HIP runtime call failed */
  BDH_E_NOMEM = -5,       /* workspace allocation failed */
  BDH_E_UNSUPPORTED = -6  /* combination not implemented */
};

/* src/positional.rs:8-15 (RotaryEmbedding; Alibi is the reference's default) */
enum bdh_rotary { BDH_ROPE = 0, BDH_ALIBI = 1, BDH_POPE = 2 };

/* storage type of the recurrent state rho.  The reference keeps it in f32; bf16 storage
 * with f32 accumulation is an extension of this library. */
enum bdh_dtype { BDH_F32 = 0, BDH_BF16 = 1 };

/* ---- library / context ------------------------------------------------------------ */
const char *bdh_version(void);
const char *bdh_status_string(int status);

/* hip_stream: a hipStream_t (NULL = the default stream).  Replaces the Burn device handle
 * every reference call receives (`&B::Device`, e.g. src/model/bdh.rs:37). */
int bdh_ctx_create(int device_id, void *hip_stream, bdh_ctx **out);
int bdh_ctx_destroy(bdh_ctx *ctx);
int bdh_ctx_set_stream(bdh_ctx *ctx, void *hip_stream);
int bdh_ctx_synchronize(bdh_ctx *ctx);
const char *bdh_last_error(const bdh_ctx *ctx);
/* Launch-shape knobs for tests and tuning; no counterpart in the reference.
 *   "state_step.split": -1 (default) pick by grid size, 0 = 256 lane pairs per workgroup,
 *                       1 = 64 lane pairs per workgroup of 8 waves (small batches).
 *   "state_step.dense_chunks": -1 (default) a call of 128+ tokens without
 *                       bitmask / row-count outputs runs as dense products on the matrix cores
 *                       (with only a few (sequence, head) slices an f32 RoPE state keeps the token loop;
 *                       from 8 tokens on for an f32 state that every token streams in full -- PoPE,
 *                       eager ALiBi -- or that is at most 64 MiB),
 *                       0 = always token by token, 1 = dense products for any T.
 *   "state_step.prompt_bf16": 0 (default) never; T0 > 0: a call of T0 or more tokens on an f32 state, with the
 *                       position given by the host and no bitmask / row-count outputs, runs as
 *                       bdh_prefill_chunked_ex does: on the bf16 matrix cores, activations, values and scores
 *                       rounded to bf16, f32 accumulation and f32 state (any rotary; a lazily decayed ALiBi state
 *                       is brought up to date first and stamped with the end of the call).  Tolerance class
 *                       2e-2 instead of 1e-3, which is why it is opt-in; applies to bdh_recurrent_attention and
 *                       to the prompt calls of bdh_model_forward*.
 *   "state_step.dense_kernel": 1 (default) PoPE and eagerly decayed ALiBi steps at d in {256,512} take
 *                       the dense streaming kernel, 0 = the generic kernel (same values).
 *   "relu_lowrank.mfma_rows": 8 (default) calls with this many rows and at most 64 (N a multiple of 4, d a
 *                       multiple of 32, enough columns for a wavefront per CU) run on the f32 matrix cores, the
 *                       weights streamed once per 32 rows: a chain of v_mfma_f32_32x32x2_f32 over k is the same
 *                       k-sequential fused-multiply-add chain per output, bit for bit; 0 = never; a negative
 *                       value -r takes it from r rows on whatever the width.
 *   "relu_lowrank.gemm_rows": 64 (default) calls with this many tokens per sequence or more (and enough tiles to
 *                       cover the chip) run as one f32 matrix-core product per (sequence, head) with the k order
 *                       of a scalar loop: the same bits again; 0 = never; a negative value -r takes it from
 *                       r tokens on whatever the grid.
 *   "relu_lowrank.scalar": 1 (default) calls with 8 to 63 rows read their inputs through the scalar
 *                       cache, 0 = stage them in LDS (same values).
 *   "relu_lowrank.row": 1 (default) a call with one input row, 128 <= d <= 512 and at most 16 MiB of
 *                       weights takes the kernel that keeps every weight in flight at once, 0 = the
 *                       column-per-thread kernel (same values).
 *   "relu_lowrank.tile": 1 (default) calls with 64+ rows take the 64-row tile kernel (same values) when
 *                       its grid covers the chip, 2 = whenever the shape allows, 0 = never.
 *   "decoder.mfma":     1 (default) the encoder E of a call with 128+ tokens per sequence runs on
 *                       the f32 matrix cores, 0 = always the VALU kernel.
 *   "decoder.splitk_rows": 24 (default) a decode step (T = 1) of this many or more sequences runs the
 *                       encoder E as a split-K product on the f32 matrix cores (all of E is streamed
 *                       once) when its tiles cover half the chip; fewer sequences, and small models, take
 *                       the VALU kernel that skips inactive rows of E.  A negative value -r takes the
 *                       matrix-core form from r sequences on whatever the size.
 *   "model.one_launch": 1 (default) a decode step (T = 1, no x_tap / viz) of a model that is
 *                       small enough does not run kernel by kernel: a small model (d <= 256 and d % 4 == 0,
 *                       h * N <= 2048 and a multiple of 32, h in {1,2,4,8,16}, V <= 1024) can take ONE launch
 *                       for the whole step, a workgroup per sequence (always for up to 4 MiB of projection
 *                       weights per step, else only for large batches); a mid-size model (128 <= d <= 512,
 *                       N a multiple of 64, at most 64 blocks of 64 neurons) takes TWO launches per layer, a
 *                       workgroup per block, while batch x weights of a layer stay under 256 MiB.
 *                       2 = the one-launch step whenever the model fits it; 0 = kernel by kernel like any
 *                       other call (values agree to 1e-5: other summation trees).
 *   "model.fused_rows": 1 (default) a decode step of ONE sequence (B = 1, T = 1, no x_tap / viz) through a RoPE
 *                       model with n_embd in {256, 512} that is too large for the forms above takes four launches
 *                       per layer instead of six: D_y sums the state step's readout partials and applies their
 *                       LayerNorm itself, the next layer's D_x sums the encoder's partials and applies the two
 *                       LayerNorms and the residual (the first layer's D_x makes its row from the embedding), each
 *                       behind its first weight loads; taken while those sums stay small against the weights
 *                       (N * n_embd <= 2 Mi and n_head * N * n_embd <= 32 Ki * fused_kb: BASELINE config 1 is the
 *                       largest such shape).  0 = kernel by kernel (values agree to 1e-5).
 *   "model.fused_kb":   rows of E per workgroup of the encoder's first stage in that form (128 .. 2048, default 256).
 *   "model.phase_batch": the two-launch layer only for at most this many sequences (default: no limit
 *                       beyond the one above; 0 = never).
 *   "fused_state_aligned.path": -1 (default) pick by T, 0 = one workgroup per query row,
 *                       1 = the two products on the matrix cores (T >= 128 by default; operands as three
 *                       bf16 terms each, f32-level accuracy), 2 = dense-pattern row-normalised calls (N a multiple
 *                       of 8) as bdh_prefill_chunked_ex computes them: inputs and scores rounded to bf16 once, about
 *                       five times faster at the config-3 shape, tolerance class 2e-2 instead of 1e-3 (other calls
 *                       as -1); reaches Attention::forward and BDH::forward_fast through bdh_model_forward_fast*. */
int bdh_ctx_set_option(bdh_ctx *ctx, const char *name, int value);

/* ---- host-side tables (computed on the host in the reference as well) --------------- */
/* src/model/attention.rs:351-373  Attention::build_freqs -> freqs_host[latent] */
int bdh_build_freqs(int latent, float theta, int rotary, float *freqs_host);
/* src/kernel/linear_attention.rs:152-163  default_alibi_slopes -> slopes_host[n_head] */
int bdh_default_alibi_slopes(int n_head, float *slopes_host);

/* Attention::rotate / rotate_positions (src/model/attention.rs:177-179,332-349; rope :305-321, pope
 * :323-330) on its own: x [B,h,T,N] -> q [B,h,T,Nq] (Nq = 2N for BDH_POPE, else N; BDH_ALIBI copies),
 * token t at position + t, or positions_dev[b] + t (device int32 [B]) when given.  x and q must not
 * overlap unless equal for BDH_ALIBI.  The state step and the attention entry points below rotate
 * internally with the same arithmetic; this entry point serves callers that want the rotated values. */
int bdh_rotate(bdh_ctx *ctx, int B, int h, int T, int N, int rotary, const float *x, const float *freqs,
               int64_t position, const int32_t *positions_dev, float *q);

/* ---- a5 + a4: the recurrent state step ------------------------------------------- */
/*
 * Replaces BDH::recurrent_attention (src/model/bdh.rs:258-307) including the
 * rotate_positions call at :265 (src/model/attention.rs:332-349, rope :305-321,
 * pope :323-330).
 *
 *   x        [B,h,T,N]   un-rotated sparse activations (the `query` argument)
 *   v        [B,T,d]     value = the layer input `current` [B,1,T,d], shared by heads
 *   freqs    [N]         table from bdh_build_freqs (ignored for BDH_ALIBI)
 *   position             start position of token 0 (state.position, src/model/bdh.rs:334)
 *   positions_dev        optional DEVICE int32[B]: per-sequence start positions that
 *                        override `position` (NULL = one shared position as in the
 *                        reference, src/model/state.rs:14)
 *   alibi_slopes_host    host float[h], BDH_ALIBI only (NULL = default slopes); after every
 *                        token rho[:,h] is scaled by exp(-slope_h) (src/model/bdh.rs:299-301)
 *   rho      [B,h,Nq,d]  recurrent state, updated IN PLACE (the reference moves it out and
 *                        back, :274,:304, so the step owns it); Nq = N, or 2N for BDH_POPE.
 *                        The caller zero-fills it where the reference would create zeros
 *                        (:274-284).
 *   out      [B,h,T,d]   out_t = sum_n rho_before_t[n,:] * q_t[n]   (readout BEFORE update)
 *   active_bitmask       optional uint64 [B,h,T,ceil(N/64)]: bit n%64 of word n/64 is set
 *                        iff x[b,h,t,n] != 0 (== x > 0 for ReLU outputs)
 *   rows_touched         optional int32 [B,h,T]: number of state rows read and written for
 *                        that token (RoPE: both rows of every lane pair with a non-zero
 *                        element; ALiBi/PoPE: Nq)
 *
 * RoPE requires even N (src/model/attention.rs:310).  T = 1 is the decode step.  A call of 128 or more
 * tokens that asks for neither bitmask nor row counts computes the same sums as dense
 * products (out = tril(-1)(Q Q^T) V + Q rho, rho += Q^T V, chunks of up to 512 tokens; for ALiBi with
 * the decay powers decay^(t-s), decay^t and decay^(T-s) applied to the three terms) on the matrix
 * cores (a bf16 state is widened to f32 for the call and rounded once at its end).  Large products
 * take every f32 operand as a sum of three bf16 terms, six bf16 matrix instructions per f32 one: what
 * is left out is below 2^-23 of a product, so results agree with the token loop to f32 reassociation
 * (option "state_step.dense_chunks").  Inputs are assumed finite.
 */
int bdh_recurrent_attention(bdh_ctx *ctx, int B, int h, int T, int N, int d, int rotary,
                            const float *x, const float *v, const float *freqs,
                            int64_t position, const int32_t *positions_dev,
                            const float *alibi_slopes_host, void *rho, int rho_dtype,
                            float *out, uint64_t *active_bitmask, int32_t *rows_touched);

/* The decode step: bdh_recurrent_attention with T = 1 (x [B,h,N], v [B,d], out [B,h,d]). */
int bdh_state_step(bdh_ctx *ctx, int B, int h, int N, int d, int rotary, const float *x,
                   const float *v, const float *freqs, int64_t position,
                   const int32_t *positions_dev, const float *alibi_slopes_host, void *rho,
                   int rho_dtype, float *out, uint64_t *active_bitmask,
                   int32_t *rows_touched);

/* bdh_state_step for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments,
 * same kernels and bit-identical results, but the readout partials [B*h, S, d] and the per-workgroup
 * row counts go to a fixed 32.25 MiB array in device memory that the library holds on every device it
 * runs on (resolved at bdh_ctx_create) instead of the context's growable workspace, and the call makes
 * no hipMalloc / hipFree.  A shape whose partials do not fit returns BDH_E_SHAPE and bdh_last_error
 * names the bytes needed: about 4*B*h*S*(d+1) with S workgroups per (sequence, head) slice (S = N/512
 * for RoPE at d in {256,512}, N/128 when that grid would leave CUs idle, N/64 for the other kernels).
 * BASELINE configs 2 and 4 need 2 and 16 MiB.  All calls on one device share the array: calls that overlap on one device (two streams, two
 * contexts) race; calls ordered on one stream do not.  Nothing in the array has to start at zero: every
 * element that is read was written by the same call.  The array's address is kept for device ids 0..63; a context
 * on a device beyond that returns BDH_E_UNSUPPORTED here. */
int bdh_state_step_noalloc(bdh_ctx *ctx, int B, int h, int N, int d, int rotary, const float *x,
                           const float *v, const float *freqs, int64_t position,
                           const int32_t *positions_dev, const float *alibi_slopes_host, void *rho,
                           int rho_dtype, float *out, uint64_t *active_bitmask,
                           int32_t *rows_touched);

/* ---- the decode step with deferred state updates ---------------------------------- */
/*
 * BDH::recurrent_attention at T = 1 (src/model/bdh.rs:258-307 with the rotation of :265; RoPE only) like
 * bdh_state_step, but the rank-1 update of :298 is LOGGED instead of written: a step reads its active state
 * rows once and writes none of them.  What differs from the reference's step:
 *   - readout: out_t = sum_n rho_base[n,:] q_t[n] + sum_s (q_t . q_s) v_s over the logged steps s, the sums of
 *     src/model/bdh.rs:293-295 reassociated (agrees with bdh_state_step to f32 rounding, ~1e-6 relative);
 *   - state: `rho` lags behind by the logged steps until a flush applies them.  bdh_state_flush (and every
 *     capacity-th call of bdh_state_step_deferred by itself, before it logs) walks the state rows the logged
 *     steps touched and applies their updates in step order, row + (q_s[n] * v_s) with the product rounded
 *     before the add: afterwards rho holds, bit for bit, what the same calls of bdh_state_step would have left
 *     (a bf16 state is rounded after every logged step, as the eager step stores it).
 * The caller flushes before anything else reads or writes rho (another entry point, an export, a copy), the way
 * bdh_alibi_materialize precedes such uses of a lazily decayed state.  A log serves ONE state tensor at a time:
 * while steps are pending, a call with another rho pointer fails with BDH_E_INVAL.
 *   bdh_state_log_create  B, h, N, d, rho_dtype as in bdh_state_step (d in {256, 512}, even N); capacity =
 *                         steps the log holds, 1..128 with capacity * d <= 32768 (the flush keeps the logged
 *                         value rows in LDS).  Device memory of the log: about B*h*(N/512)*(capacity*2 + 4.5) KiB
 *                         (config 2 at capacity 128: 521 MiB).  The larger the capacity, the less often the
 *                         state is rewritten: at config 2 a flush rewrites nearly every row from 32 steps on.
 *   bdh_state_log_pending steps logged and not yet applied.
 *   bdh_state_step_deferred  x [B,h,N], v [B,d], freqs [N], position / positions_dev, out [B,h,d],
 *                         active_bitmask and rows_touched exactly as bdh_state_step (rows_touched counts the
 *                         rows of the active pairs, which this call only reads).
 * The number of pending steps is host-side state of the log, so one step is not a fixed launch sequence: a HIP
 * graph can hold `capacity` steps followed by a flush, not a single step.
 */
typedef struct bdh_state_log bdh_state_log; /* opaque: pending rank-1 updates of one state tensor */
int bdh_state_log_create(bdh_ctx *ctx, int B, int h, int N, int d, int rho_dtype, int capacity,
                         bdh_state_log **out);
int bdh_state_log_destroy(bdh_ctx *ctx, bdh_state_log *log);
int bdh_state_log_pending(const bdh_state_log *log);
size_t bdh_state_log_bytes(const bdh_state_log *log);
int bdh_state_step_deferred(bdh_ctx *ctx, bdh_state_log *log, const float *x, const float *v,
                            const float *freqs, int64_t position, const int32_t *positions_dev, void *rho,
                            float *out, uint64_t *active_bitmask, int32_t *rows_touched);
int bdh_state_flush(bdh_ctx *ctx, bdh_state_log *log, void *rho);

/* ---- a3 / a7: ReLU low-rank projection ------------------------------------------- */
/*
 * Replaces kernel::relu_lowrank::fused_forward (src/kernel/relu_lowrank.rs:7-37) and the
 * unfused sequence at src/model/bdh.rs:346-350 and :370-374.
 *
 *   in      [B,h_in,T,d]  h_in = 1 (shared by heads, the D_x call) or h (the D_y call)
 *   weight  [h,d,N]
 *   bias    [h,N] or NULL                       (relu_lowrank.rs:19-23)
 *   threshold                                   (relu_lowrank.rs:25-27)
 *   block_size, active_blocks_host[n_blocks]    BlockPattern1d (src/kernel/block_sparse.rs:
 *                        11-63): one byte per latent block, NULL = dense pattern
 *   gate    [B,h,T,N] or NULL: when given, out = gate * relu(...) (the x (.) y product of
 *                        src/model/bdh.rs:380 fused into the D_y projection)
 *   out     [B,h,T,N] = relu(in . weight + bias - threshold) * mask
 *
 * Each output element is one k-sequential f32 fused-multiply-add chain, so the set
 * {n : out > 0} does not depend on the launch shape.
 */
int bdh_relu_lowrank(bdh_ctx *ctx, int B, int h_in, int T, int d, int h, int N,
                     const float *in, const float *weight, const float *bias, float threshold,
                     int block_size, const uint8_t *active_blocks_host, int n_blocks,
                     const float *gate, float *out);

/* BDH::layer_norm (src/model/bdh.rs:86-89): biased variance, eps 1e-5, no affine.
 * in/out [rows,d]; in == out is allowed. */
int bdh_layer_norm(bdh_ctx *ctx, int64_t rows, int d, const float *in, float *out);

/* ---- a10: parallel (training-path) causal linear attention ------------------------- */
/*
 * Replaces kernel::linear_attention::fused_state_aligned (src/kernel/linear_attention.rs:
 * 11-115) and, with the dense pattern, Attention::forward (src/model/attention.rs:142-175).
 *   query [B,h,T,N] un-rotated, value [B,T,dv] (dim 1 of size 1 repeated over heads),
 *   freqs [N], alibi_slopes_host [h] or NULL, time-block size and optional sparse
 *   (row,col) block pairs (BlockPattern2d, src/kernel/block_sparse.rs:66-117),
 *   positions 0..T.  out [B,h,T,dv] = (sum of masked score blocks . V) / (sum|score| + 1e-6).
 *   row_normalize = 0 drops the division and gives the un-normalised causal form that
 *   equals the recurrent path.
 */
int bdh_fused_state_aligned(bdh_ctx *ctx, int B, int h, int T, int N, int dv,
                            const float *query, const float *value, const float *freqs,
                            const float *alibi_slopes_host, int block_size,
                            const int32_t *block_pairs_host, int n_pairs, int rotary,
                            int row_normalize, float *out);

/* ---- chunked prefill (dense MFMA form of the recurrent path) ------------------------ */
/*
 * The recurrent path of src/model/bdh.rs:258-307 for T tokens at once, RoPE only, computed on
 * the bf16 matrix cores with f32 accumulation:
 *   out = tril(-1)(Q Q^T) V + Q rho0 ;  rho = rho0 + Q^T V ,  Q = bf16(rope(x))
 * The reference has no such function (its prefill walks tokens serially, src/generation.rs:
 * 74-104, src/model/bdh.rs:288); the sequential loop is the definition of the result.
 *   x   [B,h,T,N] bf16 (raw 16-bit patterns) un-rotated activations
 *   v   [B,T,d]   bf16, shared by the heads of a batch entry
 *   position      start position of token 0
 *   chunk         tokens per internal pass (0 = 2048).  The call walks the T tokens in passes of this
 *                 many; the workspace holds one pass (rotated activations [B*h, chunk, N] in bf16 and, for
 *                 shapes that take the chunk-recurrent form, one bf16 copy of the state per 256 tokens of
 *                 the pass), so it is linear in chunk and independent of T.  Between passes the state is
 *                 carried in the caller's f32 rho, never rounded.  The chunk-recurrent form (d = 256, N a
 *                 multiple of 256, passes of 256+ tokens) wants a multiple of 256; a remainder of fewer
 *                 than 256 tokens takes the all-scores form.
 *   flags         BDH_PREFILL_STATE_IS_ZERO: the caller promises rho holds zeros (a fresh state,
 *                 src/model/state.rs:27-45): the Q rho0 product is skipped and rho is overwritten.
 *                 BDH_PREFILL_STATE_HILO: the state carried INTO the call enters the Q rho0 product as
 *                 bf16(rho0) + bf16(rho0 - bf16(rho0)) (two products; chunk-recurrent form only), i.e. with 16
 *                 mantissa bits instead of 8.  Inside a call the state between 256-token chunks enters its
 *                 product rounded to bf16 once, like the scores and the activations do; the f32 state
 *                 itself accumulates without rounding either way.
 *                 BDH_PREFILL_ALL_SCORES: always the all-scores form (every causal 256x256 score tile of
 *                 the pass, no state copies).
 *   rho [B,h,N,d] f32 in/out,  out [B,h,T,d] f32
 * N and d must be multiples of 8.  ALiBi, PoPE and the row-normalised form: bdh_prefill_chunked_ex below.
 */
enum bdh_prefill_flags {
  BDH_PREFILL_STATE_IS_ZERO = 1,
  BDH_PREFILL_STATE_HILO = 2,
  BDH_PREFILL_ALL_SCORES = 4,
  BDH_PREFILL_ROW_NORMALIZE = 8 /* bdh_prefill_chunked_ex only */
};
int bdh_prefill_chunked(bdh_ctx *ctx, int B, int h, int T, int N, int d, const uint16_t *x_bf16,
                        const uint16_t *v_bf16, const float *freqs, int64_t position, int chunk,
                        int flags, float *rho, float *out);

/*
 * bdh_prefill_chunked for all three positional schemes, and the bf16 matrix-core form of the row-normalised
 * attention.  Same arguments, plus:
 *   rotary             BDH_ROPE: exactly bdh_prefill_chunked.
 *                      BDH_POPE: Q = bf16(cat(softplus(x) cos, softplus(x) sin)) (src/model/attention.rs:323-330),
 *                      rho [B,h,2N,d].
 *                      BDH_ALIBI: Q = x, and the state decays by g_h = exp(-slope_h) after every token
 *                      (src/model/bdh.rs:299-301):  out_t = g^t q_t rho0 + sum_{s<t} g^(t-s) (q_t . q_s) v_s,
 *                      rho = g^T rho0 + sum_s g^(T-s) q_s (x) v_s, the powers as exp(k * log(g_f32)) like the lazily
 *                      decayed step.  alibi_slopes_host: host float[h], NULL = the default slopes.  rho is an
 *                      eagerly decayed f32 state (bdh_alibi_materialize first for a lazily decayed one).
 *                      PoPE and ALiBi take the all-scores form (every causal 256x256 score tile of a pass).
 *   flags              | BDH_PREFILL_ROW_NORMALIZE: the stateless function of
 *                      kernel::linear_attention::fused_state_aligned (src/kernel/linear_attention.rs:11-115) with the
 *                      dense causal layout, as bdh_fused_state_aligned computes it in f32:
 *                        out = (S' V) / (sum_s |S'[t,s]| + 1e-6),  S' = tril(-1)(Q Q^T) [+ slope_h (s - t)]
 *                      rho is neither read nor written (may be NULL), the whole call is one pass (chunk is ignored;
 *                      the bf16 score matrix [B*h,T,T] lives in the workspace), positions start at `position`
 *                      (the reference: 0).  The additive term is applied when alibi_slopes_host is given, whatever
 *                      the rotary mode, on every element of the causal time blocks of block_size tokens -- the
 *                      diagonal block included, where it reaches the elements above the diagonal (:97-100).
 *                      The normaliser sums the bf16-rounded scores, the values the product multiplies with.
 *   block_size         tokens per time block (BDH_PREFILL_ROW_NORMALIZE with slopes only; <= 0 means 1).
 * Tolerance class of the bf16 forms: 2e-2 of the output scale.  At most 64 heads when slopes are in use.
 */
int bdh_prefill_chunked_ex(bdh_ctx *ctx, int B, int h, int T, int N, int d, int rotary, const uint16_t *x_bf16,
                           const uint16_t *v_bf16, const float *freqs, const float *alibi_slopes_host,
                           int64_t position, int chunk, int flags, int block_size, float *rho, float *out);

/* ---- a1: the whole cached step ------------------------------------------------------- */
/* src/model/config.rs:113-164 (BDHConfig) + :10-31 (FusedKernelConfig), as plain scalars */
typedef struct bdh_model_config {
  int32_t n_layer;
  int32_t n_embd;   /* d */
  int32_t n_head;   /* h */
  int32_t latent;   /* N per head = mlp_internal_dim_multiplier * n_embd / n_head */
  int32_t vocab;    /* V */
  int32_t rotary;   /* enum bdh_rotary */
  float rope_theta;      /* 65536 */
  float relu_threshold;  /* 0 */
  const float *alibi_slopes_host; /* [h] or NULL */
} bdh_model_config;

/* device pointers, in the record order of the reference module (src/model/bdh.rs:27-33) */
typedef struct bdh_model_weights {
  const float *embed;     /* [V,d] */
  const float *encoder;   /* [h,d,N]   D_x */
  const float *encoder_v; /* [h,d,N]   D_y */
  const float *decoder;   /* [h*N,d]   E   */
  const float *lm_head;   /* [d,V] */
} bdh_model_weights;

/* Replaces BDH::new as far as inference needs it (src/model/bdh.rs:37-84): records the
 * weight pointers (not copied; they must outlive the model) and builds the freqs table
 * (Attention::new, src/model/attention.rs:113-140). */
int bdh_model_create(bdh_ctx *ctx, const bdh_model_config *config,
                     const bdh_model_weights *weights, bdh_model **out);
int bdh_model_destroy(bdh_model *model);

/* bytes of recurrent state for one sequence batch: L * B * h * Nq * d * sizeof(rho_dtype)
 * (ModelState, src/model/state.rs:5-15; one rho per layer) */
size_t bdh_model_state_bytes(const bdh_model *model, int B, int rho_dtype);

/*
 * Replaces BDH::forward_with_state (src/model/bdh.rs:309-450).
 *   tokens   [B,T] int64 device
 *   rho      [L,B,h,Nq,d] in place; zero-filled by the caller for a fresh state
 *   position state.position before the call; the caller advances it by T afterwards
 *            (src/model/bdh.rs:445)
 *   logits   [B,T,V]
 *   next_tokens  optional int64 [B] device: argmax of the last position's logits (greedy
 *            decoding, the top_k = 1 case of src/generation.rs:26-72, kept on the device)
 *   x_tap    optional [L,B,h,T,N]: the sparse activations x of every layer
 */
int bdh_model_forward(bdh_model *model, const int64_t *tokens, int B, int T, void *rho,
                      int rho_dtype, int64_t position, float *logits, int64_t *next_tokens,
                      float *x_tap);

/*
 * bdh_model_forward with per-sequence start positions kept in DEVICE memory (int32 [B]); when
 * positions_dev is not NULL it overrides `position`.  Together with next_tokens feeding the next
 * call's tokens this makes one decode step a fixed sequence of launches with no host-side
 * arguments that change from token to token, so a caller can capture it in a HIP graph and replay
 * it.  (The reference keeps one host-side position, src/model/state.rs:14, and round-trips the
 * token through the host, src/generation.rs:114-124.)
 */
int bdh_model_forward_ex(bdh_model *model, const int64_t *tokens, int B, int T, void *rho,
                         int rho_dtype, int64_t position, const int32_t *positions_dev,
                         float *logits, int64_t *next_tokens, float *x_tap);

/* Replaces BDH::forward_fast (src/model/bdh.rs:96-168), the stateless forward over all tokens at once
 * that the reference trains with: the same layer as bdh_model_forward, but the attention is
 * Attention::forward (row-normalised causal scores from position 0, bdh_fused_state_aligned) instead of
 * the recurrent state.  time_block_size > 0 selects the fused branch with dense time blocks of that
 * size (FusedKernelConfig.enabled; the latent block pattern is dense, as build_model_config makes it);
 * <= 0 the plain branch.  tokens [B,T] int64 -> logits [B,T,V].  Inference only: no gradients. */
int bdh_model_forward_fast(bdh_model *model, const int64_t *tokens, int B, int T, int time_block_size,
                           float *logits);

/* bdh_model_forward_fast with the block patterns of FusedKernelConfig.block_sparse (src/model/bdh.rs:111,
 * 114-129, 134-151 and src/model/attention.rs:142-152): the time-block pairs go to the attention of every
 * layer as in bdh_fused_state_aligned (block_pairs_host [n_time_pairs][2] of (row, col), NULL = dense lower
 * triangle; needs time_block_size > 0), the latent block mask to both projections of every layer as in
 * bdh_relu_lowrank (one byte per block of latent_block_size neurons, NULL = dense). */
int bdh_model_forward_fast_ex(bdh_model *model, const int64_t *tokens, int B, int T, int time_block_size,
                              const int32_t *time_pairs_host, int n_time_pairs, int latent_block_size,
                              const uint8_t *latent_blocks_host, int n_latent_blocks, float *logits);

/* positions_dev[b] = saturating(positions_dev[b] + delta): the device-side form of
 * `state.position += T` (src/model/bdh.rs:445). */
int bdh_advance_positions(bdh_ctx *ctx, int32_t *positions_dev, int B, int delta);

/* ALiBi state kept LAZILY decayed.  The reference multiplies the whole state by exp(-slope_h) after
 * every token (src/model/bdh.rs:299-301), which makes every ALiBi step a dense pass over rho.  Here row n
 * of a slice stores the value it had when the sequence had absorbed stamps[b,h,n] tokens; its current
 * value is that times decay_h^(clock - stamp).  A step reads, brings up to date, updates, decays once
 * and re-stamps only the rows whose activation is non-zero, so its traffic follows the sparsity of x.
 * `clock` (or clocks_dev[b], int32 per sequence) = tokens the state has absorbed before this call =
 * ModelState::position.  A zero state with zero stamps is a valid fresh state.  Semantics otherwise as
 * bdh_recurrent_attention with rotary = BDH_ALIBI (q = x, no rotation); rows_touched counts the active
 * rows.  Values agree with the eager decay to rounding (decay^k is evaluated as exp(k*log(decay))). */
int bdh_recurrent_attention_lazy_alibi(bdh_ctx *ctx, int B, int h, int T, int N, int d, const float *x,
                                       const float *v, int64_t clock, const int32_t *clocks_dev,
                                       const float *alibi_slopes_host, void *rho, int rho_dtype,
                                       int32_t *stamps, float *out, uint64_t *active_bitmask,
                                       int32_t *rows_touched);

/* Brings a lazily decayed state up to date: every row *= decay_h^(clock - stamp), stamps = clock.
 * Afterwards rho [B,h,N,d] is the state the reference holds after `clock` tokens and can be handed to
 * the eager entry points (or exported). */
int bdh_alibi_materialize(bdh_ctx *ctx, int B, int h, int N, int d, int64_t clock,
                          const int32_t *clocks_dev, const float *alibi_slopes_host, void *rho,
                          int rho_dtype, int32_t *stamps);

/* bdh_model_forward_ex for an ALiBi model whose state is kept lazily decayed: stamps [L,B,h,N] int32
 * travels with rho (NULL = eager decay, identical to bdh_model_forward_ex). */
int bdh_model_forward_lazy(bdh_model *model, const int64_t *tokens, int B, int T, void *rho,
                           int rho_dtype, int32_t *stamps, int64_t position,
                           const int32_t *positions_dev, float *logits, int64_t *next_tokens,
                           float *x_tap);

/* bdh_model_forward_lazy with the state given layer by layer, the way the reference holds it: ModelState is a
 * Vec<LayerState> of independent Option<Tensor<B,4>> (src/model/state.rs:5-15), each taken out and put back by its
 * layer (src/model/bdh.rs:274,304).  rho_layers_host: HOST array of n_layer DEVICE pointers, layer l's state
 * [B,h,Nq,d]; stamps_layers_host: the same for the decay stamps [B,h,N] of a lazily decayed ALiBi state, or NULL.
 * Results are those of the one-allocation entry points bit for bit.  (Layers that happen to lie adjacent in memory
 * also take the fused decode forms of option "model.one_launch"; separate allocations run kernel by kernel.) */
int bdh_model_forward_layers(bdh_model *model, const int64_t *tokens, int B, int T, void *const *rho_layers_host,
                             int rho_dtype, int32_t *const *stamps_layers_host, int64_t position,
                             const int32_t *positions_dev, float *logits, int64_t *next_tokens, float *x_tap);

/* The energy map of a state: out[h,N] = (sum over b of (sum over c of |rho[b,h,n,c]|) / d) / B, the
 * `rho_last` of LayerVizState (src/model/bdh.rs:411-419, built under the reference's "viz" feature).
 * rho [B,h,N,d] f32 or bf16.  stamps [B,h,N] (optional, ALiBi only) marks a lazily decayed state, read
 * at `clock` (or clocks_dev[b], device int32 [B]) through its pending decay; alibi_slopes_host [h] as in
 * bdh_recurrent_attention (NULL = default slopes), ignored without stamps. */
int bdh_rho_energy(bdh_ctx *ctx, int B, int h, int N, int d, const void *rho, int rho_dtype,
                   const int32_t *stamps, int64_t clock, const int32_t *clocks_dev,
                   const float *alibi_slopes_host, float *out);

/* bdh_model_forward_lazy that also fills the per-layer LayerVizState of the reference
 * (src/model/state.rs:17-24, src/model/bdh.rs:386-434): viz [L,4,h,N] f32 receives, for every layer,
 * x_last, y_last, xy_last (first sequence, last token of this call) and rho_last (bdh_rho_energy of the
 * layer's updated state; all zeros for PoPE, whose state has 2N rows).  viz = NULL is exactly
 * bdh_model_forward_lazy.  Costs one extra D_y pass over h rows and one dense read of the state per
 * layer, so it is meant for the visualisation loop, not for throughput runs. */
int bdh_model_forward_viz(bdh_model *model, const int64_t *tokens, int B, int T, void *rho,
                          int rho_dtype, int32_t *stamps, int64_t position,
                          const int32_t *positions_dev, float *logits, int64_t *next_tokens,
                          float *x_tap, float *viz);

/* A decode step (T = 1) of bdh_model_forward_ex with the state updates of every layer deferred
 * (bdh_state_step_deferred in place of the step of src/model/bdh.rs:288-302): RoPE models with n_embd in {256, 512}.
 * `logs` holds one update log per layer for a batch of B sequences (capacity as in bdh_state_log_create; every
 * layer logs one step per call, so all layers fill and flush together, the call that finds the logs full flushing
 * them first).  Until bdh_model_flush, rho [L,B,h,N,d] lags behind by the pending steps; flush before any other
 * entry point (a prompt call, bdh_model_forward*, bdh_rho_energy, an export) touches rho.  Logits agree with
 * bdh_model_forward_ex to f32 rounding of the reassociated readout, and so does the flushed state: a layer applies
 * its logged updates bit for bit as the eager step would (the first layer's state is bit-identical), but the
 * readouts that feed the deeper layers differ by that rounding, and their updates with them. */
typedef struct bdh_model_logs bdh_model_logs; /* opaque: one bdh_state_log per layer */
int bdh_model_logs_create(bdh_model *model, int B, int rho_dtype, int capacity, bdh_model_logs **out);
int bdh_model_logs_destroy(bdh_model *model, bdh_model_logs *logs);
int bdh_model_logs_pending(const bdh_model_logs *logs);
int bdh_model_forward_deferred(bdh_model *model, bdh_model_logs *logs, const int64_t *tokens, int B, void *rho,
                               int rho_dtype, int64_t position, const int32_t *positions_dev, float *logits,
                               int64_t *next_tokens);
int bdh_model_flush(bdh_model *model, bdh_model_logs *logs, void *rho);
/* The same two calls with the state given layer by layer (rho_layers_host: HOST array of n_layer DEVICE pointers, layer
 * l's state [B,h,N,d]), as bdh_model_forward_layers takes it: the reference's ModelState of independent per-layer
 * tensors (src/model/state.rs:5-15) decodes with deferred updates without a copy.  A layer's log stays bound to the
 * pointer it first saw until it is flushed. */
int bdh_model_forward_deferred_layers(bdh_model *model, bdh_model_logs *logs, const int64_t *tokens, int B,
                                      void *const *rho_layers_host, int rho_dtype, int64_t position,
                                      const int32_t *positions_dev, float *logits, int64_t *next_tokens);
int bdh_model_flush_layers(bdh_model *model, bdh_model_logs *logs, void *const *rho_layers_host);

/* Draws the next token of every sequence on the device.  Replaces the temperature division of
 * sample_next_token (src/generation.rs:117) and sample_from_logits_values (src/generation.rs:26-72),
 * which copy the logits to the host for every token: values = logits / temperature; with
 * 0 < top_k < V everything below the k-th largest value is masked to -inf (ties with it survive);
 * softmax (uniform over V when the sum is 0 or NaN); the index is drawn as rand's WeightedIndex
 * draws it, from the running sums in index order, with uniforms[b] in [0,1) standing for the
 * variate the reference takes from thread_rng.  top_k <= 0 means no truncation (`None`).
 * logits: row b starts at logits + b*row_stride (pass the last-token row of [B,T,V] logits with
 * row_stride = T*V).  V <= 8192.  next_tokens [B] int64 can be fed back as the next call's tokens. */
int bdh_sample_top_k(bdh_ctx *ctx, int B, int V, const float *logits, int64_t row_stride,
                     float temperature, int top_k, const float *uniforms, int64_t *next_tokens);

/* Measurement aid, no counterpart in the reference: the memory traffic of the decode state step without
 * its arithmetic.  Reads, scales by 1 and writes back in place (mode 0), only reads (1) or only writes
 * zeros (2) the listed chunks of `region`: chunk c covers bytes [chunk_index[c] * chunk_kib KiB, + chunk_kib
 * KiB); one wavefront moves 1 KiB at a time, `workgroups` workgroups of 256 threads stride over the list.
 * Listed chunks that do not lie inside region_bytes are skipped.  bench.py --workload rmw_probe times it on the
 * config-2 pattern (random 2 KiB chunks, 9.75 % of 1 GiB) to report the bandwidth that pattern can reach. */
int bdh_probe_chunks(bdh_ctx *ctx, void *region, size_t region_bytes, const int32_t *chunk_index, int n_chunks,
                     int chunk_kib, int mode, int workgroups);

#ifdef __cplusplus
}
#endif
#endif /* BDH_MI355X_H */
