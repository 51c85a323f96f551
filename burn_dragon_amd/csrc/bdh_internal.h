// Internal declarations shared by the translation units of libbdh_mi355x.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../include/bdh_mi355x.h"

struct bdh_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  // growable device workspace (partials, counters); owned by the context
  void *ws = nullptr;
  size_t ws_bytes = 0;
  // a second growable buffer for inputs a launcher converts before it calls a path that sizes ctx->ws itself
  void *stage = nullptr;
  size_t stage_bytes = 0;
  int n_cu = 0;
  int opt_step_split = -1;  // -1 choose by grid size, 0 / 1 force the 256- / 64-pair workgroup
  int opt_step_dense = -1;  // many-token state step as dense f32 products: -1 from T = 128, 0 never, 1 always
  int opt_lowrank_tile = 1;  // 0: relu_lowrank never takes the 64-row tile kernel
  int opt_decoder_mfma = 1;  // 0: the encoder E never takes the f32 matrix-core form
  int opt_model_one_launch = 1;  // small model's decode step in one launch: 1 when it pays, 2 whenever it fits, 0 never
  int opt_lowrank_row = 1;     // 0: relu_lowrank with one input row and a small matrix uses the column-per-thread kernel
  int opt_model_phase_batch = 1 << 30;  // two launches per layer for a decode step of at most this many sequences (0: never)
  int opt_lowrank_gemm_rows = 64;  // relu_lowrank with this many tokens per sequence or more runs as a matrix-core product (0: never)
  int opt_lowrank_mfma_rows = 8;  // relu_lowrank takes the f32 matrix cores from this many rows on (0: never)
  int opt_lowrank_scalar = 1;  // 0: relu_lowrank with 8 to 63 rows stages its inputs in LDS instead of scalar loads
  int opt_step_dense_kernel = 1;  // 0: PoPE / eager ALiBi at d in {256,512} take the generic kernel
  int opt_decoder_splitk_rows = 24;  // decode-step encoder on the matrix cores from this many sequences on
  int opt_fsa_path = -1;    // fused_state_aligned: -1 choose by T, 0 row kernel, 1 f32 matrix cores
  int opt_model_fused_rows = 1;  // 0: a one-sequence decode step never folds its reductions into the projections
  int opt_model_fused_kb = 256;  // rows of E per workgroup of the encoder's first stage in that form
  int opt_step_prompt_bf16 = 0;  // many-token state step on the bf16 matrix cores from this many tokens on (0: never)
  // time-block mask of the last sparse fused_state_aligned pattern (device) and the pattern it was built from
  void *fsa_mask = nullptr;
  size_t fsa_mask_bytes = 0;
  std::vector<int> fsa_mask_key;
  // latent block mask of the last relu_lowrank call that had one (device) and the bytes it was built from
  void *lat_mask = nullptr;
  size_t lat_mask_bytes = 0;
  std::vector<uint8_t> lat_mask_key;
  char err[512] = {0};
};

struct bdh_model {
  bdh_ctx *ctx = nullptr;
  bdh_model_config cfg{};
  bdh_model_weights w{};
  float *freqs = nullptr;   // device [N]
  float slopes[64] = {0};   // host, ALiBi only
  // activation scratch, grown on demand to the largest (B,T) seen
  void *act = nullptr;
  size_t act_bytes = 0;
};

int bdh_fail(bdh_ctx *ctx, int status, const char *fmt, ...);

// model_phase.hip: a decode step in two launches per layer (T = 1, f32 state, 128 <= d <= 512, N a multiple of 64)
bool bdh_model_phase_fits(const bdh_model_config &c);
size_t bdh_model_phase_scratch_floats(const bdh_model_config &c, int B);
int bdh_launch_model_phases(bdh_model *m, const int64_t *tokens, int B, float *scratch, void *rho, int rho_dtype, int32_t *stamps,
                            int64_t position,
                            const int32_t *positions_dev, float **cur_final, float **dec_partial, int *G_out);
int bdh_launch_phase_head(bdh_model *m, int B, const float *cur, const float *dec_partial, int G, float *logits,
                          int64_t *next_tokens);
// projections.hip: cur[m,:] = LN(cur[m,:] + LN(sum_kb partial[kb][m][:]))
int bdh_launch_decoder_finalize(bdh_ctx *ctx, const float *partial, int KBN, int M, int d, float *cur);

// model_small.hip: the one-launch decode step of a small model (T = 1, f32 state)
bool bdh_model_small_fits(const bdh_model_config &c);
int bdh_launch_model_small(bdh_model *m, const int64_t *tokens, int B, void *rho, int rho_dtype, int32_t *stamps, int64_t position,
                           const int32_t *positions_dev, float *logits, int64_t *next_tokens);

// Grows ctx->ws to at least `bytes` (synchronises the stream before freeing the old one).
int bdh_ws_reserve(bdh_ctx *ctx, size_t bytes);
// The same for ctx->stage.
int bdh_stage_reserve(bdh_ctx *ctx, size_t bytes);

#define BDH_HIP_CHECK(ctx, call)                                                        \
  do {                                                                                  \
    hipError_t e_ = (call);                                                             \
    if (e_ != hipSuccess)                                                               \
      return bdh_fail((ctx), BDH_E_HIP, "%s failed: %s (%s:%d)", #call,                 \
                      hipGetErrorString(e_), __FILE__, __LINE__);                       \
  } while (0)

#define BDH_LAUNCH_CHECK(ctx, what)                                                     \
  do {                                                                                  \
    hipError_t e_ = hipGetLastError();                                                  \
    if (e_ != hipSuccess)                                                               \
      return bdh_fail((ctx), BDH_E_HIP, "launch of %s failed: %s", (what),              \
                      hipGetErrorString(e_));                                           \
  } while (0)

static inline size_t bdh_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline bool bdh_aligned(const void *p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

// ---- launchers implemented in the kernel translation units --------------------------
struct StateStepParams {
  int B, h, T, N, d, rotary, rho_dtype;
  const float *x, *v, *freqs;
  int64_t position;
  const int32_t *positions_dev;
  const float *slopes_host;  // resolved (never null for ALiBi)
  void *rho;
  float *out;
  uint64_t *bitmask;
  int32_t *rows_touched;
  int32_t *stamps = nullptr;  // ALiBi only: [B,h,N] decay stamps of a lazily decayed state, or null
  // T = 1 on the RoPE kernels (d in {256, 512}) only: leave the readout as the per-workgroup partial sums
  // [B*h][S][d] in the context's workspace (the caller's next kernel adds them up): no second stage, `out` unused
  struct StepPartials *partials_out = nullptr;
};
struct StepPartials {
  const float *partial = nullptr;
  int S = 0;
};
int bdh_launch_state_steps(bdh_ctx *ctx, const StateStepParams &p);

// Variant used inside the fused model step: the readout is LayerNorm-ed on the fly
// (src/model/bdh.rs:359) when out_ln != nullptr.
int bdh_launch_state_steps_ln(bdh_ctx *ctx, const StateStepParams &p, float *out_ln);
// The same with the partials in a caller-given buffer (nothing is allocated; fails when they do not fit).
int bdh_launch_state_steps_in(bdh_ctx *ctx, const StateStepParams &p, float *out_ln, void *fixed, size_t fixed_bytes);
// The fixed scratch array of the allocation-free decode step: resolve its address on the context's device
// (that device must be current), read it back, and its size.
int bdh_step_scratch_resolve(bdh_ctx *ctx);
void *bdh_step_scratch_ptr(const bdh_ctx *ctx);
size_t bdh_step_scratch_bytes();
// The same T steps as four dense products per chunk on the f32 matrix cores (attention_parallel.hip):
// RoPE / PoPE, f32 state, no bitmask or row counts.
int bdh_launch_state_chunks_f32(bdh_ctx *ctx, const StateStepParams &p, float *out_ln);
// prefill.hip: the same T steps on the bf16 matrix cores (x, v and the scores rounded to bf16, f32 accumulation and
// f32 state; tolerance class 2e-2): any rotary, a lazily decayed state is brought up to date first; host position only.
int bdh_launch_state_prefill_bf16(bdh_ctx *ctx, const StateStepParams &p, float *out_ln);
// prefill.hip: fused_state_aligned (dense causal layout, row-normalised) on the bf16 matrix cores; tolerance class 2e-2
int bdh_launch_fsa_bf16(bdh_ctx *ctx, int B, int h, int T, int N, int dv, const float *query, const float *value,
                        const float *freqs, const float *alibi_slopes_host, int block_size, int rotary, float *out);
// rho <- the up-to-date state, stamps <- clock, for a lazily decayed ALiBi state
int bdh_launch_alibi_materialize(bdh_ctx *ctx, int B, int h, int N, int d, const float *slopes_host, int64_t clock,
                                 const int32_t *clocks_dev, void *rho, int rho_dtype, int32_t *stamps);

// state_deferred.hip: the decode step with logged updates (RoPE, T = 1).  out_ln != nullptr: the readout is also
// written LayerNorm-ed (src/model/bdh.rs:359).  The flush applies the pending steps to rho and empties the log.
int bdh_launch_state_step_deferred(bdh_ctx *ctx, bdh_state_log *log, const float *x, const float *v, const float *freqs,
                                   int64_t position, const int32_t *positions_dev, void *rho, float *out, float *out_ln,
                                   uint64_t *bitmask, int32_t *rows_touched);
int bdh_launch_state_flush(bdh_ctx *ctx, bdh_state_log *log, void *rho);

struct ReluLowrankParams {
  int B, h_in, T, d, h, N;
  const float *in, *weight, *bias;
  float threshold;
  int block_size;
  const uint8_t *active_blocks_host;
  int n_blocks;
  const float *gate;
  float *out;
};
int bdh_launch_relu_lowrank(bdh_ctx *ctx, const ReluLowrankParams &p);
// the same on the f32 matrix cores for many rows per (sequence, head); csrc/attention_parallel.hip
int bdh_launch_relu_lowrank_gemm(bdh_ctx *ctx, const ReluLowrankParams &p, const unsigned char *mask_dev);
// relu_lowrank for ONE input row per head whose values are made by the kernel itself from the partial sums an earlier
// kernel left (a decode step of one sequence: the two reductions of a layer whose inputs come from other CUs ride in
// front of the projection that consumes them, behind its first weight loads):
//   mode 1 (D_y, src/model/bdh.rs:359,370-381): row of head hh = LN(sum_g partial[hh][g][:]), g < S
//   mode 2 (D_x of the next layer, :436-441 then :346-350): row = LN(cur_old + LN(sum_kb dpart[kb][:])), kb < KBN,
//           shared by the heads; the workgroup (0, 0) also writes it to cur_new
//   mode 3 (D_x of the first layer, :319-322 then :346-350): row = LN(embed[tokens[0]]), written to cur_new too
struct ReluLowrankRowParams {
  int mode, h, N, d;
  const float *weight;
  float threshold;
  const float *gate;  // [h][N] or null
  float *out;         // [h][N]
  const float *partial;  // mode 1: [h][S][d]; mode 2: [KBN][d]
  int rows;              // S or KBN
  const float *cur_old;  // mode 2
  float *cur_new;        // modes 2 and 3
  const int64_t *tokens = nullptr;  // mode 3: device, the one token; partial = the embedding table, rows = V
};
int bdh_launch_relu_lowrank_row(bdh_ctx *ctx, const ReluLowrankRowParams &p);
bool bdh_relu_lowrank_row_fits(int d, int rows);
// The first stage of the encoder for one row (M = 1): partial[kb][:] = sum over k-block kb of xy[k] E[k,:], KB rows
// per block; *KBN_out = number of blocks.  partial must hold KBN * d floats.
int bdh_launch_decoder_partial_row(bdh_ctx *ctx, int h, int N, int d, const float *xy, const float *decoder, int KB,
                                   float *partial, int *KBN_out);
// cur[m,:] = LN(cur[m,:] + LN(sum_kb partial[kb][m][:])) and, with head, the output head of the finished rows
int bdh_launch_decoder_finalize_head(bdh_ctx *ctx, const float *partial, int KBN, int M, int d, float *cur,
                                     const struct DecoderHead *head);
int bdh_launch_layer_norm(bdh_ctx *ctx, int64_t rows, int d, const float *in, float *out);
// the same for internal many-row use: statistics by wave reduction, not bit-identical to the index-order sums
int bdh_launch_layer_norm_rows(bdh_ctx *ctx, int64_t rows, int d, const float *in, float *out);

// embed gather + LN (src/model/bdh.rs:319-322); tokens validated on the device: an id
// outside [0,V) writes NaN rows (the reference would panic in the gather).
int bdh_launch_embed_ln(bdh_ctx *ctx, const int64_t *tokens, int64_t rows, int d, int V,
                        const float *embed, float *out);
// mlp = mixed . decoder with mixed[b*T+t, hh*N+n] = xy[b,hh,t,n]; cur = LN(cur + LN(mlp))
// (src/model/bdh.rs:383,436-441)
// The output head of the rows the decoder's second stage finishes, run in that same launch (the last layer of a
// model): logits[m,:] = cur[m,:] . lm_head and, optionally, the greedy token of each sequence's last row.
struct DecoderHead {
  const float *lm_head;  // [d][V]
  int T, V;
  float *logits;         // [M][V]
  int64_t *next_tokens;  // [B] or null
};
int bdh_launch_decoder_residual(bdh_ctx *ctx, int B, int T, int h, int N, int d,
                                const float *xy, const float *decoder, float *cur,
                                const DecoderHead *head = nullptr);
// logits = cur . lm_head (+ argmax of the last token per sequence) (src/model/bdh.rs:446-449)
// attention_parallel.hip: partial[hh][b*T+t][:] = xy[b,hh,t,:] . decoder[hh*N.., :] on the f32 matrix cores
int bdh_launch_decoder_partials_f32(bdh_ctx *ctx, int B, int T, int h, int N, int d, const float *xy,
                                    const float *decoder, float *partial);
// attention_parallel.hip: decode-step encoder for a batch (T = 1): partial[s][m][:] = xy[m, s*KB..] . decoder[s*KB.., :]
int bdh_launch_decoder_splitk_f32(bdh_ctx *ctx, int M, long K, int d, int KB, const float *xy, const float *decoder,
                                  float *partial);
int bdh_launch_lm_head(bdh_ctx *ctx, int B, int T, int d, int V, const float *cur,
                       const float *lm_head, float *logits, int64_t *next_tokens);
// positions[b] = min(positions[b] + delta, INT32_MAX): the device-side form of state.position += T
int bdh_launch_advance_positions(bdh_ctx *ctx, int32_t *positions_dev, int B, int delta);

// viz_taps.hip: out[h,N] = batch mean of the per-row mean |rho| (src/model/bdh.rs:411-419); with stamps the
// state is read through its pending ALiBi decay at clock (or clocks_dev[b] + clock_add)
int bdh_launch_rho_energy(bdh_ctx *ctx, int B, int h, int N, int d, const void *rho, int rho_dtype,
                          const int32_t *stamps, const float *slopes_host, int64_t clock, const int32_t *clocks_dev,
                          int clock_add, float *out);
// dst[hh, 0..cols) = src[hh * head_stride + offset + (0..cols)]
int bdh_launch_gather_head_rows(bdh_ctx *ctx, const float *src, int h, long head_stride, long offset, int cols,
                                float *dst);
int bdh_launch_fill_zero_f32(bdh_ctx *ctx, float *p, long n);

// Four adjacent elements of a state row, f32 or bf16 (raw 16-bit patterns; stores round to nearest even, NaN kept
// quiet): the element access of the decode forms that keep the state in either type.
__device__ __forceinline__ float4 bdh_rho_load4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 bdh_rho_load4(const unsigned short *p) {
  const uint2 v = *reinterpret_cast<const uint2 *>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                     __uint_as_float(v.y & 0xffff0000u));
}
__device__ __forceinline__ unsigned int bdh_bf16_rne(float f) {
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ void bdh_rho_store4(float *p, float4 v) { *reinterpret_cast<float4 *>(p) = v; }
__device__ __forceinline__ void bdh_rho_store4(unsigned short *p, float4 v) {
  uint2 o;
  o.x = bdh_bf16_rne(v.x) | (bdh_bf16_rne(v.y) << 16);
  o.y = bdh_bf16_rne(v.z) | (bdh_bf16_rne(v.w) << 16);
  *reinterpret_cast<uint2 *>(p) = o;
}
