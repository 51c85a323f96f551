// The whole cached step, BDH::forward_with_state (src/model/bdh.rs:309-450), as a
// stream-ordered sequence of the kernels of this library.
#include <new>
#include <vector>

#include "bdh_internal.h"
#include <utility>

namespace {

int ensure_act(bdh_model *m, size_t bytes) {
  if (bytes <= m->act_bytes) return BDH_OK;
  bdh_ctx *ctx = m->ctx;
  if (m->act) {
    BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    BDH_HIP_CHECK(ctx, hipFree(m->act));
    m->act = nullptr;
    m->act_bytes = 0;
  }
  bytes = bdh_align_up(bytes, size_t(1) << 20);
  hipError_t e = hipMalloc(&m->act, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return bdh_fail(ctx, BDH_E_NOMEM, "activation scratch of %zu bytes: %s", bytes, hipGetErrorString(e));
  }
  m->act_bytes = bytes;
  return BDH_OK;
}

// Where a call finds the recurrent state of layer l: one allocation [L,B,h,Nq,d] (the layers `layer_bytes` apart) or
// one pointer per layer, as the reference's ModelState holds it (a Vec of independent per-layer tensors,
// src/model/state.rs:5-15, each taken and put back by its layer, src/model/bdh.rs:274,304).
struct StateRefs {
  void *rho_base = nullptr;
  void *const *rho_layers = nullptr;
  int32_t *stamps_base = nullptr;
  int32_t *const *stamps_layers = nullptr;
  size_t layer_bytes = 0, stamps_layer = 0;
  void *rho(int l) const { return rho_layers ? rho_layers[l] : static_cast<char *>(rho_base) + (size_t)l * layer_bytes; }
  int32_t *stamps(int l) const {
    return stamps_layers ? stamps_layers[l] : (stamps_base ? stamps_base + (size_t)l * stamps_layer : nullptr);
  }
  bool contiguous(int L) const {
    if (!rho_layers) return true;
    for (int l = 1; l < L; ++l)
      if (rho_layers[l] != static_cast<char *>(rho_layers[0]) + (size_t)l * layer_bytes) return false;
    if (stamps_layers)
      for (int l = 1; l < L; ++l)
        if (stamps_layers[l] != stamps_layers[0] + (size_t)l * stamps_layer) return false;
    return true;
  }
};

int model_forward_impl(bdh_model *m, const int64_t *tokens, int B, int T, StateRefs st, int rho_dtype, int64_t position,
                       const int32_t *positions_dev, float *logits, int64_t *next_tokens, float *x_tap, float *viz,
                       bdh_model_logs *logs);

}  // namespace

// the update logs of a model's layers (bdh_model_forward_deferred): one bdh_state_log per layer
struct bdh_model_logs {
  std::vector<bdh_state_log *> layer;
  int B = 0, rho_dtype = BDH_F32, capacity = 0;
};

extern "C" {

int bdh_model_create(bdh_ctx *ctx, const bdh_model_config *c, const bdh_model_weights *w, bdh_model **out) {
  if (!ctx) return BDH_E_INVAL;
  if (!c || !w || !out) return bdh_fail(ctx, BDH_E_INVAL, "null argument");
  *out = nullptr;
  if (c->n_layer < 1 || c->n_embd < 1 || c->n_head < 1 || c->latent < 1 || c->vocab < 1)
    return bdh_fail(ctx, BDH_E_INVAL, "non-positive model dimension");
  if (c->n_head > 64) return bdh_fail(ctx, BDH_E_SHAPE, "n_head %d > 64", c->n_head);
  if (c->rotary != BDH_ROPE && c->rotary != BDH_ALIBI && c->rotary != BDH_POPE)
    return bdh_fail(ctx, BDH_E_INVAL, "rotary %d is not a bdh_rotary value", c->rotary);
  if (c->rotary == BDH_ROPE && (c->latent & 1))
    return bdh_fail(ctx, BDH_E_SHAPE, "RoPE needs an even latent size, got %d", c->latent);
  if ((c->n_embd & 3) || c->n_embd > 1024)
    return bdh_fail(ctx, BDH_E_SHAPE, "n_embd must be a multiple of 4 and <= 1024, got %d", c->n_embd);
  if (!w->embed || !w->encoder || !w->encoder_v || !w->decoder || !w->lm_head)
    return bdh_fail(ctx, BDH_E_INVAL, "null weight pointer");
  bdh_model *m = new (std::nothrow) bdh_model();
  if (!m) return bdh_fail(ctx, BDH_E_NOMEM, "host allocation failed");
  m->ctx = ctx;
  m->cfg = *c;
  m->cfg.alibi_slopes_host = nullptr;
  m->w = *w;
  if (c->rotary == BDH_ALIBI) {
    if (c->alibi_slopes_host)
      memcpy(m->slopes, c->alibi_slopes_host, sizeof(float) * c->n_head);
    else
      bdh_default_alibi_slopes(c->n_head, m->slopes);
  }
  std::vector<float> f(c->latent);
  bdh_build_freqs(c->latent, c->rope_theta, c->rotary, f.data());
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&m->freqs), sizeof(float) * (size_t)c->latent);
  if (e == hipSuccess) e = hipMemcpy(m->freqs, f.data(), sizeof(float) * (size_t)c->latent, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    if (m->freqs) (void)hipFree(m->freqs);
    delete m;
    return bdh_fail(ctx, BDH_E_HIP, "freqs table upload: %s", hipGetErrorString(e));
  }
  *out = m;
  return BDH_OK;
}

int bdh_model_destroy(bdh_model *m) {
  if (!m) return BDH_OK;
  if (m->ctx) (void)hipStreamSynchronize(m->ctx->stream);
  if (m->freqs) (void)hipFree(m->freqs);
  if (m->act) (void)hipFree(m->act);
  delete m;
  return BDH_OK;
}

int bdh_advance_positions(bdh_ctx *ctx, int32_t *positions_dev, int B, int delta) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || (B > 0 && !positions_dev)) return bdh_fail(ctx, BDH_E_INVAL, "bad positions buffer");
  if (B == 0) return BDH_OK;
  return bdh_launch_advance_positions(ctx, positions_dev, B, delta);
}

size_t bdh_model_state_bytes(const bdh_model *m, int B, int rho_dtype) {
  if (!m || B < 0) return 0;
  const size_t Nq = m->cfg.rotary == BDH_POPE ? 2 * (size_t)m->cfg.latent : (size_t)m->cfg.latent;
  const size_t es = rho_dtype == BDH_BF16 ? 2 : 4;
  return (size_t)m->cfg.n_layer * B * m->cfg.n_head * Nq * m->cfg.n_embd * es;
}

int bdh_model_forward(bdh_model *m, const int64_t *tokens, int B, int T, void *rho, int rho_dtype,
                      int64_t position, float *logits, int64_t *next_tokens, float *x_tap) {
  return bdh_model_forward_ex(m, tokens, B, T, rho, rho_dtype, position, nullptr, logits, next_tokens, x_tap);
}

int bdh_model_forward_ex(bdh_model *m, const int64_t *tokens, int B, int T, void *rho, int rho_dtype,
                         int64_t position, const int32_t *positions_dev, float *logits, int64_t *next_tokens,
                         float *x_tap) {
  return bdh_model_forward_lazy(m, tokens, B, T, rho, rho_dtype, nullptr, position, positions_dev, logits,
                                next_tokens, x_tap);
}

int bdh_model_forward_lazy(bdh_model *m, const int64_t *tokens, int B, int T, void *rho, int rho_dtype,
                           int32_t *stamps, int64_t position, const int32_t *positions_dev, float *logits,
                           int64_t *next_tokens, float *x_tap) {
  return bdh_model_forward_viz(m, tokens, B, T, rho, rho_dtype, stamps, position, positions_dev, logits, next_tokens,
                               x_tap, nullptr);
}

int bdh_model_forward_viz(bdh_model *m, const int64_t *tokens, int B, int T, void *rho, int rho_dtype,
                          int32_t *stamps, int64_t position, const int32_t *positions_dev, float *logits,
                          int64_t *next_tokens, float *x_tap, float *viz) {
  if (!m) return BDH_E_INVAL;
  if (B > 0 && T > 0 && !rho) return bdh_fail(m->ctx, BDH_E_INVAL, "null data pointer");
  StateRefs st;
  st.rho_base = rho;
  st.stamps_base = stamps;
  return model_forward_impl(m, tokens, B, T, st, rho_dtype, position, positions_dev, logits, next_tokens, x_tap, viz,
                            nullptr);
}

int bdh_model_forward_layers(bdh_model *m, const int64_t *tokens, int B, int T, void *const *rho_layers_host,
                             int rho_dtype, int32_t *const *stamps_layers_host, int64_t position,
                             const int32_t *positions_dev, float *logits, int64_t *next_tokens, float *x_tap) {
  if (!m) return BDH_E_INVAL;
  if (B > 0 && T > 0) {
    if (!rho_layers_host) return bdh_fail(m->ctx, BDH_E_INVAL, "null data pointer");
    for (int l = 0; l < m->cfg.n_layer; ++l)
      if (!rho_layers_host[l] || (stamps_layers_host && !stamps_layers_host[l]))
        return bdh_fail(m->ctx, BDH_E_INVAL, "null state pointer of layer %d", l);
  }
  StateRefs st;
  st.rho_layers = rho_layers_host;
  st.stamps_layers = stamps_layers_host;
  return model_forward_impl(m, tokens, B, T, st, rho_dtype, position, positions_dev, logits, next_tokens, x_tap,
                            nullptr, nullptr);
}

}  // extern "C"

namespace {

int model_forward_impl(bdh_model *m, const int64_t *tokens, int B, int T, StateRefs st, int rho_dtype, int64_t position,
                       const int32_t *positions_dev, float *logits, int64_t *next_tokens, float *x_tap, float *viz,
                       bdh_model_logs *logs) {
  bdh_ctx *ctx = m->ctx;
  const bool has_stamps = st.stamps_base || st.stamps_layers;
  if (has_stamps && m->cfg.rotary != BDH_ALIBI)
    return bdh_fail(ctx, BDH_E_INVAL, "decay stamps only apply to an ALiBi model");
  if (has_stamps && position + T > 0x7fffffffLL) return bdh_fail(ctx, BDH_E_INVAL, "position beyond the stamp range");
  if (B < 0 || T < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative batch or time");
  if (position < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative position");
  if (rho_dtype != BDH_F32 && rho_dtype != BDH_BF16) return bdh_fail(ctx, BDH_E_INVAL, "bad rho_dtype");
  if (B == 0 || T == 0) return BDH_OK;
  if (!tokens || !logits) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  const bdh_model_config &c = m->cfg;
  const int d = c.n_embd, h = c.n_head, N = c.latent, V = c.vocab, L = c.n_layer;
  const size_t Nq = c.rotary == BDH_POPE ? 2 * (size_t)N : (size_t)N;
  const size_t M = (size_t)B * T;
  st.layer_bytes = (size_t)B * h * Nq * d * (rho_dtype == BDH_BF16 ? 2 : 4);
  st.stamps_layer = (size_t)B * h * N;
  for (int l = 0; l < L; ++l)
    if (!bdh_aligned(st.rho(l), 16)) return bdh_fail(ctx, BDH_E_ALIGN, "rho needs 16-byte alignment");
  // the fused decode forms below walk one allocation: layers given one by one take them only when they are adjacent
  const bool contiguous = st.contiguous(L);
  void *rho = st.rho(0);
  int32_t *stamps = st.stamps(0);

  // A decode step (one token per sequence, f32 state, no by-products) need not run kernel by kernel:
  //  * a small model (d <= 256, h*N <= 2048) can run the whole step in ONE launch, a workgroup per sequence; one CU then
  //    streams all the projection weights of the step, W bytes;
  //  * a mid-size model (128 <= d <= 512, up to 64 blocks of 64 neurons) can run TWO launches per layer, a workgroup
  //    per block; every workgroup streams its share of the layer's weights once per sequence.
  // Measured at the sizes of the reference's configurations (W = 3 / 6.75 / 12 / 96 MiB; us per step, one launch | two
  // per layer | kernel by kernel): tiny 77|77|112 at B=1, 84|100|145 at B=64; small 152|82|130 at B=1, 168|127|195 at
  // B=64, 323|442|478 at B=256; base 223|83|123 at B=1, 273|210|240 at B=64, 559|-|654 at B=256; large -|210|308 at
  // B=1, -|519|554 at B=16, -|1092|981 at B=33.
  if (T == 1 && !x_tap && !viz && !logs && contiguous && ctx->opt_model_one_launch != 0) {
    const size_t w_layer = sizeof(float) * (size_t)3 * h * N * d;
    const size_t w_bytes = w_layer * L;
    const bool small_fits = bdh_model_small_fits(c);
    const bool forced = ctx->opt_model_one_launch == 2;
    const bool one_first = small_fits && (forced || w_bytes <= (size_t(4) << 20));
    const bool phases = !one_first && bdh_model_phase_fits(c) && B <= ctx->opt_model_phase_batch &&
                        (size_t)B * w_layer <= (size_t(256) << 20);
    const int b_min = w_bytes <= (size_t(8) << 20) ? 16 : 128;
    if (one_first || (!phases && small_fits && B >= b_min))
      return bdh_launch_model_small(m, tokens, B, rho, rho_dtype, stamps, position, positions_dev, logits, next_tokens);
    if (phases) {
      int rc2 = ensure_act(m, sizeof(float) * bdh_model_phase_scratch_floats(c, B));
      if (rc2 != BDH_OK) return rc2;
      float *scratch = static_cast<float *>(m->act);
      float *cur_final = nullptr, *dpart = nullptr;
      int G = 0;
      rc2 = bdh_launch_model_phases(m, tokens, B, scratch, rho, rho_dtype, stamps, position, positions_dev, &cur_final,
                                    &dpart, &G);
      if (rc2 != BDH_OK) return rc2;
      if (V <= 1024)  // the last layer's second stage (:436-441) and the head (:446-449) in one launch
        return bdh_launch_phase_head(m, B, cur_final, dpart, G, logits, next_tokens);
      rc2 = bdh_launch_decoder_finalize(ctx, dpart, G, B, d, cur_final);
      if (rc2 != BDH_OK) return rc2;
      return bdh_launch_lm_head(ctx, B, 1, d, V, cur_final, m->w.lm_head, logits, next_tokens);
    }
  }

  // A decode step of ONE sequence through a RoPE model too large for the fused forms above (BASELINE config 1): four
  // launches per layer instead of six.  The two reductions whose inputs come from other CUs -- the readout partials with
  // their LayerNorm, the encoder partials with the two LayerNorms and the residual -- are redone by every workgroup of the
  // projection that consumes the result (D_y, the next layer's D_x), behind its first weight loads.
  // Taken while what every workgroup adds up stays small against the weights it streams: at most 64 KiB of readout
  // partials per head (N/128 rows of d floats) and 128 KiB of encoder partials (h*N/KB rows); beyond that the redundant
  // sums cost more than the two launches they replace (measured at d=512, h=8, N=16384: 2.97 against 2.87 ms per token).
  const int fused_kb = ctx->opt_model_fused_kb;
  if (B == 1 && T == 1 && !x_tap && !viz && !logs && ctx->opt_model_fused_rows != 0 && c.rotary == BDH_ROPE &&
      (d == 256 || d == 512) && N >= 2 && (N % 2) == 0 && (long)N * d <= (2L << 20) &&
      (long)h * N * d <= (long)fused_kb * (1L << 15)) {
    const int KB = fused_kb;
    const size_t K = (size_t)h * N;
    const size_t kbn_max = (K + KB - 1) / KB;
    const size_t n_row = bdh_align_up((size_t)d, 64), n_lat = bdh_align_up(K, 64);
    int rc2 = ensure_act(m, sizeof(float) * (2 * n_row + 2 * n_lat + kbn_max * d));
    if (rc2 != BDH_OK) return rc2;
    float *cur_a = static_cast<float *>(m->act);
    float *cur_b = cur_a + n_row;
    float *xr = cur_b + n_row;
    float *xyr = xr + n_lat;
    float *dpart = xyr + n_lat;
    int KBN = 0;
    for (int l = 0; l < L; ++l) {
      if (l == 0) {  // :319-322, then :346-350
        ReluLowrankRowParams px{3, h, N, d, m->w.encoder, c.relu_threshold, nullptr, xr, m->w.embed, V, nullptr, cur_a, tokens};
        rc2 = bdh_launch_relu_lowrank_row(ctx, px);
      } else {  // :436-441 of the previous layer, then :346-350
        ReluLowrankRowParams px{2, h, N, d, m->w.encoder, c.relu_threshold, nullptr, xr, dpart, KBN, cur_a, cur_b};
        rc2 = bdh_launch_relu_lowrank_row(ctx, px);
        std::swap(cur_a, cur_b);
      }
      if (rc2 != BDH_OK) return rc2;
      StepPartials sp;
      StateStepParams ps{1, h, 1, N, d, c.rotary, rho_dtype, xr, cur_a, m->freqs, position, positions_dev, nullptr,
                         st.rho(l), nullptr, nullptr, nullptr, nullptr, &sp};
      rc2 = bdh_launch_state_steps(ctx, ps);
      if (rc2 != BDH_OK) return rc2;
      // :359,370-381  xy = x * relu(LN(sum of the readout partials) . encoder_v - thr)
      ReluLowrankRowParams py{1, h, N, d, m->w.encoder_v, c.relu_threshold, xr, xyr, sp.partial, sp.S, nullptr, nullptr};
      rc2 = bdh_launch_relu_lowrank_row(ctx, py);
      if (rc2 != BDH_OK) return rc2;
      rc2 = bdh_launch_decoder_partial_row(ctx, h, N, d, xyr, m->w.decoder, KB, dpart, &KBN);  // :383
      if (rc2 != BDH_OK) return rc2;
    }
    const DecoderHead head{m->w.lm_head, 1, V, logits, next_tokens};
    return bdh_launch_decoder_finalize_head(ctx, dpart, KBN, 1, d, cur_a, &head);  // :436-449
  }

  // activation scratch: cur [M,d] | x [B,h,T,N] | xy [B,h,T,N] | attn [B,h,T,d] | attn_ln [B,h,T,d] | last [h,d]
  const size_t n_cur = bdh_align_up(M * d, 64), n_x = bdh_align_up(M * h * N, 64), n_a = bdh_align_up(M * h * d, 64);
  const size_t n_last = viz ? bdh_align_up((size_t)h * d, 64) : 0;
  int rc = ensure_act(m, sizeof(float) * (n_cur + 2 * n_x + 2 * n_a + n_last));
  if (rc != BDH_OK) return rc;
  float *cur = static_cast<float *>(m->act);
  float *x = cur + n_cur;
  float *xy = x + n_x;
  float *attn = xy + n_x;
  float *attn_ln = attn + n_a;
  float *last = attn_ln + n_a;

  rc = bdh_launch_embed_ln(ctx, tokens, (int64_t)M, d, V, m->w.embed, cur);  // :319-322
  if (rc != BDH_OK) return rc;
  for (int l = 0; l < L; ++l) {  // :336 — the same weights in every layer
    float *x_l = x_tap ? x_tap + (size_t)l * M * h * N : x;
    // :337-351  x = relu(cur . encoder - thr)
    ReluLowrankParams px{B, 1, T, d, h, N, cur, m->w.encoder, nullptr, c.relu_threshold, 1, nullptr, 0, nullptr, x_l};
    rc = bdh_launch_relu_lowrank(ctx, px);
    if (rc != BDH_OK) return rc;
    // :353-359  recurrent attention (value = cur) and LayerNorm of its output
    if (logs) {  // the update of :298 goes to the layer's log, the state is only read
      rc = bdh_launch_state_step_deferred(ctx, logs->layer[l], x_l, cur, m->freqs, position, positions_dev, st.rho(l), attn,
                                          attn_ln, nullptr, nullptr);
    } else {
      StateStepParams ps{B, h, T, N, d, c.rotary, rho_dtype, x_l, cur, m->freqs, position, positions_dev,
                         c.rotary == BDH_ALIBI ? m->slopes : nullptr, st.rho(l), attn, nullptr, nullptr, st.stamps(l)};
      rc = bdh_launch_state_steps_ln(ctx, ps, attn_ln);
    }
    if (rc != BDH_OK) return rc;
    // :361-381  xy = x * relu(LN(attn) . encoder_v - thr)
    ReluLowrankParams py{B, h, T, d, h, N, attn_ln, m->w.encoder_v, nullptr, c.relu_threshold, 1, nullptr, 0, x_l, xy};
    rc = bdh_launch_relu_lowrank(ctx, py);
    if (rc != BDH_OK) return rc;
    if (viz) {  // :386-434: first sequence, last token; the state is already this call's updated one
      float *vz = viz + (size_t)l * 4 * h * N;
      const long hs = (long)T * N, off = (long)(T - 1) * N;
      rc = bdh_launch_gather_head_rows(ctx, x_l, h, hs, off, N, vz);
      if (rc != BDH_OK) return rc;
      // y alone is never stored (the gate is fused into the D_y kernel): one more D_y pass over the h rows
      rc = bdh_launch_gather_head_rows(ctx, attn_ln, h, (long)T * d, (long)(T - 1) * d, d, last);
      if (rc != BDH_OK) return rc;
      ReluLowrankParams pv{1, h, 1, d, h, N, last, m->w.encoder_v, nullptr, c.relu_threshold, 1, nullptr, 0, nullptr,
                           vz + (size_t)h * N};
      rc = bdh_launch_relu_lowrank(ctx, pv);
      if (rc != BDH_OK) return rc;
      rc = bdh_launch_gather_head_rows(ctx, xy, h, hs, off, N, vz + (size_t)2 * h * N);
      if (rc != BDH_OK) return rc;
      if (Nq == (size_t)N)
        rc = bdh_launch_rho_energy(ctx, B, h, N, d, st.rho(l), rho_dtype, st.stamps(l), m->slopes, position + T,
                                   positions_dev, T, vz + (size_t)3 * h * N);
      else  // PoPE: the state has 2N rows, the reference stores a zero map (:413-424)
        rc = bdh_launch_fill_zero_f32(ctx, vz + (size_t)3 * h * N, (long)h * N);
      if (rc != BDH_OK) return rc;
    }
    // :383,436-441  cur = LN(cur + LN(mixed . decoder)); the last layer's launch also runs the output head (:446-449)
    const DecoderHead head{m->w.lm_head, T, V, logits, next_tokens};
    rc = bdh_launch_decoder_residual(ctx, B, T, h, N, d, xy, m->w.decoder, cur, l == L - 1 ? &head : nullptr);
    if (rc != BDH_OK) return rc;
  }
  return BDH_OK;
}

}  // namespace

extern "C" {

int bdh_model_logs_create(bdh_model *m, int B, int rho_dtype, int capacity, bdh_model_logs **out) {
  if (!m) return BDH_E_INVAL;
  bdh_ctx *ctx = m->ctx;
  if (!out) return bdh_fail(ctx, BDH_E_INVAL, "null argument");
  *out = nullptr;
  const bdh_model_config &c = m->cfg;
  if (c.rotary != BDH_ROPE) return bdh_fail(ctx, BDH_E_UNSUPPORTED, "deferred state updates are built for RoPE models");
  bdh_model_logs *logs = new (std::nothrow) bdh_model_logs();
  if (!logs) return bdh_fail(ctx, BDH_E_NOMEM, "host allocation failed");
  logs->B = B;
  logs->rho_dtype = rho_dtype;
  logs->capacity = capacity;
  for (int l = 0; l < c.n_layer; ++l) {
    bdh_state_log *one = nullptr;
    const int rc = bdh_state_log_create(ctx, B, c.n_head, c.latent, c.n_embd, rho_dtype, capacity, &one);
    if (rc != BDH_OK) {
      for (bdh_state_log *p : logs->layer) bdh_state_log_destroy(ctx, p);
      delete logs;
      return rc;
    }
    logs->layer.push_back(one);
  }
  *out = logs;
  return BDH_OK;
}

int bdh_model_logs_destroy(bdh_model *m, bdh_model_logs *logs) {
  if (!logs) return BDH_OK;
  for (bdh_state_log *p : logs->layer) bdh_state_log_destroy(m ? m->ctx : nullptr, p);
  delete logs;
  return BDH_OK;
}

int bdh_model_logs_pending(const bdh_model_logs *logs) {
  return (logs && !logs->layer.empty()) ? bdh_state_log_pending(logs->layer[0]) : BDH_E_INVAL;
}

int bdh_model_forward_deferred(bdh_model *m, bdh_model_logs *logs, const int64_t *tokens, int B, void *rho, int rho_dtype,
                               int64_t position, const int32_t *positions_dev, float *logits, int64_t *next_tokens) {
  if (!m) return BDH_E_INVAL;
  bdh_ctx *ctx = m->ctx;
  if (!logs) return bdh_fail(ctx, BDH_E_INVAL, "null model logs");
  if ((int)logs->layer.size() != m->cfg.n_layer || B != logs->B || rho_dtype != logs->rho_dtype)
    return bdh_fail(ctx, BDH_E_INVAL, "the logs were created for %zu layers, batch %d, state type %d", logs->layer.size(),
                    logs->B, logs->rho_dtype);
  if (!rho) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  StateRefs st;
  st.rho_base = rho;
  return model_forward_impl(m, tokens, B, 1, st, rho_dtype, position, positions_dev, logits, next_tokens, nullptr,
                            nullptr, logs);
}

int bdh_model_forward_deferred_layers(bdh_model *m, bdh_model_logs *logs, const int64_t *tokens, int B,
                                      void *const *rho_layers_host, int rho_dtype, int64_t position,
                                      const int32_t *positions_dev, float *logits, int64_t *next_tokens) {
  if (!m) return BDH_E_INVAL;
  bdh_ctx *ctx = m->ctx;
  if (!logs) return bdh_fail(ctx, BDH_E_INVAL, "null model logs");
  if ((int)logs->layer.size() != m->cfg.n_layer || B != logs->B || rho_dtype != logs->rho_dtype)
    return bdh_fail(ctx, BDH_E_INVAL, "the logs were created for %zu layers, batch %d, state type %d", logs->layer.size(),
                    logs->B, logs->rho_dtype);
  if (!rho_layers_host) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  for (int l = 0; l < m->cfg.n_layer; ++l)
    if (!rho_layers_host[l]) return bdh_fail(ctx, BDH_E_INVAL, "null state pointer of layer %d", l);
  StateRefs st;
  st.rho_layers = rho_layers_host;
  return model_forward_impl(m, tokens, B, 1, st, rho_dtype, position, positions_dev, logits, next_tokens, nullptr,
                            nullptr, logs);
}

int bdh_model_flush_layers(bdh_model *m, bdh_model_logs *logs, void *const *rho_layers_host) {
  if (!m) return BDH_E_INVAL;
  bdh_ctx *ctx = m->ctx;
  if (!logs) return bdh_fail(ctx, BDH_E_INVAL, "null model logs");
  if ((int)logs->layer.size() != m->cfg.n_layer) return bdh_fail(ctx, BDH_E_INVAL, "the logs belong to another model");
  if (bdh_model_logs_pending(logs) == 0) return BDH_OK;
  if (!rho_layers_host) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  for (int l = 0; l < m->cfg.n_layer; ++l) {
    if (!rho_layers_host[l]) return bdh_fail(ctx, BDH_E_INVAL, "null state pointer of layer %d", l);
    const int rc = bdh_state_flush(ctx, logs->layer[l], rho_layers_host[l]);
    if (rc != BDH_OK) return rc;
  }
  return BDH_OK;
}

int bdh_model_flush(bdh_model *m, bdh_model_logs *logs, void *rho) {
  if (!m) return BDH_E_INVAL;
  bdh_ctx *ctx = m->ctx;
  if (!logs) return bdh_fail(ctx, BDH_E_INVAL, "null model logs");
  if ((int)logs->layer.size() != m->cfg.n_layer) return bdh_fail(ctx, BDH_E_INVAL, "the logs belong to another model");
  if (bdh_model_logs_pending(logs) == 0) return BDH_OK;
  if (!rho) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  const bdh_model_config &c = m->cfg;
  const size_t layer_bytes = (size_t)logs->B * c.n_head * c.latent * c.n_embd * (logs->rho_dtype == BDH_BF16 ? 2 : 4);
  for (int l = 0; l < c.n_layer; ++l) {
    const int rc = bdh_state_flush(ctx, logs->layer[l], static_cast<char *>(rho) + (size_t)l * layer_bytes);
    if (rc != BDH_OK) return rc;
  }
  return BDH_OK;
}

int bdh_model_forward_fast(bdh_model *m, const int64_t *tokens, int B, int T, int time_block_size, float *logits) {
  return bdh_model_forward_fast_ex(m, tokens, B, T, time_block_size, nullptr, 0, 1, nullptr, 0, logits);
}

int bdh_model_forward_fast_ex(bdh_model *m, const int64_t *tokens, int B, int T, int time_block_size,
                              const int32_t *time_pairs_host, int n_time_pairs, int latent_block_size,
                              const uint8_t *latent_blocks_host, int n_latent_blocks, float *logits) {
  if (!m) return BDH_E_INVAL;
  bdh_ctx *ctx = m->ctx;
  if (B < 0 || T < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative batch or time");
  if (B == 0 || T == 0) return BDH_OK;
  if (!tokens || !logits) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  const bdh_model_config &c = m->cfg;
  const int d = c.n_embd, h = c.n_head, N = c.latent, V = c.vocab, L = c.n_layer;
  const size_t M = (size_t)B * T;
  // activation scratch: cur [M,d] | x [B,h,T,N] | xy [B,h,T,N] | attn [B,h,T,d] | attn_ln [B,h,T,d]
  const size_t n_cur = bdh_align_up(M * d, 64), n_x = bdh_align_up(M * h * N, 64), n_a = bdh_align_up(M * h * d, 64);
  int rc = ensure_act(m, sizeof(float) * (n_cur + 2 * n_x + 2 * n_a));
  if (rc != BDH_OK) return rc;
  float *cur = static_cast<float *>(m->act);
  float *x = cur + n_cur;
  float *xy = x + n_x;
  float *attn = xy + n_x;
  float *attn_ln = attn + n_a;
  rc = bdh_launch_embed_ln(ctx, tokens, (int64_t)M, d, V, m->w.embed, cur);  // :97-100
  if (rc != BDH_OK) return rc;
  const int block = time_block_size > 0 ? time_block_size : 1;  // plain branch: element-wise tril(-1)
  const int lat_block = latent_block_size > 0 ? latent_block_size : 1;
  if (time_pairs_host && time_block_size <= 0)
    return bdh_fail(ctx, BDH_E_INVAL, "a time-block pattern belongs to the fused branch (time_block_size > 0)");
  if (n_time_pairs < 0 || n_latent_blocks < 0 || (n_time_pairs > 0 && !time_pairs_host))
    return bdh_fail(ctx, BDH_E_INVAL, "pattern counts do not match the pattern pointers");
  for (int l = 0; l < L; ++l) {  // :113
    ReluLowrankParams px{B, 1, T, d, h, N, cur, m->w.encoder, nullptr, c.relu_threshold, lat_block, latent_blocks_host,
                         n_latent_blocks, nullptr, x};
    rc = bdh_launch_relu_lowrank(ctx, px);  // :114-129
    if (rc != BDH_OK) return rc;
    // :131  Attention::forward: all tokens at once from position 0, row-normalised
    rc = bdh_fused_state_aligned(ctx, B, h, T, N, d, x, cur, m->freqs, c.rotary == BDH_ALIBI ? m->slopes : nullptr, block,
                                 time_pairs_host, n_time_pairs, c.rotary, 1, attn);
    if (rc != BDH_OK) return rc;
    rc = bdh_launch_layer_norm(ctx, (int64_t)M * h, d, attn, attn_ln);  // :132
    if (rc != BDH_OK) return rc;
    ReluLowrankParams py{B, h, T, d, h, N, attn_ln, m->w.encoder_v, nullptr, c.relu_threshold, lat_block, latent_blocks_host,
                         n_latent_blocks, x, xy};
    rc = bdh_launch_relu_lowrank(ctx, py);  // :134-151
    if (rc != BDH_OK) return rc;
    rc = bdh_launch_decoder_residual(ctx, B, T, h, N, d, xy, m->w.decoder, cur);  // :153-162
    if (rc != BDH_OK) return rc;
  }
  return bdh_launch_lm_head(ctx, B, T, d, V, cur, m->w.lm_head, logits, nullptr);  // :164-168
}

}  // extern "C"
