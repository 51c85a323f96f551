// C++ host-mirror test (GPU): the reference's own test recipes, written against
// burn_dragon_amd/host/bdh_host.hpp, with values checked against the C oracle.
//   tests/model_paths.rs:66-91        inference_paths_run_across_configs
//   tests/fused_kernel_tests.rs:35-68 relu_lowrank_fused_matches_reference
//   tests/fused_kernel_tests.rs:70-120 fused_attention_matches_reference_when_alibi_disabled
// Built by __graft_entry__.build(); run by tests/test_gpu_host_cpp.py.
#include <cmath>
#include <cstdio>
#include <random>

#include "../burn_dragon_amd/host/bdh_host.hpp"

extern "C" {  // oracle/bdh_oracle.c (the checker; never linked into the library)
typedef struct {
  int n_layer, n_embd, n_head, latent, vocab, rotary;
  float rope_theta, relu_threshold;
  const float *alibi_slopes;
  const float *embed, *encoder, *encoder_v, *decoder, *lm_head;
} orc_model;
int orc_forward_with_state(const orc_model *m, const int64_t *tokens, int B, int T, float *rho, int64_t *position,
                           float *logits, float *x_tap, float *attn_tap, int sparse_state);
void orc_relu_lowrank(const float *in, int B, int hin, int T, int d, const float *w, int h, int N, const float *bias,
                      float thr, int block_size, const uint8_t *active_blocks, int n_blocks, float *out);
void orc_fused_state_aligned(const float *query, const float *value, const float *freqs, const float *slopes, int B, int h,
                             int T, int N, int dv, int block_size, const int32_t *pairs, int n_pairs, int rotary, float *out);
void orc_build_freqs(int latent, float theta, int rotary, float *out);
}

using namespace bdh;

static int failures = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::printf("FAIL %s:%d  %s\n", __FILE__, __LINE__, #cond);           \
      ++failures;                                                           \
    }                                                                       \
  } while (0)

static std::vector<float> randn(std::mt19937 &g, size_t n, float scale) {
  std::normal_distribution<float> nd(0.0f, 1.0f);
  std::vector<float> v(n);
  for (auto &x : v) x = scale * nd(g);
  return v;
}

static double rel_err(const std::vector<float> &a, const std::vector<float> &b) {
  double num = 0, den = 1e-30;
  for (size_t i = 0; i < a.size(); ++i) {
    num = std::max(num, (double)std::fabs(a[i] - b[i]));
    den = std::max(den, (double)std::fabs(b[i]));
  }
  return num / den;
}

static void assert_close(const std::vector<float> &lhs, const std::vector<float> &rhs, float atol, float rtol) {
  EXPECT(lhs.size() == rhs.size());
  for (size_t i = 0; i < lhs.size() && i < rhs.size(); ++i)
    if (std::fabs(lhs[i] - rhs[i]) > atol + rtol * std::fabs(rhs[i])) {
      std::printf("FAIL difference %g at %zu (lhs=%g rhs=%g)\n", std::fabs(lhs[i] - rhs[i]), i, lhs[i], rhs[i]);
      ++failures;
      return;
    }
}

static BDHConfig build_config(RotaryEmbedding rotary, bool fused) {  // tests/model_paths.rs:12-24
  BDHConfig config;
  config.n_layer = 2;
  config.n_embd = 16;
  config.n_head = 2;
  config.mlp_internal_dim_multiplier = 4;
  config.vocab_size = 32;
  config.dropout = 0.0;
  config.fused_kernels.enabled = fused;
  config.fused_kernels.set_block_sizes(4, 4);
  config.fused_kernels.set_rotary_embedding(rotary);
  return config;
}

static void inference_paths_run_across_configs(const Context &ctx) {
  const std::pair<RotaryEmbedding, bool> configs[] = {
      {RotaryEmbedding::Rope, false}, {RotaryEmbedding::Pope, false}, {RotaryEmbedding::Alibi, false}, {RotaryEmbedding::Alibi, true}};
  for (auto [rotary, fused] : configs) {
    BDHConfig config = build_config(rotary, fused);
    std::mt19937 g(11);
    const size_t h = 2, d = 16, N = config.latent_per_head(), V = 32;
    BDHWeightsHost w{randn(g, V * d, 1.0f), randn(g, h * d * N, 0.02f), randn(g, h * d * N, 0.02f), randn(g, h * N * d, 0.02f),
                     randn(g, d * V, 0.02f)};
    BDH model(ctx, config, w);
    const std::vector<int64_t> tokens{0, 1, 2, 3, 4, 5, 6, 7};
    ModelState state = model.init_state();
    Tensor logits = model.forward_with_state(tokens, 2, 4, state);
    EXPECT((logits.shape() == std::vector<size_t>{2, 4, 32}));
    EXPECT(state.position == 4);
    // values against the oracle
    const size_t Nq = rotary == RotaryEmbedding::Pope ? 2 * N : N;
    std::vector<float> rho(2 * 2 * h * Nq * d, 0.0f), ref(2 * 4 * V);
    orc_model m{2, (int)d, (int)h, (int)N, (int)V, (int)rotary, 65536.0f, 0.0f, nullptr,
                w.embed.data(), w.encoder.data(), w.encoder_v.data(), w.decoder.data(), w.lm_head.data()};
    int64_t pos = 0;
    EXPECT(orc_forward_with_state(&m, tokens.data(), 2, 4, rho.data(), &pos, ref.data(), nullptr, nullptr, 0) == 0);
    EXPECT(pos == 4);
    const double e = rel_err(logits.to_host(), ref);
    std::printf("  %-5s fused=%d logits rel err %.2e\n", as_str(rotary), (int)fused, e);
    EXPECT(e < 1e-3);
    EXPECT(rel_err(state.storage->to_host(), rho) < 1e-3);
  }
}

static void relu_lowrank_fused_matches_reference(const Context &ctx) {
  std::mt19937 g(42);
  auto input = randn(g, 2 * 1 * 5 * 6, 1.0f), weight = randn(g, 1 * 3 * 6 * 8, 1.0f), bias = randn(g, 3 * 1 * 8, 0.5f);
  const float threshold = 0.25f;
  auto layout = kernel::BlockPattern1d::from_blocks(3, {0, 2});
  Tensor ti = Tensor::from_host(input, {2, 1, 5, 6}), tw = Tensor::from_host(weight, {1, 3, 6, 8}), tb = Tensor::from_host(bias, {3, 1, 8});
  Tensor fused = kernel::relu_lowrank::fused_forward(ctx, ti, tw, &tb, threshold, layout);
  ctx.synchronize();
  EXPECT((fused.shape() == std::vector<size_t>{2, 3, 5, 8}));
  // reference: relu(input.matmul(weight) + bias - threshold) * mask, in double
  std::vector<float> reference(2 * 3 * 5 * 8);
  const double mask[8] = {1, 1, 1, 0, 0, 0, 1, 1};
  for (int b = 0; b < 2; ++b)
    for (int hh = 0; hh < 3; ++hh)
      for (int t = 0; t < 5; ++t)
        for (int n = 0; n < 8; ++n) {
          double s = 0;
          for (int k = 0; k < 6; ++k) s += (double)input[(b * 5 + t) * 6 + k] * weight[(hh * 6 + k) * 8 + n];
          s = s + bias[hh * 8 + n] - threshold;
          reference[((b * 3 + hh) * 5 + t) * 8 + n] = (float)(std::max(s, 0.0) * mask[n]);
        }
  assert_close(fused.to_host(), reference, 1e-5f, 1e-5f);
  std::vector<float> orc(reference.size());
  const uint8_t act[3] = {1, 0, 1};
  orc_relu_lowrank(input.data(), 2, 1, 5, 6, weight.data(), 3, 8, bias.data(), threshold, 3, act, 3, orc.data());
  assert_close(fused.to_host(), orc, 1e-6f, 1e-6f);
}

static void fused_attention_matches_reference(const Context &ctx, RotaryEmbedding rotary, unsigned seed) {
  std::mt19937 g(seed);
  const int batch = 1, heads = 2, time = 6, latent = 8, value_dim = 6;
  auto query = randn(g, batch * heads * time * latent, 1.0f), value = randn(g, batch * time * value_dim, 1.0f);
  auto freqs = kernel::linear_attention::build_freqs(latent, 65536.0f, rotary);
  std::vector<float> f2(latent);
  orc_build_freqs(latent, 65536.0f, (int)rotary, f2.data());
  EXPECT(freqs == f2);
  Tensor tq = Tensor::from_host(query, {1, 2, 6, 8}), tv = Tensor::from_host(value, {1, 1, 6, 6}), tf = Tensor::from_host(freqs, {1, 1, 1, 8});
  Tensor fused = kernel::linear_attention::fused_state_aligned(ctx, tq, tv, tf, nullptr, kernel::BlockPattern2d::dense(3), rotary);
  ctx.synchronize();
  std::vector<float> ref(batch * heads * time * value_dim);
  orc_fused_state_aligned(query.data(), value.data(), freqs.data(), nullptr, batch, heads, time, latent, value_dim, 3, nullptr, 0,
                          (int)rotary, ref.data());
  assert_close(fused.to_host(), ref, 1e-4f, 1e-4f);
}

static void config_and_state_semantics() {
  BDHConfig c;
  EXPECT(c.latent_per_head() == 256 && c.latent_total() == 1024);
  EXPECT(c.fused_kernels.rotary_embedding == RotaryEmbedding::Alibi);
  c.n_head = 3;
  c.n_embd = 10;
  c.mlp_internal_dim_multiplier = 1;
  bool threw = false;
  try {
    (void)c.latent_per_head();
  } catch (const std::logic_error &) {
    threw = true;
  }
  EXPECT(threw);
  ModelOverrides o;
  o.n_layer = 2;
  o.block_size = 0;
  o.rotary_embedding = RotaryEmbedding::Rope;
  BDHConfig b = build_model_config(o, 8);
  EXPECT(b.n_layer == 2 && b.fused_kernels.block_sparse.time.block_size() == 1);
  EXPECT(b.fused_kernels.rotary_embedding == RotaryEmbedding::Rope);
  ModelState st(3);
  st.position = 5;
  st.trim(2);
  EXPECT(st.len() == 5);
  st.reset();
  EXPECT(st.is_empty() && !st.layers[0].rho.has_value());
  auto d2 = kernel::BlockPattern2d::dense(4);
  EXPECT(d2.is_active(2, 1) && !d2.is_active(1, 2) && d2.iter_cols(7, 3).size() == 3);
}

int main() {
  try {
    Context ctx(0);
    config_and_state_semantics();
    std::printf("inference_paths_run_across_configs\n");
    inference_paths_run_across_configs(ctx);
    std::printf("relu_lowrank_fused_matches_reference\n");
    relu_lowrank_fused_matches_reference(ctx);
    std::printf("fused_attention_matches_reference\n");
    fused_attention_matches_reference(ctx, RotaryEmbedding::Rope, 1337);
    fused_attention_matches_reference(ctx, RotaryEmbedding::Pope, 2024);
    // greedy generation runs and is deterministic
    BDHConfig config = build_config(RotaryEmbedding::Rope, false);
    config.n_embd = 16;
    std::mt19937 g(3);
    const size_t h = 2, d = 16, N = config.latent_per_head(), V = 32;
    BDHWeightsHost w{randn(g, V * d, 1.0f), randn(g, h * d * N, 0.02f), randn(g, h * d * N, 0.02f), randn(g, h * N * d, 0.02f),
                     randn(g, d * V, 0.02f)};
    BDH model(ctx, config, w);
    auto a = model.generate({1, 2, 3}, 5), b = model.generate({1, 2, 3}, 5);
    EXPECT(a.size() == 8 && a == b);
  } catch (const std::exception &e) {
    std::printf("FAIL exception: %s\n", e.what());
    return 2;
  }
  std::printf(failures ? "FAILED (%d)\n" : "OK\n", failures);
  return failures ? 1 : 0;
}
