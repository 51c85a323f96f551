// bdh_host.hpp — C++17 host-side mirror of the reference's interface for the BDH cached
// inference path, over the C ABI of libbdh_mi355x.so (include/bdh_mi355x.h).
//
// The reference is a Rust crate whose hot path sits behind generic functions over Burn tensors.
// This header gives the same names, argument meaning and error behaviour to a C++ caller:
//   positional::RotaryEmbedding            src/positional.rs:8-31
//   kernel::BlockPattern1d / 2d / Config   src/kernel/block_sparse.rs:11-133
//   kernel::relu_lowrank::fused_forward    src/kernel/relu_lowrank.rs:7-37
//   kernel::linear_attention::{fused_state_aligned, default_alibi_slopes}
//                                          src/kernel/linear_attention.rs:11-163
//   FusedKernelConfig, BDHConfig           src/model/config.rs:10-164
//   LayerState, ModelState                 src/model/state.rs:5-57
//   Attention::{new, forward, rotate_positions, alibi_decay}
//   BDH::{new, init_state, forward_with_state, forward, forward_fast, generate}
//                                          src/model/bdh.rs:37-84, 91-94, 170-256, 309-450
//   ModelOverrides, build_model_config     src/config/core.rs:43-53, src/inference.rs:4-40
// Contract violations that panic in the reference throw std::logic_error here; failures of the
// library throw bdh::Error with the text of bdh_last_error().  Tensors are plain device buffers
// with a shape; all computation happens in the library's HIP kernels.
#pragma once

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <memory>
#include <optional>
#include <set>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/bdh_mi355x.h"

namespace bdh {

struct Error : std::runtime_error {
  int status;
  Error(int s, const std::string &what) : std::runtime_error("bdh status " + std::to_string(s) + ": " + what), status(s) {}
};

inline void hip_check(hipError_t e, const char *what) {
  if (e != hipSuccess) throw Error(BDH_E_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

// ---- context ------------------------------------------------------------------------
class Context {
 public:
  explicit Context(int device_id = 0, hipStream_t stream = nullptr) {
    int rc = bdh_ctx_create(device_id, stream, &ctx_);
    if (rc != BDH_OK) throw Error(rc, std::string("bdh_ctx_create: ") + bdh_status_string(rc));
  }
  ~Context() { bdh_ctx_destroy(ctx_); }
  Context(const Context &) = delete;
  Context &operator=(const Context &) = delete;
  bdh_ctx *raw() const { return ctx_; }
  void check(int rc) const {
    if (rc != BDH_OK) throw Error(rc, bdh_last_error(ctx_));
  }
  void synchronize() const { check(bdh_ctx_synchronize(ctx_)); }

 private:
  bdh_ctx *ctx_ = nullptr;
};

// ---- a device tensor: shape + owned f32 buffer ----------------------------------------
class Tensor {
 public:
  Tensor() = default;
  explicit Tensor(std::vector<size_t> shape) : shape_(std::move(shape)) {
    size_t n = numel();
    if (n) hip_check(hipMalloc(reinterpret_cast<void **>(&data_), n * sizeof(float)), "hipMalloc");
  }
  static Tensor zeros(std::vector<size_t> shape) {
    Tensor t(std::move(shape));
    if (t.numel()) hip_check(hipMemset(t.data_, 0, t.numel() * sizeof(float)), "hipMemset");
    return t;
  }
  static Tensor from_host(const std::vector<float> &v, std::vector<size_t> shape) {
    Tensor t(std::move(shape));
    if (t.numel() != v.size()) throw std::logic_error("from_host: element count does not match the shape");
    if (t.numel()) hip_check(hipMemcpy(t.data_, v.data(), v.size() * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy");
    return t;
  }
  Tensor(Tensor &&o) noexcept : shape_(std::move(o.shape_)), data_(o.data_) { o.data_ = nullptr; }
  Tensor &operator=(Tensor &&o) noexcept {
    if (this != &o) {
      release();
      shape_ = std::move(o.shape_);
      data_ = o.data_;
      o.data_ = nullptr;
    }
    return *this;
  }
  Tensor(const Tensor &) = delete;
  Tensor &operator=(const Tensor &) = delete;
  ~Tensor() { release(); }

  const std::vector<size_t> &shape() const { return shape_; }
  size_t dim(size_t i) const { return shape_.at(i); }
  size_t numel() const {
    size_t n = shape_.empty() ? 0 : 1;
    for (size_t s : shape_) n *= s;
    return n;
  }
  float *data() const { return data_; }
  std::vector<float> to_host() const {
    std::vector<float> v(numel());
    if (!v.empty()) hip_check(hipMemcpy(v.data(), data_, v.size() * sizeof(float), hipMemcpyDeviceToHost), "hipMemcpy");
    return v;
  }

 private:
  void release() {
    if (data_) (void)hipFree(data_);
    data_ = nullptr;
  }
  std::vector<size_t> shape_;
  float *data_ = nullptr;
};

// ---- positional -------------------------------------------------------------------
enum class RotaryEmbedding : int { Rope = BDH_ROPE, Alibi = BDH_ALIBI, Pope = BDH_POPE };
inline const char *as_str(RotaryEmbedding r) {
  return r == RotaryEmbedding::Rope ? "rope" : (r == RotaryEmbedding::Pope ? "pope" : "alibi");
}

// ---- kernel::block_sparse ---------------------------------------------------------
namespace kernel {

class BlockPattern1d {
 public:
  static BlockPattern1d dense(size_t block_size) { return BlockPattern1d(std::max<size_t>(block_size, 1), std::nullopt); }
  static BlockPattern1d from_blocks(size_t block_size, std::set<size_t> blocks) {
    return BlockPattern1d(block_size, std::move(blocks));
  }
  size_t block_size() const { return block_size_; }
  bool is_sparse() const { return active_.has_value(); }
  bool is_block_active(size_t b) const { return !active_ || active_->count(b) > 0; }
  std::vector<uint8_t> block_bytes(size_t elements) const {
    const size_t bs = std::max<size_t>(block_size_, 1), total = (elements + bs - 1) / bs;
    std::vector<uint8_t> v(total);
    for (size_t i = 0; i < total; ++i) v[i] = is_block_active(i) ? 1 : 0;
    return v;
  }

 private:
  BlockPattern1d(size_t bs, std::optional<std::set<size_t>> a) : block_size_(bs), active_(std::move(a)) {}
  size_t block_size_;
  std::optional<std::set<size_t>> active_;
};

class BlockPattern2d {
 public:
  static BlockPattern2d dense(size_t block_size) { return BlockPattern2d(std::max<size_t>(block_size, 1), std::nullopt); }
  static BlockPattern2d from_pairs(size_t block_size, std::set<std::pair<size_t, size_t>> pairs) {
    return BlockPattern2d(block_size, std::move(pairs));
  }
  size_t block_size() const { return block_size_; }
  bool is_sparse() const { return pairs_.has_value(); }
  bool is_active(size_t row, size_t col) const { return pairs_ ? pairs_->count({row, col}) > 0 : col <= row; }
  std::vector<size_t> iter_cols(size_t row, size_t total_blocks) const {
    std::vector<size_t> cols;
    if (pairs_) {
      for (auto &p : *pairs_)
        if (p.first == row && p.second < total_blocks) cols.push_back(p.second);
    } else if (total_blocks > 0) {
      for (size_t c = 0; c <= std::min(row, total_blocks - 1); ++c) cols.push_back(c);
    }
    return cols;
  }
  std::vector<int32_t> pair_list() const {
    std::vector<int32_t> v;
    if (pairs_)
      for (auto &p : *pairs_) {
        v.push_back((int32_t)p.first);
        v.push_back((int32_t)p.second);
      }
    return v;
  }

 private:
  BlockPattern2d(size_t bs, std::optional<std::set<std::pair<size_t, size_t>>> p) : block_size_(bs), pairs_(std::move(p)) {}
  size_t block_size_;
  std::optional<std::set<std::pair<size_t, size_t>>> pairs_;
};

struct BlockSparseConfig {
  BlockPattern1d latent = BlockPattern1d::dense(64);
  BlockPattern2d time = BlockPattern2d::dense(64);
  static BlockSparseConfig dense(size_t latent_block, size_t time_block) {
    return BlockSparseConfig{BlockPattern1d::dense(latent_block), BlockPattern2d::dense(time_block)};
  }
};

namespace relu_lowrank {
// input [B,1|h,T,d], weight [1,h,d,N] (or [h,d,N]), bias [h,1,N] or null -> [B,h,T,N]
inline Tensor fused_forward(const Context &ctx, const Tensor &input, const Tensor &weight, const Tensor *bias,
                            float threshold, const BlockPattern1d &layout) {
  if (input.shape().size() != 4) throw std::logic_error("fused_forward: input must have 4 dims");
  const size_t wd = weight.shape().size();
  if (wd != 3 && !(wd == 4 && weight.dim(0) == 1)) throw std::logic_error("fused_forward: weight must be [1,h,d,N]");
  const size_t o = wd - 3;
  const int B = (int)input.dim(0), h_in = (int)input.dim(1), T = (int)input.dim(2), d = (int)input.dim(3);
  const int h = (int)weight.dim(o), dw = (int)weight.dim(o + 1), N = (int)weight.dim(o + 2);
  if (d != dw) throw std::logic_error("fused_forward: inner dimensions differ");
  Tensor out({(size_t)B, (size_t)h, (size_t)T, (size_t)N});
  std::vector<uint8_t> blocks;
  if (layout.is_sparse()) blocks = layout.block_bytes(N);
  ctx.check(bdh_relu_lowrank(ctx.raw(), B, h_in, T, d, h, N, input.data(), weight.data(), bias ? bias->data() : nullptr,
                             threshold, (int)std::max<size_t>(layout.block_size(), 1),
                             layout.is_sparse() ? blocks.data() : nullptr, (int)blocks.size(), nullptr, out.data()));
  return out;
}
}  // namespace relu_lowrank

namespace linear_attention {
inline std::vector<float> default_alibi_slopes(size_t n_head) {
  std::vector<float> v(n_head);
  int rc = bdh_default_alibi_slopes((int)n_head, v.data());
  if (rc != BDH_OK) throw Error(rc, "bdh_default_alibi_slopes");
  return v;
}
inline std::vector<float> build_freqs(size_t latent, float theta, RotaryEmbedding rotary) {
  std::vector<float> v(latent);
  int rc = bdh_build_freqs((int)latent, theta, (int)rotary, v.data());
  if (rc != BDH_OK) throw Error(rc, "bdh_build_freqs");
  return v;
}
// query [B,h,T,N], value [B,1,T,dv], freqs [1,1,1,N] -> [B,h,T,dv]
inline Tensor fused_state_aligned(const Context &ctx, const Tensor &query, const Tensor &value, const Tensor &freqs,
                                  const std::vector<float> *alibi_slopes, const BlockPattern2d &layout,
                                  RotaryEmbedding rotary_embedding) {
  const int B = (int)query.dim(0), h = (int)query.dim(1), T = (int)query.dim(2), N = (int)query.dim(3);
  const int dv = (int)value.dim(3);
  Tensor out({(size_t)B, (size_t)h, (size_t)T, (size_t)dv});
  const std::vector<int32_t> pairs = layout.pair_list();
  ctx.check(bdh_fused_state_aligned(ctx.raw(), B, h, T, N, dv, query.data(), value.data(), freqs.data(),
                                    alibi_slopes ? alibi_slopes->data() : nullptr,
                                    (int)std::max<size_t>(layout.block_size(), 1),
                                    layout.is_sparse() ? pairs.data() : nullptr, (int)(pairs.size() / 2),
                                    (int)rotary_embedding, 1, out.data()));
  return out;
}
}  // namespace linear_attention
}  // namespace kernel

// ---- model::config ------------------------------------------------------------------
struct FusedKernelConfig {
  bool enabled = false;
  kernel::BlockSparseConfig block_sparse = kernel::BlockSparseConfig::dense(64, 64);
  float rope_theta = 65536.0f;
  float relu_threshold = 0.0f;
  std::optional<std::vector<float>> alibi_slopes;
  RotaryEmbedding rotary_embedding = RotaryEmbedding::Alibi;  // the reference's default
  void set_block_sizes(size_t latent, size_t time) { block_sparse = kernel::BlockSparseConfig::dense(latent, time); }
  void set_alibi_slopes(std::vector<float> s) { alibi_slopes = std::move(s); }
  void set_rotary_embedding(RotaryEmbedding r) { rotary_embedding = r; }
};

struct BDHConfig {
  size_t n_layer = 6, n_embd = 256;
  double dropout = 0.1;
  size_t n_head = 4, mlp_internal_dim_multiplier = 4, n_expert = 1, vocab_size = 256;
  FusedKernelConfig fused_kernels;
  size_t latent_per_head() const {
    const size_t total = mlp_internal_dim_multiplier * n_embd;
    if (n_head == 0 || total % n_head != 0) throw std::logic_error("latent size must be divisible by the number of heads");
    const size_t l = total / n_head;
    if (n_expert == 0 || l % n_expert != 0) throw std::logic_error("latent per head must be divisible by experts");
    return l;
  }
  size_t latent_total() const { return latent_per_head() * n_head; }
  size_t latent_per_expert() const { return latent_per_head() / n_expert; }
};

struct ModelOverrides {
  std::optional<size_t> n_layer, n_embd, n_head, mlp_internal_dim_multiplier, block_size;
  std::optional<float> relu_threshold;
  std::optional<double> dropout;
  std::optional<bool> fused_kernels;
  std::optional<RotaryEmbedding> rotary_embedding;
};

inline BDHConfig build_model_config(const ModelOverrides &o, size_t training_block_size) {
  BDHConfig c;
  if (o.n_layer) c.n_layer = *o.n_layer;
  if (o.n_embd) c.n_embd = *o.n_embd;
  if (o.n_head) c.n_head = *o.n_head;
  if (o.mlp_internal_dim_multiplier) c.mlp_internal_dim_multiplier = *o.mlp_internal_dim_multiplier;
  if (o.relu_threshold) c.fused_kernels.relu_threshold = *o.relu_threshold;
  if (o.dropout) c.dropout = *o.dropout;
  if (o.fused_kernels) c.fused_kernels.enabled = *o.fused_kernels;
  const size_t block = std::max<size_t>(o.block_size.value_or(training_block_size), 1);
  c.fused_kernels.set_block_sizes(block, block);
  if (o.rotary_embedding) c.fused_kernels.set_rotary_embedding(*o.rotary_embedding);
  return c;
}

// ---- model::Attention (src/model/attention.rs:102-349) ---------------------------------
class Attention {
 public:
  Attention(size_t latent, size_t n_head, const FusedKernelConfig &kernel)
      : n_head_(n_head), fused_(kernel.enabled), block_pattern_(kernel.block_sparse.time),
        use_alibi_(kernel.rotary_embedding == RotaryEmbedding::Alibi), rotary_embedding_(kernel.rotary_embedding) {
    freqs_ = Tensor::from_host(kernel::linear_attention::build_freqs(latent, kernel.rope_theta, kernel.rotary_embedding),
                               {1, 1, 1, latent});
    if (use_alibi_)
      alibi_slopes_ = kernel.alibi_slopes ? *kernel.alibi_slopes : kernel::linear_attention::default_alibi_slopes(n_head);
    else
      alibi_slopes_.assign(n_head, 0.0f);  // zeros when ALiBi is off, as the reference stores them
  }

  // :142-175  query [B,h,T,N], value [B,1,T,dv] -> [B,h,T,dv].  The plain branch masks with tril(-1)
  // element-wise: the fused computation with time blocks of one token.
  Tensor forward(const Context &ctx, const Tensor &query, const Tensor &value) const {
    const kernel::BlockPattern2d plain = kernel::BlockPattern2d::dense(1);
    return kernel::linear_attention::fused_state_aligned(ctx, query, value, freqs_, use_alibi_ ? &alibi_slopes_ : nullptr,
                                                         fused_ ? block_pattern_ : plain, rotary_embedding_);
  }

  // :177-179, :332-349  values [B,h,T,N] at positions start..start+T -> [B,h,T,N] (PoPE: 2N columns)
  Tensor rotate_positions(const Context &ctx, const Tensor &values, size_t start) const {
    const size_t B = values.dim(0), h = values.dim(1), T = values.dim(2), N = values.dim(3);
    Tensor out({B, h, T, rotary_embedding_ == RotaryEmbedding::Pope ? 2 * N : N});
    ctx.check(bdh_rotate(ctx.raw(), (int)B, (int)h, (int)T, (int)N, (int)rotary_embedding_, values.data(), freqs_.data(),
                         (int64_t)start, nullptr, out.data()));
    return out;
  }

  // :181-186  exp(-slopes), or nothing without ALiBi
  std::optional<std::vector<float>> alibi_decay() const {
    if (!use_alibi_) return std::nullopt;
    std::vector<float> d(alibi_slopes_.size());
    for (size_t i = 0; i < d.size(); ++i) d[i] = std::exp(-alibi_slopes_[i]);
    return d;
  }

  const std::vector<float> &alibi_slopes() const { return alibi_slopes_; }

 private:
  Tensor freqs_;
  size_t n_head_;
  bool fused_;
  kernel::BlockPattern2d block_pattern_;
  bool use_alibi_;
  std::vector<float> alibi_slopes_;
  RotaryEmbedding rotary_embedding_;
};

// ---- model::state ---------------------------------------------------------------------
// src/model/state.rs:17-24 (the reference's "viz" feature): [h,N] maps on the host
struct LayerVizState {
  std::vector<float> x_last, y_last, xy_last, rho_last;
};

struct LayerState {
  std::optional<Tensor> rho;  // [B,h,Nq,d]
  std::optional<LayerVizState> viz;
  std::optional<LayerVizState> take_viz() {  // src/model/state.rs:76-80
    std::optional<LayerVizState> out;
    out.swap(viz);
    return out;
  }
};

struct ModelState {
  std::vector<LayerState> layers;
  size_t position = 0;
  // one allocation [L,B,h,Nq,d] backs every layer (the library walks it with a fixed stride)
  std::optional<Tensor> storage;
  explicit ModelState(size_t num_layers) : layers(num_layers) {}
  void reset() {
    for (auto &l : layers) l.rho.reset();
    storage.reset();
    position = 0;
  }
  size_t len() const { return position; }
  bool is_empty() const { return position == 0; }
  void trim(size_t) {}  // a no-op in the reference (src/model/state.rs:55-57)
  std::vector<std::optional<LayerVizState>> take_viz() {  // src/model/state.rs:59-65
    std::vector<std::optional<LayerVizState>> out;
    for (auto &l : layers) out.push_back(l.take_viz());
    return out;
  }
  void clear_viz() {  // src/model/state.rs:67-72
    for (auto &l : layers) l.viz.reset();
  }
};

// ---- model::BDH -------------------------------------------------------------------------
struct BDHWeightsHost {  // record order of the reference module
  std::vector<float> embed, encoder, encoder_v, decoder, lm_head;
};

class BDH {
 public:
  // defer_updates = K > 0 (RoPE models with n_embd 256 or 512): single-token calls log their state updates and apply
  // them every K tokens (bdh_model_forward_deferred); flush_state(), and every call that is not such a step, bring
  // state.storage up to date first.  Logits and the flushed state agree with the eager step to f32 rounding (a layer
  // fed the same inputs leaves the same bits; the readouts that feed deeper layers are reassociated sums).
  BDH(const Context &ctx, const BDHConfig &config, const BDHWeightsHost &w, size_t defer_updates = 0)
      : ctx_(ctx), config_(config), defer_updates_(defer_updates) {
    const size_t h = config.n_head, d = config.n_embd, N = config.latent_per_head(), V = config.vocab_size;
    embed_ = Tensor::from_host(w.embed, {V, d});
    encoder_ = Tensor::from_host(w.encoder, {h, d, N});
    encoder_v_ = Tensor::from_host(w.encoder_v, {h, d, N});
    decoder_ = Tensor::from_host(w.decoder, {h * N, d});
    lm_head_ = Tensor::from_host(w.lm_head, {d, V});
    const auto &k = config.fused_kernels;
    bdh_model_config c{(int32_t)config.n_layer, (int32_t)d, (int32_t)h, (int32_t)N, (int32_t)V, (int32_t)k.rotary_embedding,
                       k.rope_theta, k.relu_threshold, k.alibi_slopes ? k.alibi_slopes->data() : nullptr};
    bdh_model_weights mw{embed_.data(), encoder_.data(), encoder_v_.data(), decoder_.data(), lm_head_.data()};
    ctx_.check(bdh_model_create(ctx_.raw(), &c, &mw, &model_));
  }
  ~BDH() {
    if (logs_) bdh_model_logs_destroy(model_, logs_);
    bdh_model_destroy(model_);
  }

  // applies the logged updates of a deferred state (no-op otherwise): afterwards state.storage is the reference's state
  void flush_state(ModelState &state) {
    if (logs_ && state.storage && bdh_model_logs_pending(logs_) > 0)
      ctx_.check(bdh_model_flush(model_, logs_, state.storage->data()));
  }
  BDH(const BDH &) = delete;
  BDH &operator=(const BDH &) = delete;

  ModelState init_state() const { return ModelState(config_.n_layer); }

  // tokens [B,T] (host, row-major) -> logits [B,T,V]
  // viz = true also fills every layer's LayerVizState (src/model/bdh.rs:386-434)
  Tensor forward_with_state(const std::vector<int64_t> &tokens, size_t batch, size_t time, ModelState &state,
                            std::vector<int64_t> *next_tokens = nullptr, bool viz = false) {
    if (state.layers.size() != config_.n_layer) throw std::logic_error("model state layers mismatch");
    if (tokens.size() != batch * time) throw std::logic_error("tokens do not match [batch, time]");
    const size_t h = config_.n_head, d = config_.n_embd, N = config_.latent_per_head();
    const size_t Nq = config_.fused_kernels.rotary_embedding == RotaryEmbedding::Pope ? 2 * N : N;
    const std::vector<size_t> want{config_.n_layer, batch, h, Nq, d};
    if (!state.storage || state.storage->shape() != want) {  // bdh.rs:274-284
      drop_logs();  // pending updates belong to the storage that is replaced
      state.storage = Tensor::zeros(want);
    }
    const bool deferred = defer_updates_ > 0 && time == 1 && !viz && batch > 0;
    if (deferred && (!logs_ || logs_batch_ != batch)) {
      flush_state(state);
      drop_logs();
      ctx_.check(bdh_model_logs_create(model_, (int)batch, BDH_F32, (int)defer_updates_, &logs_));
      logs_batch_ = batch;
    }
    if (!deferred) flush_state(state);
    int64_t *tok_dev = nullptr, *next_dev = nullptr;
    hip_check(hipMalloc(reinterpret_cast<void **>(&tok_dev), sizeof(int64_t) * std::max<size_t>(tokens.size(), 1)), "hipMalloc");
    hip_check(hipMalloc(reinterpret_cast<void **>(&next_dev), sizeof(int64_t) * std::max<size_t>(batch, 1)), "hipMalloc");
    Tensor logits({batch, time, config_.vocab_size});
    int rc = BDH_OK;
    if (!tokens.empty()) {
      hip_check(hipMemcpy(tok_dev, tokens.data(), sizeof(int64_t) * tokens.size(), hipMemcpyHostToDevice), "hipMemcpy");
      std::optional<Tensor> maps;
      if (viz) maps.emplace(std::vector<size_t>{config_.n_layer, 4, h, N});
      if (deferred)
        rc = bdh_model_forward_deferred(model_, logs_, tok_dev, (int)batch, state.storage->data(), BDH_F32,
                                        (int64_t)state.position, nullptr, logits.data(), next_tokens ? next_dev : nullptr);
      else
        rc = bdh_model_forward_viz(model_, tok_dev, (int)batch, (int)time, state.storage->data(), BDH_F32, nullptr,
                                   (int64_t)state.position, nullptr, logits.data(), next_tokens ? next_dev : nullptr,
                                   nullptr, maps ? maps->data() : nullptr);
      if (rc == BDH_OK && maps) {
        ctx_.synchronize();
        const std::vector<float> host = maps->to_host();
        const size_t hn = h * N;
        for (size_t l = 0; l < config_.n_layer; ++l) {
          const float *p = host.data() + l * 4 * hn;
          state.layers[l].viz = LayerVizState{{p, p + hn}, {p + hn, p + 2 * hn}, {p + 2 * hn, p + 3 * hn},
                                              {p + 3 * hn, p + 4 * hn}};
        }
      }
    }
    if (rc == BDH_OK && next_tokens && batch > 0 && time > 0) {
      next_tokens->resize(batch);
      ctx_.synchronize();
      hip_check(hipMemcpy(next_tokens->data(), next_dev, sizeof(int64_t) * batch, hipMemcpyDeviceToHost), "hipMemcpy");
    } else {
      ctx_.synchronize();
    }
    (void)hipFree(tok_dev);
    (void)hipFree(next_dev);
    ctx_.check(rc);
    state.position = state.position > SIZE_MAX - time ? SIZE_MAX : state.position + time;  // saturating_add
    return logits;
  }

  Tensor forward(const std::vector<int64_t> &tokens, size_t batch, size_t time) {
    ModelState st = init_state();
    return forward_with_state(tokens, batch, time, st);
  }

  // BDH::forward_fast (src/model/bdh.rs:96-168): the stateless forward over all tokens at once
  Tensor forward_fast(const std::vector<int64_t> &tokens, size_t batch, size_t time) {
    if (tokens.size() != batch * time) throw std::logic_error("tokens do not match [batch, time]");
    const auto &k = config_.fused_kernels;
    if (k.enabled && (k.block_sparse.latent.is_sparse() || k.block_sparse.time.is_sparse()))
      throw std::logic_error("forward_fast takes dense block patterns");
    Tensor logits({batch, time, config_.vocab_size});
    if (tokens.empty()) return logits;
    int64_t *tok_dev = nullptr;
    hip_check(hipMalloc(reinterpret_cast<void **>(&tok_dev), sizeof(int64_t) * tokens.size()), "hipMalloc");
    hip_check(hipMemcpy(tok_dev, tokens.data(), sizeof(int64_t) * tokens.size(), hipMemcpyHostToDevice), "hipMemcpy");
    const int block = k.enabled ? (int)std::max<size_t>(k.block_sparse.time.block_size(), 1) : 0;
    const int rc = bdh_model_forward_fast(model_, tok_dev, (int)batch, (int)time, block, logits.data());
    ctx_.synchronize();
    (void)hipFree(tok_dev);
    ctx_.check(rc);
    return logits;
  }

  // greedy form (top_k = 1) of BDH::generate; batch must be 1 as in the reference
  std::vector<int64_t> generate(std::vector<int64_t> indices, size_t max_new_tokens) {
    ModelState st = init_state();
    std::vector<int64_t> next;
    forward_with_state(indices, 1, indices.size(), st, &next);
    for (size_t i = 0; i < max_new_tokens; ++i) {
      indices.push_back(next[0]);
      forward_with_state({next[0]}, 1, 1, st, &next);
    }
    return indices;
  }

  const BDHConfig &config() const { return config_; }

 private:
  void drop_logs() {
    if (logs_) bdh_model_logs_destroy(model_, logs_);
    logs_ = nullptr;
    logs_batch_ = 0;
  }

  const Context &ctx_;
  BDHConfig config_;
  Tensor embed_, encoder_, encoder_v_, decoder_, lm_head_;
  bdh_model *model_ = nullptr;
  size_t defer_updates_ = 0;
  bdh_model_logs *logs_ = nullptr;  // one update log per layer, for a batch of logs_batch_ sequences
  size_t logs_batch_ = 0;
};

}  // namespace bdh
