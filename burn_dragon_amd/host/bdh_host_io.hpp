// bdh_host_io.hpp — the callers either side of the model step, for a C++ host:
//   tokenizer::{Tokenizer, ByteTokenizer, CharVocab}   src/tokenizer/mod.rs:17-27, byte.rs, char_vocab.rs
//   record::{load_record, parse_record}                BinFileRecorder files, src/bin/infer.rs:177-186
//   generation::{GenerationSettings, prefill_state, sample_next_token, generate_tokens, generate_text, bdh_generate}
//                                                      src/generation.rs:12-260
// Everything here is host logic over bdh_host.hpp; the draw of the next token happens on the device
// (bdh_sample_top_k), so only one uniform variate goes up and one token comes down per step.
#pragma once

#include <cstdio>
#include <fstream>
#include <functional>
#include <map>
#include <random>
#include <sstream>

#include "bdh_host.hpp"

namespace bdh {

// ---- tokenizer ------------------------------------------------------------------------
namespace tokenizer {

class Tokenizer {  // src/tokenizer/mod.rs:17-27
 public:
  virtual ~Tokenizer() = default;
  virtual std::vector<uint32_t> encode(const std::string &text, bool add_bos, bool add_eos) const = 0;
  virtual std::string decode(const std::vector<uint32_t> &ids) const = 0;
  virtual size_t len() const = 0;
  bool is_empty() const { return len() == 0; }
  virtual std::optional<uint32_t> bos_id() const = 0;
  virtual std::optional<uint32_t> eos_id() const = 0;
  virtual std::optional<uint32_t> pad_id() const = 0;
  virtual std::optional<uint32_t> unk_id() const = 0;
};

class ByteTokenizer : public Tokenizer {  // src/tokenizer/byte.rs
 public:
  explicit ByteTokenizer(bool add_special_tokens) {
    if (add_special_tokens) {
      bos_ = 256;
      eos_ = 257;
      pad_ = 258;
      vocab_ = 259;
    }
  }
  std::vector<uint32_t> encode(const std::string &text, bool add_bos, bool add_eos) const override {
    std::vector<uint32_t> t;
    if (add_bos && bos_) t.push_back(*bos_);
    for (unsigned char c : text) t.push_back(c);
    if (add_eos && eos_) t.push_back(*eos_);
    return t;
  }
  std::string decode(const std::vector<uint32_t> &ids) const override {  // invalid utf-8 is passed through
    std::string out;
    for (uint32_t id : ids) {
      if ((pad_ && id == *pad_) || (bos_ && id == *bos_)) continue;
      if (eos_ && id == *eos_) break;
      if (id < 256) out.push_back((char)id);
    }
    return out;
  }
  size_t len() const override { return vocab_; }
  std::optional<uint32_t> bos_id() const override { return bos_; }
  std::optional<uint32_t> eos_id() const override { return eos_; }
  std::optional<uint32_t> pad_id() const override { return pad_; }
  std::optional<uint32_t> unk_id() const override { return std::nullopt; }

 private:
  std::optional<uint32_t> bos_, eos_, pad_;
  size_t vocab_ = 256;
};

namespace detail {
inline void append_utf8(std::string &s, uint32_t cp) {
  if (cp < 0x80) {
    s.push_back((char)cp);
  } else if (cp < 0x800) {
    s.push_back((char)(0xC0 | (cp >> 6)));
    s.push_back((char)(0x80 | (cp & 0x3F)));
  } else if (cp < 0x10000) {
    s.push_back((char)(0xE0 | (cp >> 12)));
    s.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
    s.push_back((char)(0x80 | (cp & 0x3F)));
  } else {
    s.push_back((char)(0xF0 | (cp >> 18)));
    s.push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
    s.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
    s.push_back((char)(0x80 | (cp & 0x3F)));
  }
}
// decodes one code point starting at s[i]; advances i
inline uint32_t next_code_point(const std::string &s, size_t &i) {
  const unsigned char c = (unsigned char)s[i];
  int extra = c < 0x80 ? 0 : (c >> 5) == 6 ? 1 : (c >> 4) == 14 ? 2 : (c >> 3) == 30 ? 3 : -1;
  if (extra < 0 || i + extra >= s.size() + (extra == 0)) {
    ++i;
    return 0xFFFD;
  }
  uint32_t cp = extra == 0 ? c : c & (0x3F >> extra);
  for (int k = 1; k <= extra; ++k) cp = (cp << 6) | ((unsigned char)s[i + k] & 0x3F);
  i += extra + 1;
  return cp;
}
}  // namespace detail

class CharVocab : public Tokenizer {  // src/tokenizer/char_vocab.rs
 public:
  static constexpr uint32_t PAD = 0, BOS = 1, EOS = 2, UNK = 3;  // the code points U+0000..U+0003
  CharVocab(std::vector<uint32_t> chars, bool include_unknown) {  // from_chars :47-88
    if (chars.empty()) throw std::invalid_argument("vocabulary cannot be empty");
    for (size_t i = 0; i < chars.size(); ++i)
      if (!ch2id_.emplace(chars[i], (uint32_t)i).second) throw std::invalid_argument("duplicate character");
    id2ch_ = std::move(chars);
    auto need = [&](uint32_t cp, const char *name) {
      auto it = ch2id_.find(cp);
      if (it == ch2id_.end()) throw std::invalid_argument(std::string("missing ") + name + " character in vocabulary");
      return it->second;
    };
    bos_ = need(BOS, "BOS");
    eos_ = need(EOS, "EOS");
    pad_ = need(PAD, "PAD");
    if (include_unknown) {
      auto it = ch2id_.find(UNK);
      if (it != ch2id_.end()) unk_ = it->second;
    }
  }
  static CharVocab fit(const std::vector<std::string> &texts, bool include_unknown) {  // :28-45
    std::vector<uint32_t> chars{PAD, BOS, EOS};
    if (include_unknown) chars.push_back(UNK);
    std::set<uint32_t> seen(chars.begin(), chars.end());
    for (const auto &t : texts)
      for (size_t i = 0; i < t.size();) {
        const uint32_t cp = detail::next_code_point(t, i);
        if (seen.insert(cp).second) chars.push_back(cp);
      }
    return CharVocab(std::move(chars), include_unknown);
  }
  // {"chars": ["a", "\u0001", ...], "bos": 1, "eos": 2, "pad": 0, "unk": 3 | null}   (:232-240)
  static CharVocab from_json_str(const std::string &json) {
    std::vector<uint32_t> chars;
    size_t p = json.find("\"chars\"");
    if (p == std::string::npos) throw std::invalid_argument("failed to parse vocabulary json: no chars");
    p = json.find('[', p);
    const size_t end = p == std::string::npos ? p : json.find(']', p);
    if (end == std::string::npos) throw std::invalid_argument("failed to parse vocabulary json: chars is not a list");
    for (size_t i = p + 1; i < end;) {
      if (json[i] != '"') {
        ++i;
        continue;
      }
      ++i;
      uint32_t cp;
      if (json[i] == '\\') {
        const char e = json[i + 1];
        if (e == 'u') {
          cp = (uint32_t)std::stoul(json.substr(i + 2, 4), nullptr, 16);
          i += 6;
          if (cp >= 0xD800 && cp < 0xDC00 && json.compare(i, 2, "\\u") == 0) {  // surrogate pair
            const uint32_t lo = (uint32_t)std::stoul(json.substr(i + 2, 4), nullptr, 16);
            cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
            i += 6;
          }
        } else {
          cp = e == 'n' ? '\n' : e == 't' ? '\t' : e == 'r' ? '\r' : e == 'b' ? '\b' : e == 'f' ? '\f' : (unsigned char)e;
          i += 2;
        }
      } else {
        cp = detail::next_code_point(json, i);
      }
      if (json[i] != '"') throw std::invalid_argument("failed to parse vocabulary json: entry is not one character");
      ++i;
      chars.push_back(cp);
    }
    auto field = [&](const char *name) -> std::optional<uint32_t> {
      size_t q = json.find(std::string("\"") + name + "\"", end);
      if (q == std::string::npos) return std::nullopt;
      q = json.find(':', q);
      while (++q < json.size() && (json[q] == ' ' || json[q] == '\n')) {
      }
      if (q >= json.size() || json.compare(q, 4, "null") == 0) return std::nullopt;
      return (uint32_t)std::stoul(json.substr(q));
    };
    const auto unk = field("unk");
    CharVocab v(std::move(chars), unk.has_value());
    if (auto b = field("bos")) v.bos_ = *b;  // the stored ids win over the derived ones (:100-110)
    if (auto e = field("eos")) v.eos_ = *e;
    if (auto pd = field("pad")) v.pad_ = *pd;
    v.unk_ = unk;
    return v;
  }
  static CharVocab load(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("failed to read vocabulary " + path);
    std::stringstream ss;
    ss << f.rdbuf();
    return from_json_str(ss.str());
  }
  std::vector<uint32_t> encode(const std::string &s, bool add_bos, bool add_eos) const override {  // :148-176
    std::vector<uint32_t> t;
    if (add_bos) t.push_back(bos_);
    for (size_t i = 0; i < s.size();) {
      const uint32_t cp = detail::next_code_point(s, i);
      auto it = ch2id_.find(cp);
      if (it != ch2id_.end()) {
        t.push_back(it->second);
      } else if (unk_) {
        t.push_back(*unk_);
      } else {
        throw std::out_of_range("character missing from vocabulary and no <unk> token configured");
      }
    }
    if (add_eos) t.push_back(eos_);
    return t;
  }
  std::string decode(const std::vector<uint32_t> &ids) const override {  // :178-203
    std::string text;
    for (uint32_t id : ids) {
      if (id >= id2ch_.size()) throw std::out_of_range("token id " + std::to_string(id) + " out of range");
      if (id == pad_ || id == bos_) continue;
      if (id == eos_) break;
      if (unk_ && id == *unk_) text.push_back('?');
      else detail::append_utf8(text, id2ch_[id]);
    }
    return text;
  }
  size_t len() const override { return id2ch_.size(); }
  bool contains(uint32_t cp) const { return ch2id_.count(cp) > 0; }
  std::optional<uint32_t> bos_id() const override { return bos_; }
  std::optional<uint32_t> eos_id() const override { return eos_; }
  std::optional<uint32_t> pad_id() const override { return pad_; }
  std::optional<uint32_t> unk_id() const override { return unk_; }

 private:
  std::vector<uint32_t> id2ch_;
  std::map<uint32_t, uint32_t> ch2id_;
  uint32_t bos_ = 0, eos_ = 0, pad_ = 0;
  std::optional<uint32_t> unk_;
};

}  // namespace tokenizer

// ---- record: Burn 0.19 BinFileRecorder files of the BDH module --------------------------
// bincode 2, little endian, varint lengths: five metadata strings, then the module's fields in order;
// a field that is not a parameter is one 0x00 byte; a parameter is {id string, {bytes, shape, dtype}}.
// The five parameters are identified by order and shape (embed, encoder, encoder_v, decoder, lm_head).
namespace record {

struct Metadata {
  std::string float_type, int_type, format, version, settings;
};
struct Param {
  std::string id;
  std::vector<size_t> shape;
  std::vector<float> data;
};
struct Loaded {
  Metadata meta;
  BDHWeightsHost weights;
  size_t vocab_size = 0, n_embd = 0, n_head = 0, latent_per_head = 0, mlp_internal_dim_multiplier = 0;
};

namespace detail {
struct Reader {
  const std::vector<unsigned char> &b;
  size_t off = 0;
  void need(size_t n) const {
    if (n > b.size() - off) throw std::runtime_error("truncated record at offset " + std::to_string(off));
  }
  uint64_t varint() {
    need(1);
    const unsigned char m = b[off++];
    if (m < 251) return m;
    const int n = m == 251 ? 2 : m == 252 ? 4 : m == 253 ? 8 : 0;
    if (!n) throw std::runtime_error("unsupported varint marker");
    need(n);
    uint64_t v = 0;
    for (int i = 0; i < n; ++i) v |= (uint64_t)b[off + i] << (8 * i);
    off += n;
    return v;
  }
  std::string string(size_t limit) {
    const uint64_t n = varint();
    if (n > limit) throw std::runtime_error("string too long at offset " + std::to_string(off));
    need(n);
    std::string s(b.begin() + off, b.begin() + off + n);
    off += n;
    return s;
  }
};
inline float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000) << 16, exp = (h >> 10) & 0x1F, man = h & 0x3FF;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else {
      int e = -1;
      uint32_t m = man;
      do {
        ++e;
        m <<= 1;
      } while (!(m & 0x400));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3FF) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7F800000u | (man << 13);
  } else {
    u = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
}  // namespace detail

inline std::pair<Metadata, std::vector<Param>> parse_record(const std::vector<unsigned char> &buf) {
  detail::Reader r{buf};
  Metadata m;
  m.float_type = r.string(4096);
  m.int_type = r.string(4096);
  m.format = r.string(4096);
  m.version = r.string(4096);
  m.settings = r.string(4096);
  if (m.format.find("BinFileRecorder") == std::string::npos && m.format.find("BinBytesRecorder") == std::string::npos)
    throw std::runtime_error("not a bincode recorder file: " + m.format);
  std::vector<Param> params;
  while (r.off < buf.size()) {
    if (buf[r.off] == 0) {  // ConstantRecord
      ++r.off;
      continue;
    }
    Param p;
    p.id = r.string(64);
    const uint64_t nbytes = r.varint();
    r.need(nbytes);
    const unsigned char *raw = buf.data() + r.off;
    r.off += nbytes;
    const uint64_t rank = r.varint();
    if (rank > 8) throw std::runtime_error("parameter rank " + std::to_string(rank));
    size_t count = 1;
    for (uint64_t i = 0; i < rank; ++i) {
      p.shape.push_back((size_t)r.varint());
      count *= p.shape.back();
    }
    const uint64_t dt = r.varint();  // burn-tensor DType: F64 0, F32 1, F16 3, BF16 4
    const size_t es = dt == 0 ? 8 : dt == 1 ? 4 : (dt == 3 || dt == 4) ? 2 : 0;
    if (!es) throw std::runtime_error("parameter dtype index " + std::to_string(dt) + " is not a float type");
    if (nbytes != es * count) throw std::runtime_error("parameter byte count does not match its shape");
    p.data.resize(count);
    for (size_t i = 0; i < count; ++i) {
      if (dt == 1) {
        std::memcpy(&p.data[i], raw + 4 * i, 4);
      } else if (dt == 0) {
        double d;
        std::memcpy(&d, raw + 8 * i, 8);
        p.data[i] = (float)d;
      } else {
        uint16_t h;
        std::memcpy(&h, raw + 2 * i, 2);
        if (dt == 3) {
          p.data[i] = detail::half_to_float(h);
        } else {
          const uint32_t u = (uint32_t)h << 16;
          std::memcpy(&p.data[i], &u, 4);
        }
      }
    }
    params.push_back(std::move(p));
  }
  return {m, std::move(params)};
}

inline Loaded load_record(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) {
    f.open(path + ".bin", std::ios::binary);  // the recorder appends the extension to a base name
    if (!f) throw std::runtime_error("failed to load checkpoint " + path);
  }
  std::vector<unsigned char> buf((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
  auto parsed = parse_record(buf);
  auto &ps = parsed.second;
  if (ps.size() != 5) throw std::runtime_error("expected 5 parameters, found " + std::to_string(ps.size()));
  if (ps[0].shape.size() != 2 || ps[1].shape.size() != 3 || ps[3].shape.size() != 2 || ps[4].shape.size() != 2)
    throw std::runtime_error("parameter ranks do not match the BDH module");
  Loaded out;
  out.meta = parsed.first;
  out.vocab_size = ps[0].shape[0];
  out.n_embd = ps[0].shape[1];
  out.n_head = ps[1].shape[0];
  out.latent_per_head = ps[1].shape[2];
  const size_t V = out.vocab_size, d = out.n_embd, h = out.n_head, N = out.latent_per_head;
  if (ps[1].shape[1] != d || ps[2].shape != ps[1].shape || ps[3].shape != std::vector<size_t>{h * N, d} ||
      ps[4].shape != std::vector<size_t>{d, V} || d == 0 || (h * N) % d)
    throw std::runtime_error("parameter shapes do not match the BDH module");
  out.mlp_internal_dim_multiplier = h * N / d;
  out.weights.embed = std::move(ps[0].data);
  out.weights.encoder = std::move(ps[1].data);
  out.weights.encoder_v = std::move(ps[2].data);
  out.weights.decoder = std::move(ps[3].data);
  out.weights.lm_head = std::move(ps[4].data);
  return out;
}

}  // namespace record

// ---- generation ---------------------------------------------------------------------------
namespace generation {

struct ContextStrategy {  // src/generation.rs:12-16
  std::optional<size_t> window;  // nullopt = Infinite
  static ContextStrategy infinite() { return {}; }
  static ContextStrategy sliding(size_t w) { return {w}; }
};

struct GenerationSettings {  // :18-24
  std::optional<size_t> max_new_tokens;
  float temperature = 1.0f;
  std::optional<size_t> top_k;
  ContextStrategy strategy;
};

struct GenerationConfig {  // src/config/core.rs:20-30
  std::string prompt;
  std::optional<int64_t> max_tokens;
  float temperature = 1.0f;
  std::optional<size_t> top_k;
  ContextStrategy context_strategy;
};

inline ContextStrategy resolve_context_strategy(const ContextStrategy &s, size_t default_window) {  // :243-259
  if (!s.window) return s;
  return ContextStrategy::sliding(*s.window == 0 ? std::max<size_t>(default_window, 1) : *s.window);
}
inline std::optional<size_t> normalize_max_tokens(std::optional<int64_t> m) {  // :236-241
  if (m && *m >= 0) return (size_t)*m;
  return std::nullopt;
}

// sample_from_logits_values after the temperature division (:26-72, :117), on the device.
// last_logits: device pointer to V floats; u in [0,1) replaces the draw from thread_rng.
inline int64_t sample_from_logits(const Context &ctx, const float *last_logits, size_t vocab, float temperature,
                                  std::optional<size_t> top_k, float u) {
  float *u_dev = nullptr;
  int64_t *tok_dev = nullptr;
  hip_check(hipMalloc(reinterpret_cast<void **>(&u_dev), sizeof(float)), "hipMalloc");
  hip_check(hipMalloc(reinterpret_cast<void **>(&tok_dev), sizeof(int64_t)), "hipMalloc");
  hip_check(hipMemcpy(u_dev, &u, sizeof(float), hipMemcpyHostToDevice), "hipMemcpy");
  const int rc = bdh_sample_top_k(ctx.raw(), 1, (int)vocab, last_logits, (int64_t)vocab, temperature,
                                  top_k ? (int)*top_k : 0, u_dev, tok_dev);
  int64_t tok = -1;
  if (rc == BDH_OK) {
    ctx.synchronize();
    hip_check(hipMemcpy(&tok, tok_dev, sizeof(int64_t), hipMemcpyDeviceToHost), "hipMemcpy");
  }
  (void)hipFree(u_dev);
  (void)hipFree(tok_dev);
  ctx.check(rc);
  return tok;
}

struct Prefilled {
  ModelState state;
  Tensor logits;  // [1, T, V]; the last row is the distribution of the next token
};

inline Prefilled prefill_state(BDH &model, const std::vector<int64_t> &prompt_tokens) {  // :74-105
  if (prompt_tokens.empty()) throw std::invalid_argument("prompt must contain at least one token");
  ModelState state = model.init_state();
  Tensor logits = model.forward_with_state(prompt_tokens, 1, prompt_tokens.size(), state);
  if (logits.dim(1) != prompt_tokens.size()) throw std::runtime_error("prefill produced mismatched length");
  return {std::move(state), std::move(logits)};
}

// :107-128 — draws from the last row of `logits`, feeds the token, returns it; `logits` is replaced
inline int64_t sample_next_token(const Context &ctx, BDH &model, ModelState &state, Tensor &logits, float temperature,
                                 std::optional<size_t> top_k, float u) {
  const size_t T = logits.dim(1), V = logits.dim(2);
  const int64_t next = sample_from_logits(ctx, logits.data() + (T - 1) * V, V, temperature, top_k, u);
  logits = model.forward_with_state({next}, 1, 1, state);
  return next;
}

// BDH::generate (src/model/bdh.rs:170-252): the prompt, then max_new_tokens draws from
// softmax(logits / temperature) over the top_k values; rng supplies the uniform variates the reference
// takes from thread_rng.  Batch size 1, as in the reference.
template <typename Rng>
std::vector<int64_t> bdh_generate(const Context &ctx, BDH &model, std::vector<int64_t> indices, size_t max_new_tokens,
                                  float temperature, std::optional<size_t> top_k, Rng &rng) {
  if (indices.empty()) throw std::invalid_argument("generate needs at least one prompt token");
  ModelState state = model.init_state();
  Tensor logits = model.forward_with_state(indices, 1, indices.size(), state);
  std::uniform_real_distribution<float> uniform(0.0f, 1.0f);
  for (size_t i = 0; i < max_new_tokens; ++i) {
    float u = uniform(rng);
    if (u >= 1.0f) u = std::nextafter(1.0f, 0.0f);  // some library versions round up to the bound
    indices.push_back(sample_next_token(ctx, model, state, logits, temperature, top_k, u));
  }
  return indices;
}

template <typename Rng>
std::vector<int64_t> generate_tokens(const Context &ctx, BDH &model, std::vector<int64_t> prompt_tokens,
                                     const GenerationSettings &settings, Rng &rng,
                                     const std::function<bool(int64_t)> &on_token = nullptr) {  // :158-203
  if (!settings.max_new_tokens && !on_token)
    throw std::invalid_argument("an unbounded generation needs an on_token callback that eventually returns false");
  std::vector<int64_t> full = std::move(prompt_tokens);
  Prefilled p = prefill_state(model, full);
  const auto window = settings.strategy.window;
  if (window && *window > 0 && p.state.position > *window) p.state.trim(*window);
  std::uniform_real_distribution<float> uni(0.0f, 1.0f);
  size_t generated = 0;
  while (!settings.max_new_tokens || generated < *settings.max_new_tokens) {
    const int64_t next = sample_next_token(ctx, model, p.state, p.logits, settings.temperature, settings.top_k, uni(rng));
    full.push_back(next);
    ++generated;
    if (on_token && !on_token(next)) break;  // the callback may end an unbounded run
    if (window && *window > 0 && p.state.position > *window) p.state.trim(*window);
  }
  return full;
}

template <typename Rng>
std::string generate_text(const Context &ctx, BDH &model, const tokenizer::Tokenizer &tok, size_t block_size,
                          const GenerationConfig &g, Rng &rng) {  // :205-234
  const ContextStrategy strategy = resolve_context_strategy(g.context_strategy, block_size);
  std::vector<uint32_t> ids = tok.encode(g.prompt, false, false);
  if (strategy.window && ids.size() > *strategy.window) ids.erase(ids.begin(), ids.end() - *strategy.window);
  std::vector<int64_t> prompt(ids.begin(), ids.end());
  GenerationSettings s{normalize_max_tokens(g.max_tokens), g.temperature, g.top_k, strategy};
  const std::vector<int64_t> all = generate_tokens(ctx, model, std::move(prompt), s, rng);
  std::vector<uint32_t> decoded;
  for (int64_t t : all)
    if (t >= 0) decoded.push_back((uint32_t)t);
  return tok.decode(decoded);
}

}  // namespace generation
}  // namespace bdh
