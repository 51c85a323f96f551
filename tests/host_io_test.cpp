// CPU-only test of the host-side C++ helpers (burn_dragon_amd/host/bdh_host_io.hpp): the record reader on the
// checkpoint the reference ships (argv[1] = tests/golden/tiny_shakespeare) and on damaged copies of it, and the
// tokenizers.  Built with -fsanitize=address,undefined by tests/test_host_io_cpp.py; touches no GPU entry point.
#include <cstdio>

#include "../burn_dragon_amd/host/bdh_host_io.hpp"

using namespace bdh;

static int failures = 0;
#define EXPECT(cond)                                                  \
  do {                                                                \
    if (!(cond)) {                                                    \
      std::printf("FAIL %s:%d  %s\n", __FILE__, __LINE__, #cond);     \
      ++failures;                                                     \
    }                                                                 \
  } while (0)

int main(int argc, char **argv) {
  if (argc < 2) return 2;
  const std::string dir = argv[1];
  record::Loaded rec = record::load_record(dir + "/model.bin");
  EXPECT(rec.meta.float_type == "f32" && rec.meta.version == "0.19.1");
  EXPECT(rec.vocab_size == 69 && rec.n_embd == 128 && rec.n_head == 4 && rec.latent_per_head == 128);
  EXPECT(rec.weights.embed.size() == 69u * 128 && rec.weights.decoder.size() == 512u * 128);
  EXPECT(record::load_record(dir + "/model").vocab_size == 69);  // base name, as the recorder takes it

  std::ifstream f(dir + "/model.bin", std::ios::binary);
  std::vector<unsigned char> buf((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
  // every truncation either throws or yields fewer than five complete parameters; never reads out of bounds
  size_t threw = 0, cuts = 0;
  for (size_t n = 0; n < buf.size(); n += 997) {
    std::vector<unsigned char> cut(buf.begin(), buf.begin() + n);
    ++cuts;
    try {
      auto parsed = record::parse_record(cut);
      EXPECT(parsed.second.size() < 5);
    } catch (const std::runtime_error &) {
      ++threw;
    }
  }
  EXPECT(threw > cuts / 2);
  // flipped bytes in the framing (not in the float payload) are rejected or parsed, never a crash
  for (size_t pos : {0u, 3u, 7u, 100u, 135u, 149u, 150u, 151u}) {
    std::vector<unsigned char> bad(buf);
    bad[pos] ^= 0xFF;
    try {
      (void)record::parse_record(bad);
    } catch (const std::runtime_error &) {
    }
  }

  using namespace tokenizer;
  CharVocab tok = CharVocab::load(dir + "/vocab.json");
  EXPECT(tok.len() == 69 && *tok.bos_id() == 1 && *tok.eos_id() == 2 && *tok.pad_id() == 0 && *tok.unk_id() == 3);
  const std::string text = "First Citizen:\nBefore we proceed any further, hear me speak.\n";
  EXPECT(tok.decode(tok.encode(text, true, true)) == text);
  EXPECT(tok.decode(tok.encode("café", false, false)) == "caf?");
  bool threw_range = false;
  try {
    (void)tok.decode({1000});
  } catch (const std::out_of_range &) {
    threw_range = true;
  }
  EXPECT(threw_range);
  ByteTokenizer bt(false);
  EXPECT(bt.len() == 256 && bt.decode(bt.encode("héllo", true, true)) == "héllo");
  CharVocab fitted = CharVocab::fit({"éè", "\U0001F600x"}, true);
  EXPECT(fitted.len() == 4 + 4 && fitted.decode(fitted.encode("x\U0001F600è", false, false)) == "x\U0001F600è");
  bool threw_json = false;
  try {
    (void)CharVocab::from_json_str("{\"bos\": 1}");
  } catch (const std::invalid_argument &) {
    threw_json = true;
  }
  EXPECT(threw_json);

  using namespace generation;
  EXPECT(!resolve_context_strategy(ContextStrategy::infinite(), 7).window.has_value());
  EXPECT(*resolve_context_strategy(ContextStrategy::sliding(0), 7).window == 7);
  EXPECT(*resolve_context_strategy(ContextStrategy::sliding(3), 7).window == 3);
  EXPECT(!normalize_max_tokens(-1).has_value() && *normalize_max_tokens(5) == 5 && !normalize_max_tokens(std::nullopt));

  std::printf(failures ? "FAILED (%d)\n" : "OK\n", failures);
  return failures ? 1 : 0;
}
