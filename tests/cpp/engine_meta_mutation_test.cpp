// Host-only robustness check of the sidecar reader (forward_amd/csrc/plugins/engine_meta.cpp): feeds
// it a few hundred thousand seeded mutations of valid sidecars (bytes flipped, cut, repeated,
// structural characters and escapes spliced in, deep nesting, huge numbers) and asserts that it
// either accepts the text or refuses it with a reason, that what it accepts survives a round trip
// through its own writer unchanged, and that nothing trips the address / undefined-behaviour
// sanitizers this file is built with by tests/test_engine_meta.py.
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "../../forward_amd/csrc/plugins/engine_meta.h"
#include "../../include/fwdmi.h"

using fwdmi::EngineMetaData;

static int g_failures = 0;
static long g_accepted = 0, g_refused = 0;

static void fail(const char* what, const std::string& text) {
  std::fprintf(stderr, "FAIL: %s on input of %zu bytes: %.200s\n", what, text.size(), text.c_str());
  ++g_failures;
}

static void feed(const std::string& text) {
  EngineMetaData m;
  if (!m.ParseMetaData(text)) {
    ++g_refused;
    if (fwdmi_last_error()[0] == '\0') fail("refused without a reason", text);
    return;
  }
  ++g_accepted;
  const std::string once = m.ToJson();
  EngineMetaData again;
  if (!again.ParseMetaData(once)) return fail("the writer's own text is refused", text);
  if (again.ToJson() != once) fail("round trip through the writer changes the text", text);
  if (again.Mode() != m.Mode() || again.OptBatchSize() != m.OptBatchSize() || again.MaxBatchSize() != m.MaxBatchSize() ||
      again.TorchModulePath() != m.TorchModulePath() || again.UnusedInputIndices() != m.UnusedInputIndices() ||
      again.OutputPositions() != m.OutputPositions())
    fail("round trip through the writer changes a member", text);
}

int main() {
  std::vector<std::string> seeds;
  {
    EngineMetaData m;
    seeds.push_back(m.ToJson());
    m.SetMode(fwdmi::InferMode::HALF);
    m.SetOptBatchSize(16);
    m.SetMaxBatchSize(64);
    m.SetUnusedInputIndices({0, 3, 7});
    m.SetOutputPositions({2, 1, 0, 5});
    m.SetTorchModulePath("models/\"dlrm\"\\v2/\xc3\xa9\t.pth");
    seeds.push_back(m.ToJson());
  }
  seeds.push_back("{\"infer_mode\":1,\"opt_batch_size\":1e1,\"max_batch_size\":2.0,\"torch_module_path\":\"\\ud83d\\ude00\","
                  "\"extra\":{\"a\":[1,[2,{\"b\":null}],true,false,-0.5e-3]},\"output_indices\":[],\"unused_input_indices\":[4,4]}");
  for (const std::string& s : seeds) feed(s);
  if (g_accepted != (long)seeds.size()) fail("a valid sidecar is refused", "");

  static const char* const kSplices[] = {"{", "}", "[", "]", ",", ":", "\"", "\\", "\\u", "\\ud800", "\\udc00", "-", "+", ".",
                                         "e", "E", "0", "9", "99999999999999999999", "1e999", "-2147483649", "2147483648",
                                         "null", "true", "false", "nul", " ", "\n", "\t", "\x01", "\x7f", "\xff", "\xc3",
                                         "\"infer_mode\"", "\"output_indices\"", "[[[[[[[[", "{\"a\":"};
  const int n_splices = (int)(sizeof(kSplices) / sizeof(kSplices[0]));
  std::mt19937_64 rng(20240607);
  auto uni = [&](size_t lo, size_t hi) { return std::uniform_int_distribution<size_t>(lo, hi)(rng); };
  for (int it = 0; it < 300000; ++it) {
    std::string t = seeds[uni(0, seeds.size() - 1)];
    const int edits = (int)uni(1, 4);
    for (int e = 0; e < edits && !t.empty(); ++e) {
      const size_t at = uni(0, t.size() - 1);
      switch (uni(0, 6)) {
        case 0: t[at] = (char)uni(0, 255); break;                                     // a byte replaced
        case 1: t.erase(at, uni(1, 8)); break;                                        // a piece cut out
        case 2: t.resize(at); break;                                                  // truncated
        case 3: t.insert(at, kSplices[uni(0, (size_t)n_splices - 1)]); break;         // a token spliced in
        case 4: t.insert(at, t.substr(at, uni(1, 40))); break;                        // a piece repeated
        case 5: t[at] ^= (char)(1u << uni(0, 7)); break;                              // a bit flipped
        default: std::swap(t[at], t[uni(0, t.size() - 1)]); break;                    // two bytes swapped
      }
    }
    feed(t);
  }
  // nesting far beyond any depth limit, open and closed
  for (const char* open : {"[", "{\"a\":"}) {
    std::string deep = "{\"infer_mode\":0,\"opt_batch_size\":1,\"max_batch_size\":1,\"torch_module_path\":\"\",\"x\":";
    for (int i = 0; i < 200000; ++i) deep += open;
    feed(deep);
    deep += "1";
    for (int i = 0; i < 200000; ++i) deep += open[0] == '[' ? "]" : "}";
    feed(deep + "}");
  }
  std::printf("%ld texts accepted, %ld refused, %d failures\n", g_accepted, g_refused, g_failures);
  return g_failures ? 1 : 0;
}
