// Host-only robustness check of everything that reads engine bytes: every plugin's
// deserializePlugin and the plan-file loader are fed seeded mutations of valid blobs and files
// (bytes replaced, bits flipped, pieces cut, repeated or truncated, size fields set to extreme
// values) and must answer each with NULL and a reason, or with an object that serializes, clones
// and destroys cleanly.  Then the kernel launchers are called with arguments at the ends of their
// types: without a device each call must return a status.  tests/test_plugin_host.py builds this file and the library's host code with
// the address / undefined-behaviour sanitizers; no GPU is touched (nothing is configured or enqueued).
#include <unistd.h>

#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "../../include/fwdmi.h"

static int g_failures = 0;
static long g_alive = 0, g_refused = 0;

#define CHECK(cond, ...)                                               \
  do {                                                                 \
    if (!(cond)) {                                                     \
      std::fprintf(stderr, "FAIL %s:%d: %s: ", __FILE__, __LINE__, #cond); \
      std::fprintf(stderr, __VA_ARGS__);                               \
      std::fprintf(stderr, "\n");                                      \
      ++g_failures;                                                    \
    }                                                                  \
  } while (0)

static std::mt19937_64 g_rng(77001);
static size_t uni(size_t lo, size_t hi) { return std::uniform_int_distribution<size_t>(lo, hi)(g_rng); }

static void mutate(std::vector<char>* t) {
  static const uint64_t kExtremes[] = {0, 1, 0x7fffffffu, 0x80000000u, 0xffffffffu, 0x100000000ull, 0x7fffffffffffffffull,
                                       0x8000000000000000ull, 0xffffffffffffffffull, 0xfffffffffffffffeull, 1ull << 40};
  const int edits = (int)uni(1, 3);
  for (int e = 0; e < edits && !t->empty(); ++e) {
    const size_t at = uni(0, t->size() - 1);
    switch (uni(0, 6)) {
      case 0: (*t)[at] = (char)uni(0, 255); break;
      case 1: (*t)[at] ^= (char)(1u << uni(0, 7)); break;
      case 2: t->erase(t->begin() + (long)at, t->begin() + (long)std::min(t->size(), at + uni(1, 16))); break;
      case 3: t->resize(at); break;
      case 4: {  // a piece repeated
        const size_t n = std::min(t->size() - at, uni(1, 64));
        const std::vector<char> piece(t->begin() + (long)at, t->begin() + (long)(at + n));
        t->insert(t->begin() + (long)at, piece.begin(), piece.end());
        break;
      }
      case 5: {  // a 4- or 8-byte field (headers are packed ints and size_t counts) set to an extreme value
        const size_t w = uni(0, 1) ? 4 : 8, a = std::min(at, t->size() >= w ? t->size() - w : 0) & ~(size_t)3;
        const uint64_t v = kExtremes[uni(0, sizeof(kExtremes) / sizeof(kExtremes[0]) - 1)];
        if (a + w <= t->size()) std::memcpy(t->data() + a, &v, w);
        break;
      }
      default: {  // the same, near the start, where the headers are
        const size_t a = (uni(0, 15) * 4);
        const uint32_t v = (uint32_t)kExtremes[uni(0, 4)];
        if (a + 4 <= t->size()) std::memcpy(t->data() + a, &v, 4);
        break;
      }
    }
  }
}

// A plugin that came out of damaged bytes must still behave as an object.
static void exercise(fwdmi_plugin* p) {
  const size_t n = fwdmi_plugin_get_serialization_size(p);
  CHECK(n < ((size_t)1 << 28), "serialization size %zu", n);
  if (n < ((size_t)1 << 28)) {
    std::vector<char> out(n);  // exact size: a write past it is seen
    CHECK(fwdmi_plugin_serialize(p, out.data()) == FWDMI_OK, "serialize: %s", fwdmi_last_error());
  }
  CHECK(fwdmi_plugin_get_nb_outputs(p) >= 1, "outputs");
  CHECK(fwdmi_plugin_get_type(p) != nullptr && fwdmi_plugin_get_version(p) != nullptr, "type / version");
  fwdmi_plugin* c = fwdmi_plugin_clone(p);
  if (c) {
    CHECK(fwdmi_plugin_get_serialization_size(c) == n, "a clone serializes to another size");
    fwdmi_plugin_destroy(c);
  }
}

struct Made {
  const char* name;
  const char* version;
  fwdmi_plugin* plugin;
};

int main() {
  std::vector<float> gamma(16, 1.0f), beta(16, 0.25f), word(5 * 16, 0.25f), pos(4 * 16, 0.5f), tok(2 * 16, 0.125f);
  std::vector<float> table(6 * 8, 0.5f), g_rows(8 * 4, 0.5f);
  const int dim = 8, count = 6, offset = 0, op = 0, ld = 16, f16 = FWDMI_F16, one = 1, g_dim = 4, g_counts[3] = {2, 5, 1};
  const int i64 = FWDMI_I64;
  const fwdmi_plugin_field bag[] = {{"dim", &dim, FWDMI_FIELD_I32, 1}, {"count", &count, FWDMI_FIELD_I32, 1},
                                    {"offset", &offset, FWDMI_FIELD_I32, 1}, {"op", &op, FWDMI_FIELD_I32, 1},
                                    {"data", table.data(), FWDMI_FIELD_F32, 48}};
  const fwdmi_plugin_field bag2[] = {bag[0], bag[1], bag[2], bag[3], bag[4], {"index_type", &i64, FWDMI_FIELD_I32, 1},
                                     {"output_fp16", &one, FWDMI_FIELD_I32, 1}, {"include_last_offset", &one, FWDMI_FIELD_I32, 1},
                                     {"per_sample_weights", &one, FWDMI_FIELD_I32, 1}};
  const fwdmi_plugin_field group[] = {{"dim", &g_dim, FWDMI_FIELD_I32, 1}, {"op", &op, FWDMI_FIELD_I32, 1},
                                      {"count", g_counts, FWDMI_FIELD_I32, 3}, {"data", g_rows.data(), FWDMI_FIELD_F32, 32},
                                      {"per_sample_weights", &one, FWDMI_FIELD_I32, 1}};
  const fwdmi_plugin_field ln[] = {{"ld", &ld, FWDMI_FIELD_I32, 1}, {"type_id", &f16, FWDMI_FIELD_I32, 1},
                                   {"beta", beta.data(), FWDMI_FIELD_F32, 16}, {"gamma", gamma.data(), FWDMI_FIELD_F32, 16},
                                   {"bias", beta.data(), FWDMI_FIELD_F32, 16}};
  const float eps = 1e-5f;
  const fwdmi_plugin_field emb[] = {{"bert_embeddings_layernorm_beta", beta.data(), FWDMI_FIELD_F32, 16},
                                    {"bert_embeddings_layernorm_gamma", gamma.data(), FWDMI_FIELD_F32, 16},
                                    {"bert_embeddings_word_embeddings", word.data(), FWDMI_FIELD_F32, 80},
                                    {"bert_embeddings_token_type_embeddings", tok.data(), FWDMI_FIELD_F32, 32},
                                    {"bert_embeddings_position_embeddings", pos.data(), FWDMI_FIELD_F32, 64},
                                    {"output_fp16", &one, FWDMI_FIELD_I32, 1}, {"mha_type_id", &f16, FWDMI_FIELD_I32, 1},
                                    // the SkipLayerNorm the plugin can also stand for
                                    {"skip_beta", beta.data(), FWDMI_FIELD_F32, 16}, {"skip_gamma", gamma.data(), FWDMI_FIELD_F32, 16},
                                    {"skip_bias", beta.data(), FWDMI_FIELD_F32, 16}, {"skip_eps", &eps, FWDMI_FIELD_F32, 1}};
  struct Recipe {
    const char* name;
    const char* version;
    const fwdmi_plugin_field* fields;
    int n;
  } recipes[] = {{"EmbeddingBag_TRT", "001", bag, 5},
                 {"EmbeddingBag_TRT", "002", bag2, 9},
                 {"EmbeddingBagGroup_TRT", "001", group, 5},
                 {"ForwardLayerNormPluginDynamic", "1", ln, 5},
                 {"CustomSkipLayerNormPluginDynamic", "1", ln, 5},
                 {"CustomEmbLayerNormPluginDynamic", "1", emb, 7},
                 {"CustomEmbLayerNormPluginDynamic", "1", emb, 11}};

  std::vector<Made> made;
  for (const Recipe& r : recipes) {
    fwdmi_creator* cr = fwdmi_get_plugin_creator(r.name, r.version);
    CHECK(cr != nullptr, "%s/%s is not registered", r.name, r.version);
    if (!cr) return 1;
    fwdmi_plugin* p = fwdmi_creator_create_plugin(cr, "layer", r.fields, r.n);
    CHECK(p != nullptr, "%s/%s: %s", r.name, r.version, fwdmi_last_error());
    if (!p) return 1;
    made.push_back({r.name, r.version, p});
    std::vector<char> good(fwdmi_plugin_get_serialization_size(p));
    CHECK(fwdmi_plugin_serialize(p, good.data()) == FWDMI_OK, "serialize");
    fwdmi_plugin* again = fwdmi_creator_deserialize_plugin(cr, "layer", good.data(), good.size());
    CHECK(again != nullptr && fwdmi_plugin_get_serialization_size(again) == good.size(), "%s: its own blob", r.name);
    if (again) fwdmi_plugin_destroy(again);
    for (size_t n = 0; n < good.size(); ++n) {  // every truncation, from an exact-size heap copy
      std::vector<char> cut(good.begin(), good.begin() + (long)n);
      fwdmi_plugin* q = fwdmi_creator_deserialize_plugin(cr, "layer", cut.data(), cut.size());
      if (q) exercise(q), fwdmi_plugin_destroy(q), ++g_alive;
      else ++g_refused;
    }
    for (int trial = 0; trial < 30000; ++trial) {
      std::vector<char> bad(good);
      mutate(&bad);
      std::vector<char> exact(bad.begin(), bad.end());
      fwdmi_plugin* q = fwdmi_creator_deserialize_plugin(cr, "layer", exact.data(), exact.size());
      if (q) {
        exercise(q);
        fwdmi_plugin_destroy(q);
        ++g_alive;
      } else {
        CHECK(fwdmi_last_error()[0] != '\0', "%s: refused without a reason", r.name);
        ++g_refused;
      }
    }
  }

  // ---- shape, format and type queries with arguments no builder would send -----------------------
  // Everything here is host code of a plugin that was never configured: it must answer (or refuse)
  // without reading past its arguments or overflowing on the way.
  {
    const int32_t ds[] = {-1, 0, 1, 2, 5, 16, 128, 65536, 1 << 30, INT32_MAX, INT32_MIN};
    const int32_t ts[] = {FWDMI_F32, FWDMI_F16, FWDMI_I8, FWDMI_I32, FWDMI_BOOL, FWDMI_I64, -1, 1000};
    auto pick_d = [&]() { return ds[uni(0, sizeof(ds) / sizeof(ds[0]) - 1)]; };
    auto pick_t = [&]() { return ts[uni(0, sizeof(ts) / sizeof(ts[0]) - 1)]; };
    long answered = 0;
    for (const Made& m : made) {
      for (int it = 0; it < 20000; ++it) {
        fwdmi_dims in[8];
        fwdmi_tensor_desc io[12];
        for (auto& d : in) {
          d.nbDims = uni(0, 9) ? (int32_t)uni(0, 8) : pick_d();
          for (auto& v : d.d) v = uni(0, 2) ? (int32_t)uni(1, 64) : pick_d();
        }
        for (auto& t : io) {
          t.dims = in[uni(0, 7)];
          t.type = pick_t();
          t.format = uni(0, 5) ? FWDMI_FORMAT_LINEAR : pick_d();
          t.scale = 1.0f;
        }
        const int nb_in = uni(0, 9) ? (int)uni(0, 6) : pick_d(), nb_out = uni(0, 9) ? (int)uni(0, 3) : pick_d();
        fwdmi_dims out{};
        // counts beyond the arrays above are only sent where the callee looks at the count first
        const int in_ok = nb_in >= 0 && nb_in <= 8 ? nb_in : 0, out_ok = nb_out >= 0 && nb_out <= 4 ? nb_out : 0;
        (void)fwdmi_plugin_get_output_dimensions(m.plugin, uni(0, 5) ? (int)uni(0, 2) : pick_d(), in, in_ok, &out);
        (void)fwdmi_plugin_get_output_dimensions(m.plugin, 0, uni(0, 9) ? in : nullptr, in_ok, uni(0, 9) ? &out : nullptr);
        (void)fwdmi_plugin_supports_format_combination(m.plugin, uni(0, 5) ? (int)uni(0, 6) : pick_d(), io, in_ok, out_ok);
        (void)fwdmi_plugin_get_workspace_size(m.plugin, io, in_ok, io + in_ok, out_ok);
        int32_t types[8];
        for (auto& t : types) t = pick_t();
        (void)fwdmi_plugin_get_output_data_type(m.plugin, uni(0, 5) ? (int)uni(0, 2) : pick_d(), types, in_ok);
        const void* ins[8] = {};
        void* outs[4] = {};
        const int rc = fwdmi_plugin_enqueue(m.plugin, io, io + in_ok, ins, outs, nullptr, nullptr);
        CHECK(rc < 0, "%s: enqueue on a plugin that was never configured returned %d", m.name, rc);
        ++answered;
      }
    }
    std::printf("%ld rounds of shape / format / type queries answered\n", answered);
  }

  // ---- null handles: a status, NULL or an empty answer, never a dereference -------------------------
  {
    fwdmi_dims d{};
    fwdmi_tensor_desc t{};
    int32_t ty = 0;
    const int32_t* arr = nullptr;
    CHECK(fwdmi_get_plugin_creator(nullptr, nullptr) == nullptr, "creator of no name");
    CHECK(fwdmi_get_plugin_creator("EmbeddingBag_TRT", nullptr) == nullptr, "creator of no version");
    CHECK(fwdmi_registry_at(-1) == nullptr && fwdmi_registry_at(fwdmi_registry_size()) == nullptr, "registry index");
    (void)fwdmi_creator_name(nullptr), (void)fwdmi_creator_version(nullptr), (void)fwdmi_creator_num_fields(nullptr);
    (void)fwdmi_creator_field_name(nullptr, 0), (void)fwdmi_creator_field_type(nullptr, 0);
    fwdmi_creator* cr = fwdmi_get_plugin_creator("EmbeddingBag_TRT", "001");
    (void)fwdmi_creator_field_name(cr, -1), (void)fwdmi_creator_field_name(cr, 1000), (void)fwdmi_creator_field_type(cr, -1);
    CHECK(fwdmi_creator_create_plugin(nullptr, "x", nullptr, 0) == nullptr, "plugin of no creator");
    CHECK(fwdmi_creator_create_plugin(cr, nullptr, nullptr, 5) == nullptr, "plugin of no fields");
    CHECK(fwdmi_creator_deserialize_plugin(nullptr, "x", "abc", 3) == nullptr, "blob for no creator");
    CHECK(fwdmi_creator_deserialize_plugin(cr, "x", nullptr, 100) == nullptr, "no blob");
    CHECK(fwdmi_plugin_get_nb_outputs(nullptr) < 0, "outputs of no plugin");
    CHECK(fwdmi_plugin_get_output_dimensions(nullptr, 0, &d, 1, &d) < 0, "dims of no plugin");
    CHECK(fwdmi_plugin_supports_format_combination(nullptr, 0, &t, 1, 1) <= 0, "formats of no plugin");
    CHECK(fwdmi_plugin_configure(nullptr, &t, 1, &t, 1) < 0, "configure no plugin");
    (void)fwdmi_plugin_get_workspace_size(nullptr, &t, 1, &t, 1);
    CHECK(fwdmi_plugin_initialize(nullptr) < 0, "initialize no plugin");
    fwdmi_plugin_terminate(nullptr);
    CHECK(fwdmi_plugin_enqueue(nullptr, &t, &t, nullptr, nullptr, nullptr, nullptr) < 0, "enqueue no plugin");
    (void)fwdmi_plugin_get_serialization_size(nullptr);
    CHECK(fwdmi_plugin_serialize(nullptr, &d) < 0, "serialize no plugin");
    CHECK(fwdmi_plugin_serialize(made[0].plugin, nullptr) < 0, "serialize into nothing");
    (void)fwdmi_plugin_get_type(nullptr), (void)fwdmi_plugin_get_version(nullptr), (void)fwdmi_plugin_get_namespace(nullptr);
    fwdmi_plugin_set_namespace(nullptr, "x");
    fwdmi_plugin_set_namespace(made[0].plugin, nullptr);
    CHECK(fwdmi_plugin_get_output_data_type(nullptr, 0, &ty, 1) < 0, "type of no plugin");
    CHECK(fwdmi_plugin_clone(nullptr) == nullptr, "clone of no plugin");
    fwdmi_plugin_destroy(nullptr);
    CHECK(fwdmi_plugin_take_oob_flag(nullptr, nullptr) < 0, "flag of no plugin");
    CHECK(fwdmi_plan_save(nullptr, nullptr, nullptr, 0, nullptr) < 0, "plan without a path");
    CHECK(fwdmi_plan_save("/tmp/fwdmi_never_written.plan", nullptr, nullptr, 3, nullptr) < 0, "plan of no plugins");
    CHECK(fwdmi_plan_load(nullptr) == nullptr, "plan of no path");
    CHECK(fwdmi_plan_size(nullptr) <= 0, "size of no plan");
    (void)fwdmi_plan_layer_name(nullptr, 0);
    CHECK(fwdmi_plan_take_plugin(nullptr, 0) == nullptr, "plugin of no plan");
    (void)fwdmi_plan_meta(nullptr);
    CHECK(fwdmi_plan_meta_data(nullptr) == nullptr, "sidecar of no plan");
    fwdmi_plan_close(nullptr);
    CHECK(fwdmi_meta_load(nullptr) == nullptr && fwdmi_meta_parse(nullptr) == nullptr, "sidecar of nothing");
    CHECK(fwdmi_meta_save(nullptr, "/tmp/x") < 0, "save no sidecar");
    (void)fwdmi_meta_json(nullptr), (void)fwdmi_meta_infer_mode(nullptr), (void)fwdmi_meta_opt_batch_size(nullptr);
    (void)fwdmi_meta_max_batch_size(nullptr), (void)fwdmi_meta_torch_module_path(nullptr);
    (void)fwdmi_meta_unused_input_indices(nullptr, &arr), (void)fwdmi_meta_output_indices(nullptr, nullptr);
    CHECK(fwdmi_meta_set(nullptr, 0, 1, 1, nullptr, 0, nullptr, 0, nullptr) < 0, "set no sidecar");
    fwdmi_meta* m = fwdmi_meta_new();
    CHECK(m != nullptr, "a new sidecar");
    if (m) {
      CHECK(fwdmi_meta_set(m, 0, 1, 1, nullptr, 3, nullptr, 0, nullptr) < 0, "three indices from no array");
      CHECK(fwdmi_meta_set(m, 0, 1, 1, nullptr, -1, nullptr, -1, nullptr) < 0, "negative counts");
      CHECK(fwdmi_meta_save(m, nullptr) < 0, "save to no path");
      fwdmi_meta_free(m);
    }
    fwdmi_meta_free(nullptr);
    int32_t cus = 0;
    (void)fwdmi_bag_device_topology(nullptr, nullptr), (void)fwdmi_bag_device_topology(&cus, nullptr);
    CHECK(fwdmi_bag_tables_fill(nullptr, 3, nullptr, nullptr) < 0, "fill from nothing");
    CHECK(fwdmi_bag_table_cost(nullptr, 3, nullptr) < 0, "cost of nothing");
  }

  // ---- plan files -----------------------------------------------------------------------------
  char dir[] = "/tmp/fwdmi_mutation_XXXXXX";
  CHECK(mkdtemp(dir) != nullptr, "mkdtemp");
  const std::string path = std::string(dir) + "/engine.plan", bad_path = std::string(dir) + "/damaged.plan";
  std::vector<fwdmi_plugin*> handles;
  std::vector<const char*> names;
  static const char* const kNames[] = {"bag", "bag2", "group", "ln", "skip_ln", "emb", "emb_skip"};
  for (size_t i = 0; i < made.size(); ++i) handles.push_back(made[i].plugin), names.push_back(kNames[i]);
  const char* meta = "{\"infer_mode\":1,\"opt_batch_size\":8,\"max_batch_size\":32,\"torch_module_path\":\"m.pth\","
                     "\"unused_input_indices\":[1],\"output_indices\":[0,2]}";
  CHECK(fwdmi_plan_save(path.c_str(), handles.data(), names.data(), (int)handles.size(), meta) == FWDMI_OK, "save: %s",
        fwdmi_last_error());
  std::vector<char> file;
  {
    FILE* f = std::fopen(path.c_str(), "rb");
    CHECK(f != nullptr, "open the saved plan");
    if (f) {
      char buf[4096];
      size_t n;
      while ((n = std::fread(buf, 1, sizeof buf, f)) > 0) file.insert(file.end(), buf, buf + n);
      std::fclose(f);
    }
  }
  auto load_and_walk = [&](const std::string& where) {
    fwdmi_plan* plan = fwdmi_plan_load(where.c_str());
    if (!plan) {
      CHECK(fwdmi_last_error()[0] != '\0', "plan refused without a reason");
      ++g_refused;
      return false;
    }
    ++g_alive;
    const int n = fwdmi_plan_size(plan);
    CHECK(n >= 0 && n < 100000, "plan of %d entries", n);
    for (int i = 0; i < n && i < 64; ++i) {
      CHECK(fwdmi_plan_layer_name(plan, i) != nullptr, "layer name %d", i);
      fwdmi_plugin* p = fwdmi_plan_take_plugin(plan, i);
      if (p) exercise(p), fwdmi_plugin_destroy(p);
      CHECK(fwdmi_plan_take_plugin(plan, i) == nullptr, "entry %d handed out twice", i);
    }
    CHECK(fwdmi_plan_meta(plan) != nullptr, "meta text");
    fwdmi_meta* m = fwdmi_plan_meta_data(plan);
    if (m) fwdmi_meta_free(m);
    fwdmi_plan_close(plan);
    return true;
  };
  CHECK(load_and_walk(path), "the saved plan does not load: %s", fwdmi_last_error());
  // the sidecar of the damaged copies: sometimes the good one, sometimes damaged, sometimes none
  std::vector<char> meta_file;
  {
    FILE* f = std::fopen((path + ".meta").c_str(), "rb");
    CHECK(f != nullptr, "the sidecar was not written");
    if (f) {
      char buf[4096];
      size_t n;
      while ((n = std::fread(buf, 1, sizeof buf, f)) > 0) meta_file.insert(meta_file.end(), buf, buf + n);
      std::fclose(f);
    }
  }
  auto write_file = [](const std::string& where, const std::vector<char>& bytes) {
    FILE* f = std::fopen(where.c_str(), "wb");
    if (!f) return false;
    const bool ok = bytes.empty() || std::fwrite(bytes.data(), 1, bytes.size(), f) == bytes.size();
    return std::fclose(f) == 0 && ok;
  };
  for (int trial = 0; trial < 6000; ++trial) {
    std::vector<char> bad(file);
    if (trial % 3 != 2) mutate(&bad);
    CHECK(write_file(bad_path, bad), "write the damaged plan");
    const int kind = trial % 3;
    if (kind == 0) {
      CHECK(write_file(bad_path + ".meta", meta_file), "write the sidecar");
    } else if (kind == 1) {
      std::remove((bad_path + ".meta").c_str());
    } else {
      std::vector<char> bad_meta(meta_file);
      mutate(&bad_meta);
      CHECK(write_file(bad_path + ".meta", bad_meta), "write the damaged sidecar");
    }
    load_and_walk(bad_path);
  }
  std::remove(bad_path.c_str());
  std::remove((bad_path + ".meta").c_str());
  std::remove(path.c_str());
  std::remove((path + ".meta").c_str());
  rmdir(dir);
  for (const Made& m : made) fwdmi_plugin_destroy(m.plugin);

  // ---- launchers with arguments at the ends of their types ---------------------------------------
  // Without a device every launcher must come back with a status: its argument checks and sizing
  // arithmetic run on the host before anything is enqueued, and the sanitizers see them.  (With a
  // device present this part is skipped: the pointers below are not device memory.)
  long statuses = 0, nothing_to_do = 0;
  if (fwdmi_device_count() == 0) {
    alignas(16) static char mem[256];
    const int64_t big[] = {-1, 0, 1, 7, 768, 1024, 65536, 2147483647, 2147483648ll, (int64_t)1 << 40, (int64_t)1 << 62, INT64_MAX};
    const int32_t small[] = {-1, 0, 1, 2, 8, 128, 768, 1024, 16384, 1 << 24, 1 << 30, INT32_MAX};
    const int32_t types[] = {FWDMI_F32, FWDMI_F16, FWDMI_F32, FWDMI_F16, FWDMI_I8, FWDMI_I32, FWDMI_I64, -1, 99};
    const int32_t ops[] = {0, 1, 2, 3, 0, 999, -1, 12345};
    const float epss[] = {0.0f, 1e-12f, 1e-5f, -1.0f, 3e38f, -3e38f};
#define PICK(a) a[uni(0, sizeof(a) / sizeof(a[0]) - 1)]
    auto ptr = [&]() -> void* { return uni(0, 7) ? (void*)mem : nullptr; };
    for (int it = 0; it < 100000; ++it) {
      int rc = 1;
      fwdmi_bag_ext x{};
      x.table_dtype = PICK(types), x.index_dtype = uni(0, 2) ? (uni(0, 1) ? FWDMI_I32 : FWDMI_I64) : PICK(types);
      x.out_dtype = PICK(types), x.include_last_offset = (int32_t)uni(0, 1), x.out_row_stride = uni(0, 2) ? 0 : PICK(big);
      x.flags = (int32_t)uni(0, 7) & ~FWDMI_BAG_TABLE_AVG_LEN;
      x.per_sample_weights = uni(0, 5) ? nullptr : mem, x.max_indices = uni(0, 5) ? nullptr : mem;
      x.square_sum_out = uni(0, 5) ? nullptr : mem, x.oob_flag = uni(0, 3) ? nullptr : (int32_t*)mem;
      const fwdmi_bag_ext* xp = uni(0, 4) ? &x : nullptr;
      bool empty_work = false;  // FWDMI_OK is the answer to a call that has nothing to do: no launch, no device needed
      const int64_t n0 = PICK(big), n1 = PICK(big), n2 = PICK(big), n3 = PICK(big);
      const int32_t s0 = PICK(small), s1 = PICK(small), s2 = PICK(small);
      switch (uni(0, 8)) {
        case 0: rc = fwdmi_layer_norm(nullptr, s0, n0, ptr(), (float*)ptr(), (float*)ptr(), ptr(), (float*)ptr(),
                                      PICK(types), PICK(epss));
                empty_work = n0 == 0;
                break;
        case 1: rc = fwdmi_skip_layer_norm(nullptr, s0, n0, ptr(), ptr(), (float*)ptr(), (float*)ptr(), ptr(),
                                           (float*)ptr(), PICK(types), PICK(epss));
                empty_work = n0 == 0;
                break;
        case 2: {
          fwdmi_emb_ext e{(int32_t)uni(0, 1), PICK(epss), ptr(), (float*)ptr(), (float*)ptr(), (float*)ptr(), ptr()};
          rc = fwdmi_emb_layer_norm_ex(nullptr, s0, s1, s2, (int32_t*)ptr(), (int32_t*)ptr(),
                                       (int32_t*)ptr(), (float*)ptr(), (float*)ptr(), ptr(), ptr(), ptr(), PICK(small), PICK(small),
                                       PICK(small), ptr(), (int32_t*)ptr(), PICK(types), PICK(epss), (int32_t*)ptr(),
                                       uni(0, 1) ? &e : nullptr);
          empty_work = s0 == 0 || s1 == 0;
          break;
        }
        case 3: rc = fwdmi_embedding_bag(ptr(), ptr(), ptr(), n0, n1, ptr(), n2, s0, n3, PICK(ops), xp, nullptr);
                empty_work = n1 == 0;
                break;
        case 4: rc = fwdmi_embedding_bag_fixed(ptr(), ptr(), n0, n1, ptr(), n2, s0, n3, PICK(ops), xp, nullptr);
                empty_work = n0 == 0;
                break;
        case 5: rc = fwdmi_gather(ptr(), ptr(), n0, n1, ptr(), n2, s0, n3, xp, nullptr);
                empty_work = n0 == 0 || n1 == 0;
                break;
        case 6:
        case 7: {
          const int n = (int)uni(0, 70);
          std::vector<fwdmi_bag_table> t((size_t)n);
          for (auto& d : t) d = fwdmi_bag_table{ptr(), ptr(), ptr(), PICK(big), PICK(big), PICK(big), PICK(big), ptr()};
          const int32_t n_arg = uni(0, 9) ? n : PICK(small);
          if (n_arg > n || n_arg < 0) {  // a count beyond the array: only the forms that refuse it before reading
            rc = fwdmi_embedding_bag_multi_host(nullptr, n_arg, nullptr, n0, ptr(), s0, PICK(ops), 4.0, xp, nullptr);
          } else if (uni(0, 1)) {
            rc = fwdmi_embedding_bag_multi_host(t.data(), n_arg, (fwdmi_bag_table*)ptr(), n0, ptr(), s0, PICK(ops),
                                                uni(0, 3) ? 4.0 : (double)PICK(big), xp, nullptr);
          } else {
            rc = fwdmi_embedding_bag_multi_noalloc(t.data(), n_arg, n0, ptr(), s0, PICK(ops), 4.0, xp, nullptr);
          }
          empty_work = n0 == 0;
          break;
        }
        default: {
          const int n = (int)uni(0, 70);
          std::vector<int64_t> bytes((size_t)n);
          for (auto& b : bytes) b = PICK(big);
          std::vector<float> cost((size_t)n + 1);
          rc = fwdmi_bag_table_cost(uni(0, 9) ? bytes.data() : nullptr, uni(0, 9) ? n : -n, uni(0, 9) ? cost.data() : nullptr);
          if (rc == FWDMI_OK) rc = -100;  // the one call here that can succeed without a device
          break;
        }
      }
      CHECK(rc < 0 || (rc == FWDMI_OK && empty_work), "launcher call #%d returned %d without a device", it, rc);
      CHECK(rc == -100 || rc == FWDMI_OK || fwdmi_last_error()[0] != '\0', "launcher call #%d: status %d without a reason", it, rc);
      if (rc == FWDMI_OK) ++nothing_to_do;
      ++statuses;
    }
#undef PICK
  }
  std::printf("%ld damaged inputs gave an object, %ld were refused, %ld launcher calls without a device returned a status (%ld had nothing to do), %d failures\n",
              g_alive, g_refused, statuses, nothing_to_do, g_failures);
  return g_failures ? 1 : 0;
}
