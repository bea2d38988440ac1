// Plan files: the plugins of an engine saved to / loaded from one file, plus the JSON sidecar.
//
// Counterpart of the persistence step of the reference engine (TrtForwardEngine::Save / Load,
// source/trt_engine/trt_engine/trt_fwd_engine.cpp:156-209): there TensorRT writes each plugin's
// serialize() bytes into its engine blob and finds the creator again by (type, version,
// namespace) when loading; the engine's settings go to "<file>.meta" as JSON
// (source/trt_engine/trt_common/trt_meta_data.cpp:42-97).  Here the container is explicit:
//
//   char magic[8] = "FWDMIPL1" | uint32 n | n x { str layer | str type | str version | str namespace |
//                                               uint64 blob_len | blob }      (str = uint32 len + bytes)
//
// and the sidecar is read and written through the typed EngineMetaData (engine_meta.h): what is saved
// is the reference's form of the document, and a sidecar that the reference's reader would reject
// (a missing key, a value of the wrong type) fails the save or the load here too.
#include <cstdio>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "engine_meta.h"
#include "plugin_util.h"

using namespace fwdmi;

namespace {

constexpr char kMagic[8] = {'F', 'W', 'D', 'M', 'I', 'P', 'L', '1'};

struct PlanEntry {
  std::string layer;
  IPluginV2DynamicExt* plugin = nullptr;  // owned until taken
};

struct Plan {
  std::vector<PlanEntry> entries;
  EngineMetaData meta;
  bool has_meta = false;
  std::string meta_text;
  ~Plan() {
    for (auto& e : entries)
      if (e.plugin) e.plugin->destroy();
  }
};

void put_str(std::ofstream& f, const std::string& s) {
  const uint32_t n = (uint32_t)s.size();
  f.write(reinterpret_cast<const char*>(&n), 4);
  f.write(s.data(), n);
}

bool get_str(std::ifstream& f, std::string* s) {
  uint32_t n = 0;
  if (!f.read(reinterpret_cast<char*>(&n), 4) || n > (1u << 20)) return false;
  s->resize(n);
  return n == 0 || (bool)f.read(&(*s)[0], n);
}

}  // namespace

extern "C" {

int fwdmi_plan_save(const char* path, fwdmi_plugin* const* plugins, const char* const* layer_names, int n,
                    const char* meta_json) {
  clear_error();
  if (!path || n < 0 || (n > 0 && (!plugins || !layer_names)))
    return set_error(FWDMI_ERR_BAD_ARG, "plan_save: null argument");
  if (meta_json) {  // checked before anything is written
    EngineMetaData probe;
    if (!probe.ParseMetaData(meta_json)) return FWDMI_ERR_BAD_ARG;
  }
  std::ofstream f(path, std::ios::binary | std::ios::trunc);
  if (!f) return set_error(FWDMI_ERR_BAD_ARG, "plan_save: cannot open '%s' for writing", path);
  f.write(kMagic, 8);
  const uint32_t count = (uint32_t)n;
  f.write(reinterpret_cast<const char*>(&count), 4);
  std::vector<char> blob;
  for (int i = 0; i < n; ++i) {
    auto* p = reinterpret_cast<IPluginV2DynamicExt*>(plugins[i]);
    if (!p) return set_error(FWDMI_ERR_BAD_ARG, "plan_save: plugin %d is null", i);
    put_str(f, layer_names[i] ? layer_names[i] : "");
    put_str(f, p->getPluginType());
    put_str(f, p->getPluginVersion());
    put_str(f, p->getPluginNamespace());
    blob.resize(p->getSerializationSize());
    p->serialize(blob.data());
    const uint64_t len = blob.size();
    f.write(reinterpret_cast<const char*>(&len), 8);
    f.write(blob.data(), (std::streamsize)len);
  }
  if (!f) return set_error(FWDMI_ERR_BAD_ARG, "plan_save: write to '%s' failed", path);
  f.close();
  if (meta_json) {
    EngineMetaData meta;
    if (!meta.ParseMetaData(meta_json)) return FWDMI_ERR_BAD_ARG;  // the reason is the thread's last error
    if (!meta.SaveMetaData(std::string(path) + ".meta")) return FWDMI_ERR_BAD_ARG;
  }
  return FWDMI_OK;
}

fwdmi_plan* fwdmi_plan_load(const char* path) {
  clear_error();
  if (!path) {
    set_error(FWDMI_ERR_BAD_ARG, "plan_load: null path");
    return nullptr;
  }
  std::ifstream f(path, std::ios::binary);
  char magic[8];
  uint32_t n = 0;
  if (!f || !f.read(magic, 8) || std::memcmp(magic, kMagic, 8) != 0 || !f.read(reinterpret_cast<char*>(&n), 4)) {
    set_error(FWDMI_ERR_TRUNCATED, "plan_load: '%s' is not a plan file", path);
    return nullptr;
  }
  std::unique_ptr<Plan> plan(new Plan());
  std::vector<char> blob;
  for (uint32_t i = 0; i < n; ++i) {
    std::string layer, type, version, ns;
    uint64_t len = 0;
    if (!get_str(f, &layer) || !get_str(f, &type) || !get_str(f, &version) || !get_str(f, &ns) ||
        !f.read(reinterpret_cast<char*>(&len), 8)) {
      set_error(FWDMI_ERR_TRUNCATED, "plan_load: entry %u of '%s' is truncated", i, path);
      return nullptr;
    }
    const std::streampos here = f.tellg();
    f.seekg(0, std::ios::end);
    const uint64_t remaining = (uint64_t)(f.tellg() - here);
    f.seekg(here);
    if (len > remaining) {
      set_error(FWDMI_ERR_TRUNCATED, "plan_load: blob of entry %u of '%s' is truncated", i, path);
      return nullptr;
    }
    blob.resize(len);
    if (len && !f.read(blob.data(), (std::streamsize)len)) {
      set_error(FWDMI_ERR_TRUNCATED, "plan_load: blob of entry %u of '%s' is truncated", i, path);
      return nullptr;
    }
    // same lookup TensorRT performs when it deserializes an engine
    IPluginCreator* c = getPluginRegistry()->getPluginCreator(type.c_str(), version.c_str(), "");
    if (!c) {
      set_error(FWDMI_ERR_UNSUPPORTED, "plan_load: no creator for %s version %s", type.c_str(), version.c_str());
      return nullptr;
    }
    IPluginV2DynamicExt* p = c->deserializePlugin(layer.c_str(), blob.data(), blob.size());
    if (!p) return nullptr;  // the creator left the reason in last_error
    p->setPluginNamespace(ns.c_str());
    plan->entries.push_back(PlanEntry{layer, p});
  }
  std::ifstream m(std::string(path) + ".meta");
  if (m) {  // a plan without a sidecar is a plan without engine settings; a sidecar that is there must be valid
    m.close();
    if (!plan->meta.LoadMetaData(std::string(path) + ".meta")) return nullptr;
    plan->has_meta = true;
    plan->meta_text = plan->meta.ToJson();
  }
  return reinterpret_cast<fwdmi_plan*>(plan.release());
}

int fwdmi_plan_size(fwdmi_plan* plan) {
  return plan ? (int)reinterpret_cast<Plan*>(plan)->entries.size() : FWDMI_ERR_BAD_ARG;
}

const char* fwdmi_plan_layer_name(fwdmi_plan* plan, int i) {
  auto* p = reinterpret_cast<Plan*>(plan);
  return (p && i >= 0 && i < (int)p->entries.size()) ? p->entries[i].layer.c_str() : nullptr;
}

fwdmi_plugin* fwdmi_plan_take_plugin(fwdmi_plan* plan, int i) {
  auto* p = reinterpret_cast<Plan*>(plan);
  if (!p || i < 0 || i >= (int)p->entries.size()) return nullptr;
  IPluginV2DynamicExt* out = p->entries[i].plugin;
  p->entries[i].plugin = nullptr;
  return reinterpret_cast<fwdmi_plugin*>(out);
}

const char* fwdmi_plan_meta(fwdmi_plan* plan) { return plan ? reinterpret_cast<Plan*>(plan)->meta_text.c_str() : nullptr; }

void fwdmi_plan_close(fwdmi_plan* plan) { delete reinterpret_cast<Plan*>(plan); }

// ---- the typed sidecar by itself ---------------------------------------------------------------
namespace {
struct MetaHandle {
  EngineMetaData meta;
  std::vector<int32_t> unused, outputs;  // what the array getters point into
  std::string text;
};
inline MetaHandle* M(fwdmi_meta* m) { return reinterpret_cast<MetaHandle*>(m); }
}  // namespace

fwdmi_meta* fwdmi_meta_new(void) { return reinterpret_cast<fwdmi_meta*>(new MetaHandle()); }

fwdmi_meta* fwdmi_meta_load(const char* meta_file) {
  clear_error();
  if (!meta_file) {
    set_error(FWDMI_ERR_BAD_ARG, "meta_load: null path");
    return nullptr;
  }
  std::unique_ptr<MetaHandle> h(new MetaHandle());
  if (!h->meta.LoadMetaData(meta_file)) return nullptr;
  return reinterpret_cast<fwdmi_meta*>(h.release());
}

fwdmi_meta* fwdmi_meta_parse(const char* json_text) {
  clear_error();
  if (!json_text) {
    set_error(FWDMI_ERR_BAD_ARG, "meta_parse: null text");
    return nullptr;
  }
  std::unique_ptr<MetaHandle> h(new MetaHandle());
  if (!h->meta.ParseMetaData(json_text)) return nullptr;
  return reinterpret_cast<fwdmi_meta*>(h.release());
}

fwdmi_meta* fwdmi_plan_meta_data(fwdmi_plan* plan) {
  auto* p = reinterpret_cast<Plan*>(plan);
  if (!p || !p->has_meta) return nullptr;
  MetaHandle* h = new MetaHandle();
  h->meta = p->meta;
  return reinterpret_cast<fwdmi_meta*>(h);
}

int fwdmi_meta_save(fwdmi_meta* m, const char* meta_file) {
  clear_error();
  if (!m || !meta_file) return set_error(FWDMI_ERR_BAD_ARG, "meta_save: null argument");
  return M(m)->meta.SaveMetaData(meta_file) ? FWDMI_OK : FWDMI_ERR_BAD_ARG;
}

const char* fwdmi_meta_json(fwdmi_meta* m) {
  if (!m) return nullptr;
  M(m)->text = M(m)->meta.ToJson();
  return M(m)->text.c_str();
}

int32_t fwdmi_meta_infer_mode(fwdmi_meta* m) { return m ? static_cast<int32_t>(M(m)->meta.Mode()) : -1; }
int32_t fwdmi_meta_opt_batch_size(fwdmi_meta* m) { return m ? M(m)->meta.OptBatchSize() : -1; }
int32_t fwdmi_meta_max_batch_size(fwdmi_meta* m) { return m ? M(m)->meta.MaxBatchSize() : -1; }
const char* fwdmi_meta_torch_module_path(fwdmi_meta* m) { return m ? M(m)->meta.TorchModulePath().c_str() : nullptr; }

int32_t fwdmi_meta_unused_input_indices(fwdmi_meta* m, const int32_t** data) {
  if (!m) return FWDMI_ERR_BAD_ARG;
  M(m)->unused.assign(M(m)->meta.UnusedInputIndices().begin(), M(m)->meta.UnusedInputIndices().end());
  if (data) *data = M(m)->unused.data();
  return (int32_t)M(m)->unused.size();
}

int32_t fwdmi_meta_output_indices(fwdmi_meta* m, const int32_t** data) {
  if (!m) return FWDMI_ERR_BAD_ARG;
  M(m)->outputs.assign(M(m)->meta.OutputPositions().begin(), M(m)->meta.OutputPositions().end());
  if (data) *data = M(m)->outputs.data();
  return (int32_t)M(m)->outputs.size();
}

int fwdmi_meta_set(fwdmi_meta* m, int32_t infer_mode, int32_t opt_batch_size, int32_t max_batch_size,
                   const int32_t* unused_input_indices, int32_t n_unused, const int32_t* output_indices,
                   int32_t n_outputs, const char* torch_module_path) {
  clear_error();
  if (!m || n_unused < 0 || n_outputs < 0 || (n_unused > 0 && !unused_input_indices) || (n_outputs > 0 && !output_indices))
    return set_error(FWDMI_ERR_BAD_ARG, "meta_set: null argument or negative count");
  EngineMetaData& e = M(m)->meta;
  e.SetMode(static_cast<InferMode>(infer_mode));
  e.SetOptBatchSize(opt_batch_size);
  e.SetMaxBatchSize(max_batch_size);
  e.SetUnusedInputIndices(std::set<int>(unused_input_indices, unused_input_indices + n_unused));
  e.SetOutputPositions(std::vector<int>(output_indices, output_indices + n_outputs));
  e.SetTorchModulePath(torch_module_path ? torch_module_path : "");
  return FWDMI_OK;
}

void fwdmi_meta_free(fwdmi_meta* m) { delete M(m); }

}  // extern "C"
