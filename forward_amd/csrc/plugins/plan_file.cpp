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
// and the sidecar text is passed through unchanged.
#include <cstdio>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

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
  std::string meta;
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
    std::ofstream m(std::string(path) + ".meta", std::ios::trunc);
    m << meta_json;
    if (!m) return set_error(FWDMI_ERR_BAD_ARG, "plan_save: cannot write '%s.meta'", path);
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
  if (m) {
    std::stringstream ss;
    ss << m.rdbuf();
    plan->meta = ss.str();
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

const char* fwdmi_plan_meta(fwdmi_plan* plan) { return plan ? reinterpret_cast<Plan*>(plan)->meta.c_str() : nullptr; }

void fwdmi_plan_close(fwdmi_plan* plan) { delete reinterpret_cast<Plan*>(plan); }

}  // extern "C"
