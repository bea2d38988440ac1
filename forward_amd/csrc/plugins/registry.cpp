// Process-wide plugin registry: creators are looked up by (name, version, namespace), the way
// the reference's layer creators find theirs (getPluginRegistry()->getPluginCreator(...),
// source/trt_engine/trt_network_crt/layer_creators/trt_embedding_bag_creator.h:54-55).
#include <mutex>
#include <string>
#include <vector>

#include "plugin_util.h"

namespace fwdmi {
namespace {

class PluginRegistry final : public IPluginRegistry {
 public:
  bool registerCreator(IPluginCreator& creator, const char* pluginNamespace) noexcept override {
    std::lock_guard<std::mutex> lock(mu_);
    const std::string ns = pluginNamespace ? pluginNamespace : "";
    for (IPluginCreator* c : creators_)
      if (same(c, creator.getPluginName(), creator.getPluginVersion(), ns.c_str())) return false;
    creator.setPluginNamespace(ns.c_str());
    creators_.push_back(&creator);
    return true;
  }

  IPluginCreator* getPluginCreator(const char* pluginName, const char* pluginVersion,
                                   const char* pluginNamespace) noexcept override {
    if (!pluginName || !pluginVersion) return nullptr;
    std::lock_guard<std::mutex> lock(mu_);
    for (IPluginCreator* c : creators_)
      if (same(c, pluginName, pluginVersion, pluginNamespace ? pluginNamespace : "")) return c;
    return nullptr;
  }

  IPluginCreator* const* getPluginCreatorList(int* numCreators) const noexcept override {
    if (numCreators) *numCreators = (int)creators_.size();
    return creators_.data();
  }

 private:
  static bool same(IPluginCreator* c, const char* name, const char* version, const char* ns) {
    return std::string(c->getPluginName()) == name && std::string(c->getPluginVersion()) == version &&
           std::string(c->getPluginNamespace()) == ns;
  }
  std::mutex mu_;
  std::vector<IPluginCreator*> creators_;
};

}  // namespace

IPluginRegistry* getPluginRegistry() noexcept {
  static PluginRegistry registry;
  return &registry;
}

}  // namespace fwdmi
