// Process-wide plugin registry: creators are looked up by (name, version, namespace), the way
// the reference's layer creators find theirs (getPluginRegistry()->getPluginCreator(...),
// source/trt_engine/trt_network_crt/layer_creators/trt_embedding_bag_creator.h:54-55).
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

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

HostDeviceBlob::~HostDeviceBlob() {
  if (dev_) (void)hipFree(dev_);
  if (map_base_) munmap(map_base_, map_len_);
}

std::shared_ptr<HostDeviceBlob> HostDeviceBlob::map_file(const std::string& path, uint64_t offset, size_t nbytes) {
  const int fd = open(path.c_str(), O_RDONLY);
  if (fd < 0) {
    set_error(FWDMI_ERR_BAD_ARG, "cannot open table file '%s'", path.c_str());
    return nullptr;
  }
  struct stat st {};
  // compared without forming offset + nbytes, which a corrupt header could make wrap
  if (fstat(fd, &st) != 0 || offset > (uint64_t)st.st_size || nbytes > (uint64_t)st.st_size - offset) {
    close(fd);
    set_error(FWDMI_ERR_TRUNCATED, "table file '%s' is shorter than offset %llu + %zu bytes", path.c_str(),
              (unsigned long long)offset, nbytes);
    return nullptr;
  }
  const uint64_t page = (uint64_t)sysconf(_SC_PAGESIZE);
  const uint64_t base = offset / page * page;
  const size_t len = (size_t)(offset - base) + nbytes;
  void* m = len ? mmap(nullptr, len, PROT_READ, MAP_PRIVATE, fd, (off_t)base) : nullptr;
  close(fd);
  if (len && m == MAP_FAILED) {
    set_error(FWDMI_ERR_BAD_ARG, "mmap of table file '%s' failed", path.c_str());
    return nullptr;
  }
  std::shared_ptr<HostDeviceBlob> b(new HostDeviceBlob());
  b->path_ = path;
  b->file_offset_ = offset;
  b->map_base_ = m;
  b->map_len_ = len;
  b->data_ = static_cast<const uint8_t*>(m) + (offset - base);
  b->size_ = nbytes;
  return b;
}

IPluginRegistry* getPluginRegistry() noexcept {
  static PluginRegistry registry;
  return &registry;
}

}  // namespace fwdmi
