// Helpers shared by the plugin classes: byte-stream (de)serialisation with the reference's
// layout rules, creator-field access, fp16 conversion of host weights, device buffers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../common.h"
#include "fwdmi_plugin.h"

namespace fwdmi {

// ---- byte streams ---------------------------------------------------------------------------
// Layout rules of the reference serializer (plugins/common/serialize.hpp:41-103): a POD is its
// raw sizeof(T) bytes, a vector is a size_t element count followed by the raw elements,
// host-endian, no header.  Reads are bounds-checked and report truncation instead of asserting.
class ByteWriter {
 public:
  explicit ByteWriter(void* p) : p_(static_cast<char*>(p)) {}
  template <typename T>
  void pod(const T& v) {
    std::memcpy(p_, &v, sizeof(T));
    p_ += sizeof(T);
  }
  void bytes(const void* src, size_t n) {
    if (n) std::memcpy(p_, src, n);
    p_ += n;
  }
  template <typename T>
  void vec(const T* data, size_t count) {
    pod<size_t>(count);
    bytes(data, count * sizeof(T));
  }

 private:
  char* p_;
};

class ByteReader {
 public:
  ByteReader(const void* p, size_t n) : p_(static_cast<const char*>(p)), left_(n) {}
  template <typename T>
  bool pod(T* v) {
    if (left_ < sizeof(T)) return fail();
    std::memcpy(v, p_, sizeof(T));
    advance(sizeof(T));
    return true;
  }
  bool bytes(void* dst, size_t n) {
    if (left_ < n) return fail();
    if (n) std::memcpy(dst, p_, n);
    advance(n);
    return true;
  }
  // Reads a size_t count followed by count elements of `elem` bytes into `out`.
  bool vec(std::vector<uint8_t>* out, size_t elem, size_t* count) {
    size_t n = 0;
    if (!pod(&n)) return false;
    if (elem != 0 && n > left_ / elem) return fail();
    out->resize(n * elem);
    *count = n;
    return bytes(out->data(), n * elem);
  }
  size_t left() const { return left_; }
  bool ok() const { return ok_; }

 private:
  bool fail() {
    ok_ = false;
    return false;
  }
  void advance(size_t n) {
    p_ += n;
    left_ -= n;
  }
  const char* p_;
  size_t left_;
  bool ok_ = true;
};

// ---- creator fields ---------------------------------------------------------------------------
inline const PluginField* find_field(const PluginFieldCollection* fc, const char* name) {
  for (int i = 0; i < fc->nbFields; ++i)
    if (fc->fields[i].name && std::strcmp(fc->fields[i].name, name) == 0) return &fc->fields[i];
  return nullptr;
}

inline size_t field_elem_size(int32_t type) {
  switch (type) {
    case FWDMI_FIELD_F16: return 2;
    case FWDMI_FIELD_F32: return 4;
    case FWDMI_FIELD_F64: return 8;
    case FWDMI_FIELD_I8: return 1;
    case FWDMI_FIELD_I16: return 2;
    case FWDMI_FIELD_I32: return 4;
    case FWDMI_FIELD_CHAR: return 1;
    default: return 0;
  }
}

// Reads a float array field (FLOAT32 or FLOAT16) as fp32 values.
inline bool field_to_f32(const PluginField& f, std::vector<float>* out) {
  if (!f.data || f.length < 0) return false;
  out->resize(f.length);
  if (f.type == FWDMI_FIELD_F32) {
    std::memcpy(out->data(), f.data, sizeof(float) * f.length);
  } else if (f.type == FWDMI_FIELD_F16) {
    const _Float16* h = static_cast<const _Float16*>(f.data);
    for (int i = 0; i < f.length; ++i) (*out)[i] = (float)h[i];
  } else {
    return false;
  }
  return true;
}

// Rounds fp32 values through fp16 (what storing parameters in a half-precision plugin does,
// reference: WeightsWithOwnership::convertAndCopy, plugins/common/plugin_common.h:185-228).
inline void round_through_f16(std::vector<float>* v) {
  for (float& x : *v) x = (float)(_Float16)x;
}

inline void f32_to_f16_bytes(const float* src, size_t n, void* dst) {
  _Float16* h = static_cast<_Float16*>(dst);
  for (size_t i = 0; i < n; ++i) h[i] = (_Float16)src[i];
}

// ---- device memory ------------------------------------------------------------------------------
// A host byte image with a lazily created, reference-counted device copy.  Clones of a plugin
// share one HostDeviceBlob, so a table is held once on the host and once on the device no
// matter how many times the plugin is cloned.
class HostDeviceBlob {
 public:
  explicit HostDeviceBlob(std::vector<uint8_t> host) : host_(std::move(host)) {
    data_ = host_.data();
    size_ = host_.size();
  }
  // A read-only mapping of `nbytes` of `path` starting at `offset`: the table stays in the
  // page cache instead of being copied into the process (and into every serialized engine).
  static std::shared_ptr<HostDeviceBlob> map_file(const std::string& path, uint64_t offset, size_t nbytes);
  ~HostDeviceBlob();
  HostDeviceBlob(const HostDeviceBlob&) = delete;
  HostDeviceBlob& operator=(const HostDeviceBlob&) = delete;

  const uint8_t* data() const { return data_; }
  size_t size() const { return size_; }
  bool by_reference() const { return !path_.empty(); }
  const std::string& path() const { return path_; }
  uint64_t file_offset() const { return file_offset_; }
  // Takes a device reference, uploading on first use.  Returns a status.
  int acquire(void** dev) {
    std::lock_guard<std::mutex> lock(mu_);
    if (!dev_) {
      const size_t n = size_ ? size_ : 16;
      void* p = nullptr;
      FWDMI_HIP_CHECK(hipMalloc(&p, n));
      if (size_) {
        hipError_t e = hipMemcpy(p, data_, size_, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
          (void)hipFree(p);
          return set_error(FWDMI_ERR_HIP, "hipMemcpy (table upload) failed: %s", hipGetErrorString(e));
        }
      }
      dev_ = p;
    }
    ++users_;
    *dev = dev_;
    return FWDMI_OK;
  }
  void release() {
    std::lock_guard<std::mutex> lock(mu_);
    if (users_ > 0 && --users_ == 0 && dev_) {
      (void)hipFree(dev_);
      dev_ = nullptr;
    }
  }

 private:
  HostDeviceBlob() = default;
  std::vector<uint8_t> host_;
  const uint8_t* data_ = nullptr;
  size_t size_ = 0;
  std::string path_;       // non-empty: data_ points into a file mapping
  uint64_t file_offset_ = 0;
  void* map_base_ = nullptr;
  size_t map_len_ = 0;
  std::mutex mu_;
  void* dev_ = nullptr;
  int users_ = 0;
};

inline std::shared_ptr<HostDeviceBlob> make_blob(const void* data, size_t nbytes) {
  std::vector<uint8_t> v(nbytes);
  if (nbytes) std::memcpy(v.data(), data, nbytes);
  return std::make_shared<HostDeviceBlob>(std::move(v));
}

inline std::shared_ptr<HostDeviceBlob> make_blob_f32(const std::vector<float>& v) {
  return make_blob(v.data(), v.size() * sizeof(float));
}

inline int64_t volume(const Dims& d) {
  int64_t v = 1;
  for (int i = 0; i < d.nbDims; ++i) v *= d.d[i];
  return v;
}

inline Dims error_dims() {
  Dims d{};
  d.nbDims = -1;
  return d;
}

// Namespace handling common to all creators (reference: BaseCreator, plugins/common/plugin.h:38-47).
class BaseCreator : public IPluginCreator {
 public:
  void setPluginNamespace(const char* libNamespace) noexcept override { mNamespace = libNamespace ? libNamespace : ""; }
  const char* getPluginNamespace() const noexcept override { return mNamespace.c_str(); }
  const PluginFieldCollection* getFieldNames() noexcept override {
    mFC.nbFields = (int32_t)mPluginAttributes.size();
    mFC.fields = mPluginAttributes.data();
    return &mFC;
  }

 protected:
  void declare(const char* name, PluginFieldType type) {
    mPluginAttributes.push_back(PluginField{name, nullptr, (int32_t)type, 1});
  }
  std::string mNamespace;
  PluginFieldCollection mFC{};
  std::vector<PluginField> mPluginAttributes;
};

}  // namespace fwdmi
