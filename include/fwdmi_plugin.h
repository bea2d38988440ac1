// fwdmi_plugin.h -- C++ plugin interface of the MI355X embedding-side path.
//
// A self-owned restatement of the contract the reference's plugins implement
// (nvinfer1::IPluginV2DynamicExt / IPluginCreator / IPluginRegistry as used by
// source/trt_engine/trt_network_crt/plugins/embedding_bag_plugin/embedding_bag_plugin.h:51-161 and
// source/trt_engine/trt_network_crt/plugins/layer_norm_plugin/layer_norm_plugin.h:41-130):
// same method names, argument meaning and call order, with a HIP stream in enqueue() and
// concrete dimensions in getOutputDimensions() instead of TensorRT's symbolic DimsExprs.
// Methods never abort: contract violations return an error value and leave a message in
// fwdmi_last_error().
#pragma once

#include <cstddef>
#include <cstdint>

#include "fwdmi.h"

namespace fwdmi {

enum class DataType : int32_t { kFLOAT = FWDMI_F32, kHALF = FWDMI_F16, kINT8 = FWDMI_I8, kINT32 = FWDMI_I32,
                                kBOOL = FWDMI_BOOL, kINT64 = FWDMI_I64 };
enum class TensorFormat : int32_t { kLINEAR = FWDMI_FORMAT_LINEAR };
enum class PluginFieldType : int32_t {
  kFLOAT16 = FWDMI_FIELD_F16, kFLOAT32 = FWDMI_FIELD_F32, kFLOAT64 = FWDMI_FIELD_F64, kINT8 = FWDMI_FIELD_I8,
  kINT16 = FWDMI_FIELD_I16, kINT32 = FWDMI_FIELD_I32, kCHAR = FWDMI_FIELD_CHAR, kDIMS = FWDMI_FIELD_DIMS,
  kUNKNOWN = FWDMI_FIELD_UNKNOWN
};

using Dims = fwdmi_dims;                    // {nbDims, d[8]}; nbDims < 0 marks an error result
using PluginTensorDesc = fwdmi_tensor_desc; // {dims, type, format, scale}
using PluginField = fwdmi_plugin_field;     // {name, data, type, length}

struct DynamicPluginTensorDesc {
  PluginTensorDesc desc;
  Dims min;
  Dims max;
};

struct PluginFieldCollection {
  int32_t nbFields;
  const PluginField* fields;
};

class IPluginV2DynamicExt {
 public:
  virtual int getNbOutputs() const noexcept = 0;
  virtual Dims getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept = 0;
  virtual bool supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                         int nbOutputs) noexcept = 0;
  // Uploads tables / parameters to the current HIP device (idempotent).  Returns a status
  // where the reference returns void and aborts on failure.
  virtual int configurePlugin(const DynamicPluginTensorDesc* in, int nbInputs,
                              const DynamicPluginTensorDesc* out, int nbOutputs) noexcept = 0;
  virtual size_t getWorkspaceSize(const PluginTensorDesc* inputs, int nbInputs, const PluginTensorDesc* outputs,
                                  int nbOutputs) const noexcept = 0;
  virtual int initialize() noexcept = 0;
  virtual void terminate() noexcept = 0;
  // Device pointers; stream-ordered; no host synchronisation and no allocation inside.
  virtual int enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc,
                      const void* const* inputs, void* const* outputs, void* workspace,
                      void* hipStream) noexcept = 0;
  virtual size_t getSerializationSize() const noexcept = 0;
  virtual void serialize(void* buffer) const noexcept = 0;
  virtual const char* getPluginType() const noexcept = 0;
  virtual const char* getPluginVersion() const noexcept = 0;
  virtual void destroy() noexcept = 0;
  virtual IPluginV2DynamicExt* clone() const noexcept = 0;
  virtual void setPluginNamespace(const char* pluginNamespace) noexcept = 0;
  virtual const char* getPluginNamespace() const noexcept = 0;
  virtual DataType getOutputDataType(int index, const DataType* inputTypes, int nbInputs) const noexcept = 0;
  // Diagnostic extension: device flag raised when an id fell outside its table (nullptr if none).
  virtual int32_t* oobFlagDevice() const noexcept { return nullptr; }

 protected:
  virtual ~IPluginV2DynamicExt() = default;
};

class IPluginCreator {
 public:
  virtual const char* getPluginName() const noexcept = 0;
  virtual const char* getPluginVersion() const noexcept = 0;
  virtual const PluginFieldCollection* getFieldNames() noexcept = 0;
  virtual IPluginV2DynamicExt* createPlugin(const char* name, const PluginFieldCollection* fc) noexcept = 0;
  virtual IPluginV2DynamicExt* deserializePlugin(const char* name, const void* serialData,
                                                 size_t serialLength) noexcept = 0;
  virtual void setPluginNamespace(const char* libNamespace) noexcept = 0;
  virtual const char* getPluginNamespace() const noexcept = 0;
  virtual ~IPluginCreator() = default;
};

class IPluginRegistry {
 public:
  virtual bool registerCreator(IPluginCreator& creator, const char* pluginNamespace) noexcept = 0;
  virtual IPluginCreator* getPluginCreator(const char* pluginName, const char* pluginVersion,
                                           const char* pluginNamespace = "") noexcept = 0;
  virtual IPluginCreator* const* getPluginCreatorList(int* numCreators) const noexcept = 0;
  virtual ~IPluginRegistry() = default;
};

// The process-wide registry (reference: getPluginRegistry(), trt_embedding_bag_creator.h:54).
IPluginRegistry* getPluginRegistry() noexcept;

template <typename T>
class PluginRegistrar {
 public:
  PluginRegistrar() { getPluginRegistry()->registerCreator(instance, ""); }

 private:
  T instance{};
};

}  // namespace fwdmi

// Counterpart of REGISTER_TENSORRT_PLUGIN (trt_creator_manager.cpp:81-98).
#define FWDMI_REGISTER_PLUGIN(name) static ::fwdmi::PluginRegistrar<name> pluginRegistrar##name {}
