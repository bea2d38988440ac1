// LayerNorm-family plugins:
//   "ForwardLayerNormPluginDynamic" v1      1 input   out = LN(input (+ bias))
//   "CustomSkipLayerNormPluginDynamic" v1   2 inputs  out = LN(input + skip (+ bias))
//   "CustomEmbLayerNormPluginDynamic" v1    3 inputs  BERT embedding lookup + LN, mask index
//
// The first mirrors LayerNormPluginDynamic of the reference
// (source/trt_engine/trt_network_crt/plugins/layer_norm_plugin/layer_norm_plugin.h:41-130,
// layer_norm_plugin.cpp:34-391).  The other two are the plugins the reference obtains by name
// from NVIDIA's plugin library (trt_bert_creator.h:127-128, :219-220); their creator fields,
// input order and output use are taken from those call sites.
#pragma once

#include <memory>
#include <string>

#include "plugin_util.h"

namespace fwdmi {

constexpr const char* FWD_LAYER_NORM_NAME{"ForwardLayerNormPluginDynamic"};
constexpr const char* FWD_LAYER_NORM_VERSION{"1"};
constexpr const char* SKIP_LAYER_NORM_NAME{"CustomSkipLayerNormPluginDynamic"};
constexpr const char* SKIP_LAYER_NORM_VERSION{"1"};
constexpr const char* EMB_LAYER_NORM_NAME{"CustomEmbLayerNormPluginDynamic"};
constexpr const char* EMB_LAYER_NORM_VERSION{"1"};

// Dimension roles of the BERT activations [S, B, H, 1, 1] (plugins/common/plugin_common.h:39-41).
constexpr uint32_t BDIM = 1;
constexpr uint32_t SDIM = 0;
constexpr uint32_t HDIM = 2;

// LN(input (+ skip) (+ bias)); `with_skip` selects the two-input plugin.
class LayerNormPluginDynamic final : public IPluginV2DynamicExt {
 public:
  // beta/gamma/bias are fp32 host values; in a half-precision plugin they are rounded through
  // fp16 first, as storing them in the configured type does in the reference.
  LayerNormPluginDynamic(std::string name, bool with_skip, DataType type, size_t ld, std::vector<float> beta,
                         std::vector<float> gamma, std::vector<float> bias, float eps);
  static LayerNormPluginDynamic* deserialize(const std::string& name, bool with_skip, const void* data,
                                             size_t length);
  ~LayerNormPluginDynamic() noexcept override;

  IPluginV2DynamicExt* clone() const noexcept override;
  Dims getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept override;
  bool supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                 int nbOutputs) noexcept override;
  int configurePlugin(const DynamicPluginTensorDesc* in, int nbInputs, const DynamicPluginTensorDesc* out,
                      int nbOutputs) noexcept override;
  size_t getWorkspaceSize(const PluginTensorDesc*, int, const PluginTensorDesc*, int) const noexcept override;
  int enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc, const void* const* inputs,
              void* const* outputs, void* workspace, void* hipStream) noexcept override;
  DataType getOutputDataType(int index, const DataType* inputTypes, int nbInputs) const noexcept override;
  const char* getPluginType() const noexcept override;
  const char* getPluginVersion() const noexcept override;
  int getNbOutputs() const noexcept override;
  int initialize() noexcept override;
  void terminate() noexcept override;
  size_t getSerializationSize() const noexcept override;
  void serialize(void* buffer) const noexcept override;
  void destroy() noexcept override;
  void setPluginNamespace(const char* pluginNamespace) noexcept override;
  const char* getPluginNamespace() const noexcept override;

 private:
  int nb_inputs() const { return with_skip_ ? 2 : 1; }
  const std::string layer_name_;
  const bool with_skip_;
  DataType type_;      // plugin I/O type
  DataType cfg_type_;  // type the parameters are stored (and serialized) in
  size_t ld_;
  bool has_bias_;
  float eps_;
  std::vector<float> beta_, gamma_, bias_;
  std::shared_ptr<HostDeviceBlob> params_;  // beta | gamma | bias as fp32, shared with clones
  float* d_params_ = nullptr;
  bool configured_ = false;
  std::string namespace_;
};

class LayerNormCreatorBase : public BaseCreator {
 public:
  explicit LayerNormCreatorBase(bool with_skip);
  IPluginV2DynamicExt* createPlugin(const char* name, const PluginFieldCollection* fc) noexcept override;
  IPluginV2DynamicExt* deserializePlugin(const char* name, const void* serialData,
                                         size_t serialLength) noexcept override;

 private:
  bool with_skip_;
};

class LayerNormPluginDynamicCreator : public LayerNormCreatorBase {
 public:
  LayerNormPluginDynamicCreator() : LayerNormCreatorBase(false) {}
  const char* getPluginName() const noexcept override { return FWD_LAYER_NORM_NAME; }
  const char* getPluginVersion() const noexcept override { return FWD_LAYER_NORM_VERSION; }
};

class SkipLayerNormPluginDynamicCreator : public LayerNormCreatorBase {
 public:
  SkipLayerNormPluginDynamicCreator() : LayerNormCreatorBase(true) {}
  const char* getPluginName() const noexcept override { return SKIP_LAYER_NORM_NAME; }
  const char* getPluginVersion() const noexcept override { return SKIP_LAYER_NORM_VERSION; }
};

class EmbLayerNormPluginDynamic final : public IPluginV2DynamicExt {
 public:
  struct Tables {
    std::vector<float> beta, gamma;                // [ld] fp32
    std::shared_ptr<HostDeviceBlob> word, pos, tok;  // rows in the output type
    int word_count = 0, pos_count = 0, tok_count = 0;
    // The SkipLayerNorm that consumes the embedding, when the plugin stands for both layers: a fourth
    // input (the residual, shaped like output 0) and output 0 = LN2(embedding + residual (+ bias2)).
    bool fused_skip = false;
    std::vector<float> beta2, gamma2, bias2;  // [ld] fp32; bias2 may be empty
    float eps2 = 0.0f;
  };
  EmbLayerNormPluginDynamic(std::string name, DataType type, DataType mha_type, int ld, Tables tables, float eps,
                            bool batch_major = false);
  static EmbLayerNormPluginDynamic* deserialize(const std::string& name, const void* data, size_t length);
  ~EmbLayerNormPluginDynamic() noexcept override;

  IPluginV2DynamicExt* clone() const noexcept override;
  Dims getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept override;
  bool supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                 int nbOutputs) noexcept override;
  int configurePlugin(const DynamicPluginTensorDesc* in, int nbInputs, const DynamicPluginTensorDesc* out,
                      int nbOutputs) noexcept override;
  size_t getWorkspaceSize(const PluginTensorDesc*, int, const PluginTensorDesc*, int) const noexcept override;
  int enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc, const void* const* inputs,
              void* const* outputs, void* workspace, void* hipStream) noexcept override;
  DataType getOutputDataType(int index, const DataType* inputTypes, int nbInputs) const noexcept override;
  const char* getPluginType() const noexcept override;
  const char* getPluginVersion() const noexcept override;
  int getNbOutputs() const noexcept override;
  int initialize() noexcept override;
  void terminate() noexcept override;
  size_t getSerializationSize() const noexcept override;
  void serialize(void* buffer) const noexcept override;
  void destroy() noexcept override;
  void setPluginNamespace(const char* pluginNamespace) noexcept override;
  const char* getPluginNamespace() const noexcept override;
  int32_t* oobFlagDevice() const noexcept override { return d_oob_; }

 private:
  const std::string layer_name_;
  DataType type_;      // output / table type
  DataType mha_type_;  // type of the attention consumer (kept and serialized, not used here)
  int ld_;
  float eps_;
  bool batch_major_;  // ids are [B, S] and the output [B, S, H, 1, 1] (no transposes around the plugin)
  Tables t_;
  std::shared_ptr<HostDeviceBlob> params_;  // beta | gamma [| beta2 | gamma2 [| bias2]] fp32
  int nb_inputs() const { return t_.fused_skip ? 4 : 3; }
  float* d_params_ = nullptr;
  void *d_word_ = nullptr, *d_pos_ = nullptr, *d_tok_ = nullptr;
  int32_t* d_oob_ = nullptr;
  bool configured_ = false;
  std::string namespace_;
};

class EmbLayerNormPluginDynamicCreator : public BaseCreator {
 public:
  EmbLayerNormPluginDynamicCreator();
  const char* getPluginName() const noexcept override { return EMB_LAYER_NORM_NAME; }
  const char* getPluginVersion() const noexcept override { return EMB_LAYER_NORM_VERSION; }
  IPluginV2DynamicExt* createPlugin(const char* name, const PluginFieldCollection* fc) noexcept override;
  IPluginV2DynamicExt* deserializePlugin(const char* name, const void* serialData,
                                         size_t serialLength) noexcept override;
};

}  // namespace fwdmi
