// EmbeddingBag plugin: host-side object behind "EmbeddingBag_TRT".
//
// Mirrors EmbeddingBagPlugin / EmbeddingBagPluginCreator of the reference
// (source/trt_engine/trt_network_crt/plugins/embedding_bag_plugin/embedding_bag_plugin.h:51-161,
// embedding_bag_plugin.cpp:37-300): same creator fields, shape rules, format rules, dispatch
// and serialized bytes.  Version "001" is the reference contract (fp32 table, int32 ids,
// fp32 output, exactly five fields).  Version "002" adds optional fields for fp16 tables,
// int64 ids, fp16 output, include_last_offset, a per-sample-weights input and a second output
// with the sums of squares (the pair a factorisation-machine term needs, from one pass), and
// appends them to the serialized layout.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "plugin_util.h"

namespace fwdmi {

constexpr const char* EMBEDDING_BAG_PLUGIN_NAME{"EmbeddingBag_TRT"};
constexpr const char* EMBEDDING_BAG_PLUGIN_VERSION{"001"};
constexpr const char* EMBEDDING_BAG_PLUGIN_VERSION_EXT{"002"};

enum class ReduceOperation : int32_t { GATHER = 999, SUM = 0, MEAN = 1, MAX = 2, SQUARE_SUM = 3 };

struct EmbeddingBagOptions {
  int32_t table_dtype = FWDMI_F32;
  int32_t index_dtype = FWDMI_I32;
  int32_t out_dtype = FWDMI_F32;
  int32_t include_last_offset = 0;
  int32_t per_sample_weights = 0;  // 1: a third input carries per-sample weights
  int32_t with_square_sum = 0;     // 1 (op SUM): a second output carries the sums of squares
  bool is_default() const {
    return table_dtype == FWDMI_F32 && index_dtype == FWDMI_I32 && out_dtype == FWDMI_F32 &&
           !include_last_offset && !per_sample_weights && !with_square_sum;
  }
};

class EmbeddingBagPlugin final : public IPluginV2DynamicExt {
 public:
  // `version_ext` selects the "002" contract.
  EmbeddingBagPlugin(std::shared_ptr<HostDeviceBlob> table, int dim, int count, int offset,
                     ReduceOperation op, const EmbeddingBagOptions& opt, bool version_ext);
  // nullptr on a truncated / inconsistent blob.
  static EmbeddingBagPlugin* deserialize(const void* data, size_t length, bool version_ext);
  ~EmbeddingBagPlugin() noexcept override;

  int getNbOutputs() const noexcept override;
  Dims getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept override;
  bool supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                 int nbOutputs) noexcept override;
  int configurePlugin(const DynamicPluginTensorDesc* in, int nbInputs, const DynamicPluginTensorDesc* out,
                      int nbOutputs) noexcept override;
  size_t getWorkspaceSize(const PluginTensorDesc* inputs, int nbInputs, const PluginTensorDesc* outputs,
                          int nbOutputs) const noexcept override;
  int initialize() noexcept override;
  void terminate() noexcept override;
  int enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc, const void* const* inputs,
              void* const* outputs, void* workspace, void* hipStream) noexcept override;
  size_t getSerializationSize() const noexcept override;
  void serialize(void* buffer) const noexcept override;
  const char* getPluginType() const noexcept override;
  const char* getPluginVersion() const noexcept override;
  void destroy() noexcept override;
  IPluginV2DynamicExt* clone() const noexcept override;
  void setPluginNamespace(const char* pluginNamespace) noexcept override;
  const char* getPluginNamespace() const noexcept override;
  DataType getOutputDataType(int index, const DataType* inputTypes, int nbInputs) const noexcept override;
  int32_t* oobFlagDevice() const noexcept override { return d_oob_; }

 private:
  int dim_;
  int count_;
  int data_offset_;
  ReduceOperation op_;
  EmbeddingBagOptions opt_;
  bool version_ext_;
  std::shared_ptr<HostDeviceBlob> table_;  // shared with clones
  void* d_data_ = nullptr;
  int32_t* d_oob_ = nullptr;
  bool initialized_ = false;
  std::string namespace_;
};

class EmbeddingBagPluginCreator : public BaseCreator {
 public:
  explicit EmbeddingBagPluginCreator(bool version_ext = false);
  const char* getPluginName() const noexcept override;
  const char* getPluginVersion() const noexcept override;
  IPluginV2DynamicExt* createPlugin(const char* name, const PluginFieldCollection* fc) noexcept override;
  IPluginV2DynamicExt* deserializePlugin(const char* name, const void* serialData,
                                         size_t serialLength) noexcept override;

 private:
  bool version_ext_;
};

class EmbeddingBagPluginCreatorExt : public EmbeddingBagPluginCreator {
 public:
  EmbeddingBagPluginCreatorExt() : EmbeddingBagPluginCreator(true) {}
};

// ---- all tables of a sparse stage as one plugin --------------------------------------------------
// "EmbeddingBagGroup_TRT" / "001": T tables of one dim reduce the same number of bags in ONE
// launch and write the concatenated [B, T*dim] matrix directly.  It stands for the T
// EmbeddingBag_TRT layers plus the concatenation layer a DLRM-style graph holds (the reference
// builds one plugin layer per aten::embedding_bag node, layer_creators/trt_embedding_bag_creator.h:44-85,
// and concatenates afterwards).  Inputs: ids_0 [N_0], offsets_0 [B] or [1, B] (, weights_0 [N_0]), ids_1, ...
// Output t*dim .. (t+1)*dim-1 of every row equals what EmbeddingBag_TRT "002" gives for table t.
constexpr const char* EMBEDDING_BAG_GROUP_PLUGIN_NAME{"EmbeddingBagGroup_TRT"};
constexpr const char* EMBEDDING_BAG_GROUP_PLUGIN_VERSION{"001"};
constexpr int kMaxGroupTables = 1024;

struct EmbeddingBagGroupSpec {
  int dim = 0;
  ReduceOperation op = ReduceOperation::SUM;
  std::vector<int> count;     // rows per table
  std::vector<int> offset;    // data_offset per table
  std::vector<float> cost;    // relative cost of one bag per table (balances the per-XCD split)
  EmbeddingBagOptions opt;    // per_sample_weights: a third input per table (sum only)
  int xcd_affinity = 1;
  int n_tables() const { return (int)count.size(); }
  size_t total_rows() const {
    size_t n = 0;
    for (int c : count) n += (size_t)c;
    return n;
  }
};

class EmbeddingBagGroupPlugin final : public IPluginV2DynamicExt {
 public:
  // `tables`: the T tables back to back, table t at row sum(count[0..t)).
  EmbeddingBagGroupPlugin(std::shared_ptr<HostDeviceBlob> tables, EmbeddingBagGroupSpec spec);
  static EmbeddingBagGroupPlugin* deserialize(const void* data, size_t length);
  ~EmbeddingBagGroupPlugin() noexcept override;

  int getNbOutputs() const noexcept override;
  Dims getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept override;
  bool supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                 int nbOutputs) noexcept override;
  int configurePlugin(const DynamicPluginTensorDesc* in, int nbInputs, const DynamicPluginTensorDesc* out,
                      int nbOutputs) noexcept override;
  // Device memory for the T table descriptors of one enqueue.
  size_t getWorkspaceSize(const PluginTensorDesc* inputs, int nbInputs, const PluginTensorDesc* outputs,
                          int nbOutputs) const noexcept override;
  int initialize() noexcept override;
  void terminate() noexcept override;
  int enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc, const void* const* inputs,
              void* const* outputs, void* workspace, void* hipStream) noexcept override;
  size_t getSerializationSize() const noexcept override;
  void serialize(void* buffer) const noexcept override;
  const char* getPluginType() const noexcept override;
  const char* getPluginVersion() const noexcept override;
  void destroy() noexcept override;
  IPluginV2DynamicExt* clone() const noexcept override;
  void setPluginNamespace(const char* pluginNamespace) noexcept override;
  const char* getPluginNamespace() const noexcept override;
  DataType getOutputDataType(int index, const DataType* inputTypes, int nbInputs) const noexcept override;
  int32_t* oobFlagDevice() const noexcept override { return d_oob_; }

 private:
  int inputs_per_table() const { return spec_.opt.per_sample_weights ? 3 : 2; }
  EmbeddingBagGroupSpec spec_;
  std::shared_ptr<HostDeviceBlob> tables_;  // shared with clones
  void* d_data_ = nullptr;
  int32_t* d_oob_ = nullptr;
  bool initialized_ = false;
  std::string namespace_;
};

class EmbeddingBagGroupPluginCreator : public BaseCreator {
 public:
  EmbeddingBagGroupPluginCreator();
  const char* getPluginName() const noexcept override;
  const char* getPluginVersion() const noexcept override;
  IPluginV2DynamicExt* createPlugin(const char* name, const PluginFieldCollection* fc) noexcept override;
  IPluginV2DynamicExt* deserializePlugin(const char* name, const void* serialData,
                                         size_t serialLength) noexcept override;
};

}  // namespace fwdmi
