// Host side of the LayerNorm-family plugins (see layer_norm_plugins.h).  Reference behaviour
// cited per method; paths under source/trt_engine/trt_network_crt/.
#include "layer_norm_plugins.h"

namespace fwdmi {

namespace {

bool float_type(DataType t) { return t == DataType::kFLOAT || t == DataType::kHALF; }

// Copies `src` (fp32) into `dst` as `type` elements; returns the byte count.
size_t put_params(const std::vector<float>& src, DataType type, ByteWriter* w) {
  if (type == DataType::kHALF) {
    std::vector<uint8_t> tmp(src.size() * 2);
    f32_to_f16_bytes(src.data(), src.size(), tmp.data());
    w->bytes(tmp.data(), tmp.size());
    return tmp.size();
  }
  w->bytes(src.data(), src.size() * 4);
  return src.size() * 4;
}

bool get_params(ByteReader* r, DataType type, size_t n, std::vector<float>* out) {
  out->resize(n);
  if (type == DataType::kHALF) {
    std::vector<_Float16> tmp(n);
    if (!r->bytes(tmp.data(), n * 2)) return false;
    for (size_t i = 0; i < n; ++i) (*out)[i] = (float)tmp[i];
    return true;
  }
  return r->bytes(out->data(), n * 4);
}

// Converts fp32 rows to the plugin's table type.
std::shared_ptr<HostDeviceBlob> table_blob(const std::vector<float>& rows, DataType type) {
  if (type == DataType::kHALF) {
    std::vector<uint8_t> b(rows.size() * 2);
    f32_to_f16_bytes(rows.data(), rows.size(), b.data());
    return std::make_shared<HostDeviceBlob>(std::move(b));
  }
  return make_blob(rows.data(), rows.size() * 4);
}

}  // namespace

// ================================================================================================
//  LayerNorm / SkipLayerNorm
// ================================================================================================

// Parameters are kept in the plugin's own precision (layer_norm_plugin.cpp:34-58: mCfgType = mType,
// convertAndCopy of beta / gamma / bias).
LayerNormPluginDynamic::LayerNormPluginDynamic(std::string name, bool with_skip, DataType type, size_t ld,
                                               std::vector<float> beta, std::vector<float> gamma,
                                               std::vector<float> bias, float eps)
    : layer_name_(std::move(name)), with_skip_(with_skip), type_(type), cfg_type_(type), ld_(ld),
      has_bias_(!bias.empty()), eps_(eps), beta_(std::move(beta)), gamma_(std::move(gamma)),
      bias_(std::move(bias)) {
  if (cfg_type_ == DataType::kHALF) {
    round_through_f16(&beta_);
    round_through_f16(&gamma_);
    round_through_f16(&bias_);
  }
  std::vector<float> all;
  all.reserve(ld_ * 3);
  all.insert(all.end(), beta_.begin(), beta_.end());
  all.insert(all.end(), gamma_.begin(), gamma_.end());
  all.insert(all.end(), bias_.begin(), bias_.end());
  params_ = make_blob_f32(all);
}

LayerNormPluginDynamic::~LayerNormPluginDynamic() noexcept { terminate(); }

// Byte layout of layer_norm_plugin.cpp:257-277:
//   DataType mType(4) | DataType mCfgType(4) | size_t mLd(8) | bool mHasBias(1) |
//   beta[ld] | gamma[ld] | [bias[ld]]   (parameters in mCfgType)
// followed, only when eps != 0, by float eps(4).
size_t LayerNormPluginDynamic::getSerializationSize() const noexcept {
  const size_t ws = dtype_size((int)cfg_type_);
  return 2 * sizeof(int32_t) + sizeof(size_t) + sizeof(bool) + (has_bias_ ? 3 : 2) * ld_ * ws +
         (eps_ != 0.0f ? sizeof(float) : 0);
}

void LayerNormPluginDynamic::serialize(void* buffer) const noexcept {
  ByteWriter w(buffer);
  w.pod<int32_t>((int32_t)type_);
  w.pod<int32_t>((int32_t)cfg_type_);
  w.pod<size_t>(ld_);
  w.pod<bool>(has_bias_);
  put_params(beta_, cfg_type_, &w);
  put_params(gamma_, cfg_type_, &w);
  if (has_bias_) put_params(bias_, cfg_type_, &w);
  if (eps_ != 0.0f) w.pod<float>(eps_);
}

LayerNormPluginDynamic* LayerNormPluginDynamic::deserialize(const std::string& name, bool with_skip,
                                                           const void* data, size_t length) {
  clear_error();
  ByteReader r(data, length);
  int32_t type = -1, cfg = -1;
  size_t ld = 0;
  uint8_t bias_byte = 0;  // the reference writes a bool here; read as a byte, since any other value is not a bool to load
  r.pod(&type);
  r.pod(&cfg);
  r.pod(&ld);
  r.pod(&bias_byte);
  const bool has_bias = bias_byte != 0;
  if (!r.ok()) {
    set_error(FWDMI_ERR_TRUNCATED, "LayerNorm: serialized header truncated");
    return nullptr;
  }
  if (!float_type((DataType)type) || !float_type((DataType)cfg) || ld == 0 || ld > (size_t)1 << 24) {
    set_error(FWDMI_ERR_BAD_ARG, "LayerNorm: serialized header malformed (type %d, cfg %d, ld %zu)", type, cfg, ld);
    return nullptr;
  }
  std::vector<float> beta, gamma, bias;
  bool ok = get_params(&r, (DataType)cfg, ld, &beta) && get_params(&r, (DataType)cfg, ld, &gamma);
  if (ok && has_bias) ok = get_params(&r, (DataType)cfg, ld, &bias);
  float eps = 0.0f;
  if (ok && r.left() >= sizeof(float)) r.pod(&eps);
  if (!ok) {
    set_error(FWDMI_ERR_TRUNCATED, "LayerNorm: serialized parameters truncated");
    return nullptr;
  }
  auto* p = new LayerNormPluginDynamic(name, with_skip, (DataType)type, ld, std::move(beta), std::move(gamma),
                                       std::move(bias), eps);
  p->cfg_type_ = (DataType)cfg;
  return p;
}

// layer_norm_plugin.cpp:86-93 (the reference also calls initialize() on the clone; it is a no-op).
IPluginV2DynamicExt* LayerNormPluginDynamic::clone() const noexcept {
  auto* p = new LayerNormPluginDynamic(layer_name_, with_skip_, type_, ld_, beta_, gamma_, bias_, eps_);
  p->cfg_type_ = cfg_type_;
  p->params_ = params_;
  p->initialize();
  p->setPluginNamespace(namespace_.c_str());
  return p;
}

// Output has the shape of input 0 (layer_norm_plugin.cpp:95-101).
Dims LayerNormPluginDynamic::getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept {
  clear_error();
  if (outputIndex != 0 || !inputs || nbInputs != nb_inputs()) {
    set_error(FWDMI_ERR_BAD_ARG, "%s: output %d with %d inputs", getPluginType(), outputIndex, nbInputs);
    return error_dims();
  }
  return inputs[0];
}

// layer_norm_plugin.cpp:103-132 without the int8 branch: input 0 has the plugin's type, linear;
// every later tensor matches the one before it.
bool LayerNormPluginDynamic::supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                                       int nbOutputs) noexcept {
  if (!inOut || nbInputs != nb_inputs() || nbOutputs != 1 || pos < 0 || pos >= nbInputs + nbOutputs) return false;
  const PluginTensorDesc& in = inOut[pos];
  if (pos == 0) return in.type == (int32_t)type_ && in.format == FWDMI_FORMAT_LINEAR;
  const PluginTensorDesc& prev = inOut[pos - 1];
  return in.type == prev.type && in.format == prev.format;
}

// Uploads beta / gamma / bias (layer_norm_plugin.cpp:134-162).
int LayerNormPluginDynamic::configurePlugin(const DynamicPluginTensorDesc* in, int nbInputs,
                                            const DynamicPluginTensorDesc*, int nbOutputs) noexcept {
  clear_error();
  if (!in || nbInputs != nb_inputs() || nbOutputs != 1)
    return set_error(FWDMI_ERR_BAD_ARG, "%s::configurePlugin: %d inputs, %d outputs", getPluginType(), nbInputs,
                     nbOutputs);
  if (in[0].desc.type != (int32_t)type_)
    return set_error(FWDMI_ERR_UNSUPPORTED, "%s: input type %d differs from type_id %d", getPluginType(),
                     in[0].desc.type, (int)type_);
  if (configured_) return FWDMI_OK;
  void* p = nullptr;
  int rc = params_->acquire(&p);
  if (rc != FWDMI_OK) return rc;
  d_params_ = static_cast<float*>(p);
  configured_ = true;
  return FWDMI_OK;
}

size_t LayerNormPluginDynamic::getWorkspaceSize(const PluginTensorDesc*, int, const PluginTensorDesc*, int) const noexcept {
  return 0;
}

// layer_norm_plugin.cpp:171-229: the kernel wrapper's status is returned; a type that is neither
// float nor half yields -1.
int LayerNormPluginDynamic::enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc*,
                                    const void* const* inputs, void* const* outputs, void*,
                                    void* hipStream) noexcept {
  clear_error();
  if (!inputDesc || !inputs || !outputs) return set_error(FWDMI_ERR_BAD_ARG, "%s::enqueue: null argument", getPluginType());
  if (!configured_) return set_error(FWDMI_ERR_NOT_CONFIGURED, "%s::enqueue before configurePlugin", getPluginType());
  const int32_t t = inputDesc[0].type;
  if (t != FWDMI_F32 && t != FWDMI_F16)
    return set_error(FWDMI_ERR_UNSUPPORTED, "Unsupported type error, expected [kHALF,kFLOAT], but received %d.", t);
  const int64_t n = volume(inputDesc[0].dims);
  const float* beta = d_params_;
  const float* gamma = d_params_ + ld_;
  const float* bias = has_bias_ ? d_params_ + 2 * ld_ : nullptr;
  if (with_skip_)
    return fwdmi_skip_layer_norm(hipStream, (int)ld_, n, inputs[0], inputs[1], beta, gamma, outputs[0], bias, t, eps_);
  return fwdmi_layer_norm(hipStream, (int)ld_, n, inputs[0], beta, gamma, outputs[0], bias, t, eps_);
}

DataType LayerNormPluginDynamic::getOutputDataType(int, const DataType* inputTypes, int nbInputs) const noexcept {
  return (inputTypes && nbInputs > 0) ? inputTypes[0] : type_;
}

const char* LayerNormPluginDynamic::getPluginType() const noexcept {
  return with_skip_ ? SKIP_LAYER_NORM_NAME : FWD_LAYER_NORM_NAME;
}
const char* LayerNormPluginDynamic::getPluginVersion() const noexcept {
  return with_skip_ ? SKIP_LAYER_NORM_VERSION : FWD_LAYER_NORM_VERSION;
}
int LayerNormPluginDynamic::getNbOutputs() const noexcept { return 1; }
int LayerNormPluginDynamic::initialize() noexcept { return 0; }
void LayerNormPluginDynamic::terminate() noexcept {
  if (!configured_) return;
  params_->release();
  d_params_ = nullptr;
  configured_ = false;
}
void LayerNormPluginDynamic::destroy() noexcept { delete this; }
void LayerNormPluginDynamic::setPluginNamespace(const char* ns) noexcept { namespace_ = ns ? ns : ""; }
const char* LayerNormPluginDynamic::getPluginNamespace() const noexcept { return namespace_.c_str(); }

// ---- creators ----------------------------------------------------------------------------------
LayerNormCreatorBase::LayerNormCreatorBase(bool with_skip) : with_skip_(with_skip) {
  declare("ld", PluginFieldType::kINT32);
  declare("type_id", PluginFieldType::kINT32);
  declare("beta", PluginFieldType::kFLOAT32);
  declare("gamma", PluginFieldType::kFLOAT32);
  declare("bias", PluginFieldType::kFLOAT32);
  declare("eps", PluginFieldType::kFLOAT32);
}

// Field handling of layer_norm_plugin.cpp:316-376: ld, type_id, beta, gamma, optional bias; any
// other field (the second caller sends has_skip and batch_size, trt_normalization_creator.h:156-157)
// is ignored.  Invalid values yield nullptr with a message instead of a log line.
IPluginV2DynamicExt* LayerNormCreatorBase::createPlugin(const char* name, const PluginFieldCollection* fc) noexcept {
  clear_error();
  if (!fc || (fc->nbFields > 0 && !fc->fields)) {
    set_error(FWDMI_ERR_BAD_ARG, "%s: null field collection", getPluginName());
    return nullptr;
  }
  int ld = 0, type_id = -1;
  float eps = 0.0f;
  std::vector<float> beta, gamma, bias;
  for (int i = 0; i < fc->nbFields; ++i) {
    const PluginField& f = fc->fields[i];
    const std::string field_name = f.name ? f.name : "";
    bool ok = true;
    if (field_name == "ld") ok = f.data && f.type == FWDMI_FIELD_I32, ld = ok ? *static_cast<const int*>(f.data) : 0;
    else if (field_name == "type_id") ok = f.data && f.type == FWDMI_FIELD_I32, type_id = ok ? *static_cast<const int*>(f.data) : -1;
    else if (field_name == "eps") ok = f.data && f.type == FWDMI_FIELD_F32, eps = ok ? *static_cast<const float*>(f.data) : 0.0f;
    else if (field_name == "beta") ok = field_to_f32(f, &beta);
    else if (field_name == "gamma") ok = field_to_f32(f, &gamma);
    else if (field_name == "bias") ok = field_to_f32(f, &bias);
    if (!ok) {
      set_error(FWDMI_ERR_BAD_ARG, "%s: field '%s' has the wrong type or no data", getPluginName(), field_name.c_str());
      return nullptr;
    }
  }
  if (type_id == FWDMI_I8) {
    set_error(FWDMI_ERR_UNSUPPORTED, "%s: int8 (type_id 2) is not supported", getPluginName());
    return nullptr;
  }
  if (type_id != FWDMI_F32 && type_id != FWDMI_F16) {
    set_error(FWDMI_ERR_BAD_ARG, "%s: Invalid type ID: %d", getPluginName(), type_id);
    return nullptr;
  }
  if (ld <= 0 || beta.size() != (size_t)ld || gamma.size() != (size_t)ld || (!bias.empty() && bias.size() != (size_t)ld)) {
    set_error(FWDMI_ERR_BAD_ARG, "%s: ld=%d but beta/gamma/bias hold %zu/%zu/%zu values", getPluginName(), ld,
              beta.size(), gamma.size(), bias.size());
    return nullptr;
  }
  auto* p = new LayerNormPluginDynamic(name ? name : "", with_skip_, (DataType)type_id, (size_t)ld, std::move(beta),
                                       std::move(gamma), std::move(bias), eps);
  p->setPluginNamespace(mNamespace.c_str());
  return p;
}

IPluginV2DynamicExt* LayerNormCreatorBase::deserializePlugin(const char* name, const void* serialData,
                                                             size_t serialLength) noexcept {
  auto* p = LayerNormPluginDynamic::deserialize(name ? name : "", with_skip_, serialData, serialLength);
  if (p) p->setPluginNamespace(mNamespace.c_str());
  return p;
}

// ================================================================================================
//  EmbLayerNorm
// ================================================================================================

EmbLayerNormPluginDynamic::EmbLayerNormPluginDynamic(std::string name, DataType type, DataType mha_type, int ld,
                                                     Tables tables, float eps, bool batch_major)
    : layer_name_(std::move(name)), type_(type), mha_type_(mha_type), ld_(ld), eps_(eps),
      batch_major_(batch_major), t_(std::move(tables)) {
  std::vector<float> all(t_.beta);
  all.insert(all.end(), t_.gamma.begin(), t_.gamma.end());
  if (t_.fused_skip) {
    all.insert(all.end(), t_.beta2.begin(), t_.beta2.end());
    all.insert(all.end(), t_.gamma2.begin(), t_.gamma2.end());
    all.insert(all.end(), t_.bias2.begin(), t_.bias2.end());
  }
  params_ = make_blob_f32(all);
}

EmbLayerNormPluginDynamic::~EmbLayerNormPluginDynamic() noexcept { terminate(); }

IPluginV2DynamicExt* EmbLayerNormPluginDynamic::clone() const noexcept {
  auto* p = new EmbLayerNormPluginDynamic(layer_name_, type_, mha_type_, ld_, t_, eps_, batch_major_);
  p->params_ = params_;
  p->setPluginNamespace(namespace_.c_str());
  return p;
}

// Inputs are three [S, B] id tensors (trt_bert_creator.h:64-71).  Output 0 is the embedding
// consumed as [S, B, H, 1, 1] (plugins/common/plugin_common.h:39-41); output 1 is the mask index,
// one int per batch row in the unfused layout (plugin_common.h:63,77-94).  With the optional
// `batch_major` field the ids are [B, S] and output 0 is [B, S, H, 1, 1].  A plugin that also stands for
// the SkipLayerNorm behind it (fields skip_beta / skip_gamma, trt_bert_creator.h:199-239) takes that
// layer's second input, the residual, as its fourth: shaped like output 0 ([.., .., H] or [.., .., H, 1, 1]).
Dims EmbLayerNormPluginDynamic::getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept {
  clear_error();
  if (!inputs || nbInputs != nb_inputs() || outputIndex < 0 || outputIndex > 1) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: output %d with %d inputs (the plugin takes %d)", outputIndex, nbInputs,
              nb_inputs());
    return error_dims();
  }
  if (t_.fused_skip) {
    const Dims& r = inputs[3];
    bool ok = (r.nbDims == 3 || r.nbDims == 5) && r.d[0] == inputs[0].d[0] && r.d[1] == inputs[0].d[1] && r.d[2] == ld_;
    for (int i = 3; ok && i < r.nbDims; ++i) ok = r.d[i] == 1;
    if (!ok) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: the residual input must be shaped like the embedding output");
      return error_dims();
    }
  }
  for (int i = 0; i < 3; ++i)
    if (inputs[i].nbDims != 2 || inputs[i].d[0] != inputs[0].d[0] || inputs[i].d[1] != inputs[0].d[1]) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: inputs must be three [S, B] tensors of equal shape");
      return error_dims();
    }
  Dims out{};
  if (outputIndex == 0) {
    out.nbDims = 5;
    out.d[0] = inputs[0].d[0];
    out.d[1] = inputs[0].d[1];
    out.d[2] = ld_;
    out.d[3] = 1;
    out.d[4] = 1;
  } else {
    out.nbDims = 2;
    out.d[0] = inputs[0].d[batch_major_ ? 0 : BDIM];
    out.d[1] = 1;
  }
  return out;
}

bool EmbLayerNormPluginDynamic::supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                                          int nbOutputs) noexcept {
  if (!inOut || nbInputs != nb_inputs() || nbOutputs != 2 || pos < 0 || pos >= nbInputs + 2) return false;
  const PluginTensorDesc& d = inOut[pos];
  if (d.format != FWDMI_FORMAT_LINEAR) return false;
  if (pos == nbInputs || (t_.fused_skip && pos == 3)) return d.type == (int32_t)type_;  // output 0, the residual
  return d.type == FWDMI_I32;
}

int EmbLayerNormPluginDynamic::configurePlugin(const DynamicPluginTensorDesc* in, int nbInputs,
                                               const DynamicPluginTensorDesc*, int nbOutputs) noexcept {
  clear_error();
  if (!in || nbInputs != nb_inputs() || nbOutputs != 2)
    return set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm::configurePlugin: %d inputs, %d outputs", nbInputs, nbOutputs);
  if (configured_) return FWDMI_OK;
  void* p = nullptr;
  int rc = params_->acquire(&p);
  if (rc != FWDMI_OK) return rc;
  d_params_ = static_cast<float*>(p);
  int got = 0;
  if ((rc = t_.word->acquire(&d_word_)) == FWDMI_OK) ++got;
  if (rc == FWDMI_OK && (rc = t_.pos->acquire(&d_pos_)) == FWDMI_OK) ++got;
  if (rc == FWDMI_OK && (rc = t_.tok->acquire(&d_tok_)) == FWDMI_OK) ++got;
  if (rc == FWDMI_OK) {
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&d_oob_), sizeof(int32_t));
    if (e == hipSuccess) e = hipMemset(d_oob_, 0, sizeof(int32_t));
    if (e != hipSuccess) rc = set_error(FWDMI_ERR_HIP, "EmbLayerNorm: flag allocation failed: %s", hipGetErrorString(e));
  }
  if (rc != FWDMI_OK) {
    if (got > 2) t_.tok->release();
    if (got > 1) t_.pos->release();
    if (got > 0) t_.word->release();
    params_->release();
    if (d_oob_) (void)hipFree(d_oob_);
    d_oob_ = nullptr;
    return rc;
  }
  configured_ = true;
  return FWDMI_OK;
}

size_t EmbLayerNormPluginDynamic::getWorkspaceSize(const PluginTensorDesc*, int, const PluginTensorDesc*, int) const noexcept {
  return 0;
}

int EmbLayerNormPluginDynamic::enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc,
                                       const void* const* inputs, void* const* outputs, void*,
                                       void* hipStream) noexcept {
  clear_error();
  if (!inputDesc || !outputDesc || !inputs || !outputs) return set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm::enqueue: null argument");
  if (!configured_) return set_error(FWDMI_ERR_NOT_CONFIGURED, "EmbLayerNorm::enqueue before configurePlugin");
  if (inputDesc[0].type != FWDMI_I32 || outputDesc[0].type != (int32_t)type_)
    return set_error(FWDMI_ERR_UNSUPPORTED, "EmbLayerNorm: unsupported types (ids %d, output %d)", inputDesc[0].type,
                     outputDesc[0].type);
  const int S = inputDesc[0].dims.d[batch_major_ ? 1 : SDIM], B = inputDesc[0].dims.d[batch_major_ ? 0 : BDIM];
  fwdmi_emb_ext ext{};
  ext.batch_major = batch_major_ ? 1 : 0;
  if (t_.fused_skip) {
    if (inputDesc[3].type != (int32_t)type_)
      return set_error(FWDMI_ERR_UNSUPPORTED, "EmbLayerNorm: the residual input has type %d, the output %d",
                       inputDesc[3].type, (int32_t)type_);
    ext.skip = inputs[3];
    ext.beta2 = d_params_ + 2 * (size_t)ld_;
    ext.gamma2 = d_params_ + 3 * (size_t)ld_;
    ext.bias2 = t_.bias2.empty() ? nullptr : d_params_ + 4 * (size_t)ld_;
    ext.eps2 = t_.eps2;
  }
  return fwdmi_emb_layer_norm_ex(hipStream, S, B, ld_, static_cast<const int32_t*>(inputs[0]),
                                 static_cast<const int32_t*>(inputs[1]), static_cast<const int32_t*>(inputs[2]),
                                 d_params_, d_params_ + ld_, d_word_, d_pos_, d_tok_, t_.word_count, t_.pos_count,
                                 t_.tok_count, outputs[0], static_cast<int32_t*>(outputs[1]), (int32_t)type_, eps_,
                                 d_oob_, &ext);
}

DataType EmbLayerNormPluginDynamic::getOutputDataType(int index, const DataType*, int) const noexcept {
  return index == 0 ? type_ : DataType::kINT32;
}
const char* EmbLayerNormPluginDynamic::getPluginType() const noexcept { return EMB_LAYER_NORM_NAME; }
const char* EmbLayerNormPluginDynamic::getPluginVersion() const noexcept { return EMB_LAYER_NORM_VERSION; }
int EmbLayerNormPluginDynamic::getNbOutputs() const noexcept { return 2; }
int EmbLayerNormPluginDynamic::initialize() noexcept { return 0; }
void EmbLayerNormPluginDynamic::terminate() noexcept {
  if (!configured_) return;
  t_.tok->release();
  t_.pos->release();
  t_.word->release();
  params_->release();
  if (d_oob_) (void)hipFree(d_oob_);
  d_oob_ = nullptr;
  d_params_ = nullptr;
  d_word_ = d_pos_ = d_tok_ = nullptr;
  configured_ = false;
}

// Own layout (the NVIDIA plugin's bytes are not part of the reference tree):
//   int type | int mha_type | int ld | int word_count | int pos_count | int tok_count | float eps |
//   beta f32[ld] | gamma f32[ld] | word[word_count*ld] | pos[pos_count*ld] | tok[tok_count*ld]
// followed, only for a batch-major plugin or one that also stands for the SkipLayerNorm behind it, by
// int batch_major, and for the latter by int 1 | float eps2 | int has_bias2 | beta2 f32[ld] | gamma2 f32[ld] [| bias2 f32[ld]].
size_t EmbLayerNormPluginDynamic::getSerializationSize() const noexcept {
  size_t n = 6 * sizeof(int32_t) + sizeof(float) + 2 * (size_t)ld_ * sizeof(float) + t_.word->size() +
             t_.pos->size() + t_.tok->size() + ((batch_major_ || t_.fused_skip) ? sizeof(int32_t) : 0);
  if (t_.fused_skip)
    n += 2 * sizeof(int32_t) + sizeof(float) + (2 + (t_.bias2.empty() ? 0 : 1)) * (size_t)ld_ * sizeof(float);
  return n;
}

void EmbLayerNormPluginDynamic::serialize(void* buffer) const noexcept {
  ByteWriter w(buffer);
  w.pod<int32_t>((int32_t)type_);
  w.pod<int32_t>((int32_t)mha_type_);
  w.pod<int32_t>(ld_);
  w.pod<int32_t>(t_.word_count);
  w.pod<int32_t>(t_.pos_count);
  w.pod<int32_t>(t_.tok_count);
  w.pod<float>(eps_);
  w.bytes(t_.beta.data(), t_.beta.size() * 4);
  w.bytes(t_.gamma.data(), t_.gamma.size() * 4);
  w.bytes(t_.word->data(), t_.word->size());
  w.bytes(t_.pos->data(), t_.pos->size());
  w.bytes(t_.tok->data(), t_.tok->size());
  if (batch_major_ || t_.fused_skip) w.pod<int32_t>(batch_major_ ? 1 : 0);
  if (t_.fused_skip) {
    w.pod<int32_t>(1);
    w.pod<float>(t_.eps2);
    w.pod<int32_t>(t_.bias2.empty() ? 0 : 1);
    w.bytes(t_.beta2.data(), t_.beta2.size() * 4);
    w.bytes(t_.gamma2.data(), t_.gamma2.size() * 4);
    w.bytes(t_.bias2.data(), t_.bias2.size() * 4);
  }
}

EmbLayerNormPluginDynamic* EmbLayerNormPluginDynamic::deserialize(const std::string& name, const void* data,
                                                                 size_t length) {
  clear_error();
  ByteReader r(data, length);
  int32_t type = -1, mha = -1, ld = 0;
  Tables t;
  float eps = 0.0f;
  r.pod(&type);
  r.pod(&mha);
  r.pod(&ld);
  r.pod(&t.word_count);
  r.pod(&t.pos_count);
  r.pod(&t.tok_count);
  r.pod(&eps);
  if (!r.ok()) {
    set_error(FWDMI_ERR_TRUNCATED, "EmbLayerNorm: serialized header truncated");
    return nullptr;
  }
  // ld is bounded as in the LayerNorm plugin, so that the size below cannot wrap 64 bits
  // (3 x 2^31 rows x 2^24 x 4 bytes < 2^59)
  if (!float_type((DataType)type) || ld <= 0 || ld > (1 << 24) || t.word_count <= 0 || t.pos_count <= 0 ||
      t.tok_count <= 0) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: serialized header malformed");
    return nullptr;
  }
  const size_t es = dtype_size(type);
  const size_t need = 2 * (size_t)ld * 4 + ((size_t)t.word_count + t.pos_count + t.tok_count) * ld * es;
  if (r.left() < need) {
    set_error(FWDMI_ERR_TRUNCATED, "EmbLayerNorm: serialized tables truncated");
    return nullptr;
  }
  t.beta.resize(ld);
  t.gamma.resize(ld);
  r.bytes(t.beta.data(), (size_t)ld * 4);
  r.bytes(t.gamma.data(), (size_t)ld * 4);
  auto read_table = [&](int rows) {
    std::vector<uint8_t> b((size_t)rows * ld * es);
    r.bytes(b.data(), b.size());
    return std::make_shared<HostDeviceBlob>(std::move(b));
  };
  t.word = read_table(t.word_count);
  t.pos = read_table(t.pos_count);
  t.tok = read_table(t.tok_count);
  int32_t batch_major = 0;
  if (r.left() >= sizeof(int32_t)) r.pod(&batch_major);
  if (r.left() > 0) {  // the SkipLayerNorm the plugin also stands for
    int32_t fused = 0, has_bias = 0;
    r.pod(&fused);
    r.pod(&t.eps2);
    r.pod(&has_bias);
    if (!r.ok() || fused != 1 || (has_bias != 0 && has_bias != 1) || r.left() != (size_t)(2 + has_bias) * ld * 4) {
      set_error(FWDMI_ERR_TRUNCATED, "EmbLayerNorm: serialized second stage truncated or malformed");
      return nullptr;
    }
    t.fused_skip = true;
    t.beta2.resize(ld);
    t.gamma2.resize(ld);
    r.bytes(t.beta2.data(), (size_t)ld * 4);
    r.bytes(t.gamma2.data(), (size_t)ld * 4);
    if (has_bias) {
      t.bias2.resize(ld);
      r.bytes(t.bias2.data(), (size_t)ld * 4);
    }
  }
  if (!r.ok()) {
    set_error(FWDMI_ERR_TRUNCATED, "EmbLayerNorm: serialized tables truncated");
    return nullptr;
  }
  return new EmbLayerNormPluginDynamic(name, (DataType)type, (DataType)mha, ld, std::move(t), eps, batch_major != 0);
}

void EmbLayerNormPluginDynamic::destroy() noexcept { delete this; }
void EmbLayerNormPluginDynamic::setPluginNamespace(const char* ns) noexcept { namespace_ = ns ? ns : ""; }
const char* EmbLayerNormPluginDynamic::getPluginNamespace() const noexcept { return namespace_.c_str(); }

// Fields as the reference's caller fills them (trt_bert_creator.h:130-141, names :515-521).
EmbLayerNormPluginDynamicCreator::EmbLayerNormPluginDynamicCreator() {
  declare("bert_embeddings_layernorm_beta", PluginFieldType::kFLOAT32);
  declare("bert_embeddings_layernorm_gamma", PluginFieldType::kFLOAT32);
  declare("bert_embeddings_word_embeddings", PluginFieldType::kFLOAT32);
  declare("bert_embeddings_token_type_embeddings", PluginFieldType::kFLOAT32);
  declare("bert_embeddings_position_embeddings", PluginFieldType::kFLOAT32);
  declare("output_fp16", PluginFieldType::kINT32);
  declare("mha_type_id", PluginFieldType::kINT32);
  declare("eps", PluginFieldType::kFLOAT32);
  declare("batch_major", PluginFieldType::kINT32);
  // the SkipLayerNorm behind the embedding (its own fields are beta / gamma / bias, trt_bert_creator.h:219-229)
  declare("skip_beta", PluginFieldType::kFLOAT32);
  declare("skip_gamma", PluginFieldType::kFLOAT32);
  declare("skip_bias", PluginFieldType::kFLOAT32);
  declare("skip_eps", PluginFieldType::kFLOAT32);
}

IPluginV2DynamicExt* EmbLayerNormPluginDynamicCreator::createPlugin(const char* name,
                                                                    const PluginFieldCollection* fc) noexcept {
  clear_error();
  if (!fc || (fc->nbFields > 0 && !fc->fields)) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: null field collection");
    return nullptr;
  }
  std::vector<float> beta, gamma, word, tok, pos, beta2, gamma2, bias2;
  int output_fp16 = 0, mha_type = 0, batch_major = 0;
  float eps = 0.0f, eps2 = 0.0f;
  for (int i = 0; i < fc->nbFields; ++i) {
    const PluginField& f = fc->fields[i];
    const std::string n = f.name ? f.name : "";
    bool ok = true;
    if (n == "batch_major") ok = f.data && f.type == FWDMI_FIELD_I32, batch_major = ok ? *static_cast<const int*>(f.data) : 0;
    else if (n == "bert_embeddings_layernorm_beta") ok = field_to_f32(f, &beta);
    else if (n == "bert_embeddings_layernorm_gamma") ok = field_to_f32(f, &gamma);
    else if (n == "bert_embeddings_word_embeddings") ok = field_to_f32(f, &word);
    else if (n == "bert_embeddings_token_type_embeddings") ok = field_to_f32(f, &tok);
    else if (n == "bert_embeddings_position_embeddings") ok = field_to_f32(f, &pos);
    else if (n == "output_fp16") ok = f.data && f.type == FWDMI_FIELD_I32, output_fp16 = ok ? *static_cast<const int*>(f.data) : 0;
    else if (n == "mha_type_id") ok = f.data && f.type == FWDMI_FIELD_I32, mha_type = ok ? *static_cast<const int*>(f.data) : 0;
    else if (n == "eps") ok = f.data && f.type == FWDMI_FIELD_F32, eps = ok ? *static_cast<const float*>(f.data) : 0.0f;
    else if (n == "skip_beta") ok = field_to_f32(f, &beta2);
    else if (n == "skip_gamma") ok = field_to_f32(f, &gamma2);
    else if (n == "skip_bias") ok = field_to_f32(f, &bias2);
    else if (n == "skip_eps") ok = f.data && f.type == FWDMI_FIELD_F32, eps2 = ok ? *static_cast<const float*>(f.data) : 0.0f;
    if (!ok) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: field '%s' has the wrong type or no data", n.c_str());
      return nullptr;
    }
  }
  const size_t ld = beta.size();
  if (ld == 0 || gamma.size() != ld || word.empty() || pos.empty() || tok.empty() || word.size() % ld ||
      pos.size() % ld || tok.size() % ld) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: inconsistent sizes (beta %zu, gamma %zu, word %zu, pos %zu, tok %zu)",
              beta.size(), gamma.size(), word.size(), pos.size(), tok.size());
    return nullptr;
  }
  const bool fused = !beta2.empty() || !gamma2.empty() || !bias2.empty();
  if (fused && (beta2.size() != ld || gamma2.size() != ld || (!bias2.empty() && bias2.size() != ld))) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbLayerNorm: skip_beta / skip_gamma (/ skip_bias) must hold %zu values each", ld);
    return nullptr;
  }
  const DataType type = output_fp16 ? DataType::kHALF : DataType::kFLOAT;
  EmbLayerNormPluginDynamic::Tables t;
  t.fused_skip = fused;
  t.beta2 = std::move(beta2);
  t.gamma2 = std::move(gamma2);
  t.bias2 = std::move(bias2);
  t.eps2 = eps2;
  t.word_count = (int)(word.size() / ld);
  t.pos_count = (int)(pos.size() / ld);
  t.tok_count = (int)(tok.size() / ld);
  t.word = table_blob(word, type);
  t.pos = table_blob(pos, type);
  t.tok = table_blob(tok, type);
  t.beta = std::move(beta);
  t.gamma = std::move(gamma);
  auto* p = new EmbLayerNormPluginDynamic(name ? name : "", type, (DataType)mha_type, (int)ld, std::move(t), eps,
                                          batch_major != 0);
  p->setPluginNamespace(mNamespace.c_str());
  return p;
}

IPluginV2DynamicExt* EmbLayerNormPluginDynamicCreator::deserializePlugin(const char* name, const void* serialData,
                                                                         size_t serialLength) noexcept {
  auto* p = EmbLayerNormPluginDynamic::deserialize(name ? name : "", serialData, serialLength);
  if (p) p->setPluginNamespace(mNamespace.c_str());
  return p;
}

FWDMI_REGISTER_PLUGIN(LayerNormPluginDynamicCreator);
FWDMI_REGISTER_PLUGIN(SkipLayerNormPluginDynamicCreator);
FWDMI_REGISTER_PLUGIN(EmbLayerNormPluginDynamicCreator);

}  // namespace fwdmi
