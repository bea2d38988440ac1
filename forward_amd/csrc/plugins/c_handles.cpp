// Opaque-handle C view of the plugin classes (section 2 of fwdmi.h).
#include "plugin_util.h"

using namespace fwdmi;

namespace {
inline IPluginV2DynamicExt* P(fwdmi_plugin* p) { return reinterpret_cast<IPluginV2DynamicExt*>(p); }
inline IPluginCreator* C(fwdmi_creator* c) { return reinterpret_cast<IPluginCreator*>(c); }
inline fwdmi_plugin* H(IPluginV2DynamicExt* p) { return reinterpret_cast<fwdmi_plugin*>(p); }

std::vector<DynamicPluginTensorDesc> dynamic_descs(const fwdmi_tensor_desc* d, int n) {
  std::vector<DynamicPluginTensorDesc> v(n > 0 ? n : 0);
  for (int i = 0; i < n; ++i) v[i] = DynamicPluginTensorDesc{d[i], d[i].dims, d[i].dims};
  return v;
}
}  // namespace

extern "C" {

fwdmi_creator* fwdmi_get_plugin_creator(const char* name, const char* version) {
  return reinterpret_cast<fwdmi_creator*>(getPluginRegistry()->getPluginCreator(name, version, ""));
}

int fwdmi_registry_size(void) {
  int n = 0;
  getPluginRegistry()->getPluginCreatorList(&n);
  return n;
}

fwdmi_creator* fwdmi_registry_at(int i) {
  int n = 0;
  IPluginCreator* const* list = getPluginRegistry()->getPluginCreatorList(&n);
  return (i >= 0 && i < n) ? reinterpret_cast<fwdmi_creator*>(list[i]) : nullptr;
}

const char* fwdmi_creator_name(fwdmi_creator* c) { return c ? C(c)->getPluginName() : nullptr; }
const char* fwdmi_creator_version(fwdmi_creator* c) { return c ? C(c)->getPluginVersion() : nullptr; }
int fwdmi_creator_num_fields(fwdmi_creator* c) { return c ? C(c)->getFieldNames()->nbFields : FWDMI_ERR_BAD_ARG; }

const char* fwdmi_creator_field_name(fwdmi_creator* c, int i) {
  if (!c) return nullptr;
  const PluginFieldCollection* fc = C(c)->getFieldNames();
  return (i >= 0 && i < fc->nbFields) ? fc->fields[i].name : nullptr;
}

int fwdmi_creator_field_type(fwdmi_creator* c, int i) {
  if (!c) return FWDMI_ERR_BAD_ARG;
  const PluginFieldCollection* fc = C(c)->getFieldNames();
  return (i >= 0 && i < fc->nbFields) ? fc->fields[i].type : FWDMI_ERR_BAD_ARG;
}

fwdmi_plugin* fwdmi_creator_create_plugin(fwdmi_creator* c, const char* name, const fwdmi_plugin_field* fields,
                                          int n_fields) {
  if (!c) {
    set_error(FWDMI_ERR_BAD_ARG, "create_plugin: null creator");
    return nullptr;
  }
  PluginFieldCollection fc{n_fields, fields};
  return H(C(c)->createPlugin(name, &fc));
}

fwdmi_plugin* fwdmi_creator_deserialize_plugin(fwdmi_creator* c, const char* name, const void* data, size_t length) {
  if (!c || (!data && length)) {
    set_error(FWDMI_ERR_BAD_ARG, "deserialize_plugin: null argument");
    return nullptr;
  }
  return H(C(c)->deserializePlugin(name, data, length));
}

int fwdmi_plugin_get_nb_outputs(fwdmi_plugin* p) { return p ? P(p)->getNbOutputs() : FWDMI_ERR_BAD_ARG; }

int fwdmi_plugin_get_output_dimensions(fwdmi_plugin* p, int output_index, const fwdmi_dims* inputs, int nb_inputs,
                                       fwdmi_dims* out) {
  if (!p || !out) return set_error(FWDMI_ERR_BAD_ARG, "get_output_dimensions: null argument");
  const Dims d = P(p)->getOutputDimensions(output_index, inputs, nb_inputs);
  if (d.nbDims < 0) return FWDMI_ERR_BAD_ARG;
  *out = d;
  return FWDMI_OK;
}

int fwdmi_plugin_supports_format_combination(fwdmi_plugin* p, int pos, const fwdmi_tensor_desc* in_out, int nb_inputs,
                                             int nb_outputs) {
  if (!p || !in_out) return FWDMI_ERR_BAD_ARG;
  return P(p)->supportsFormatCombination(pos, in_out, nb_inputs, nb_outputs) ? 1 : 0;
}

int fwdmi_plugin_configure(fwdmi_plugin* p, const fwdmi_tensor_desc* in, int nb_inputs, const fwdmi_tensor_desc* out,
                           int nb_outputs) {
  if (!p || (nb_inputs > 0 && !in) || (nb_outputs > 0 && !out))
    return set_error(FWDMI_ERR_BAD_ARG, "configure: null argument");
  auto din = dynamic_descs(in, nb_inputs), dout = dynamic_descs(out, nb_outputs);
  return P(p)->configurePlugin(din.data(), nb_inputs, dout.data(), nb_outputs);
}

size_t fwdmi_plugin_get_workspace_size(fwdmi_plugin* p, const fwdmi_tensor_desc* in, int nb_inputs,
                                       const fwdmi_tensor_desc* out, int nb_outputs) {
  return p ? P(p)->getWorkspaceSize(in, nb_inputs, out, nb_outputs) : 0;
}

int fwdmi_plugin_initialize(fwdmi_plugin* p) { return p ? P(p)->initialize() : FWDMI_ERR_BAD_ARG; }
void fwdmi_plugin_terminate(fwdmi_plugin* p) {
  if (p) P(p)->terminate();
}

int fwdmi_plugin_enqueue(fwdmi_plugin* p, const fwdmi_tensor_desc* in_desc, const fwdmi_tensor_desc* out_desc,
                         const void* const* inputs, void* const* outputs, void* workspace, void* stream) {
  if (!p) return set_error(FWDMI_ERR_BAD_ARG, "enqueue: null plugin");
  return P(p)->enqueue(in_desc, out_desc, inputs, outputs, workspace, stream);
}

size_t fwdmi_plugin_get_serialization_size(fwdmi_plugin* p) { return p ? P(p)->getSerializationSize() : 0; }

int fwdmi_plugin_serialize(fwdmi_plugin* p, void* buffer) {
  if (!p || !buffer) return set_error(FWDMI_ERR_BAD_ARG, "serialize: null argument");
  P(p)->serialize(buffer);
  return FWDMI_OK;
}

const char* fwdmi_plugin_get_type(fwdmi_plugin* p) { return p ? P(p)->getPluginType() : nullptr; }
const char* fwdmi_plugin_get_version(fwdmi_plugin* p) { return p ? P(p)->getPluginVersion() : nullptr; }
void fwdmi_plugin_set_namespace(fwdmi_plugin* p, const char* ns) {
  if (p) P(p)->setPluginNamespace(ns);
}
const char* fwdmi_plugin_get_namespace(fwdmi_plugin* p) { return p ? P(p)->getPluginNamespace() : nullptr; }

int fwdmi_plugin_get_output_data_type(fwdmi_plugin* p, int index, const int32_t* input_types, int nb_inputs) {
  if (!p) return FWDMI_ERR_BAD_ARG;
  return (int)P(p)->getOutputDataType(index, reinterpret_cast<const DataType*>(input_types), nb_inputs);
}

fwdmi_plugin* fwdmi_plugin_clone(fwdmi_plugin* p) { return p ? H(P(p)->clone()) : nullptr; }
void fwdmi_plugin_destroy(fwdmi_plugin* p) {
  if (p) P(p)->destroy();
}

int fwdmi_plugin_take_oob_flag(fwdmi_plugin* p, void* stream) {
  if (!p) return set_error(FWDMI_ERR_BAD_ARG, "take_oob_flag: null plugin");
  int32_t* d = P(p)->oobFlagDevice();
  if (!d) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t v = 0;
  FWDMI_HIP_CHECK(hipMemcpyAsync(&v, d, sizeof(v), hipMemcpyDeviceToHost, s));
  FWDMI_HIP_CHECK(hipStreamSynchronize(s));
  if (v) {
    const int32_t zero = 0;
    FWDMI_HIP_CHECK(hipMemcpyAsync(d, &zero, sizeof(zero), hipMemcpyHostToDevice, s));
    FWDMI_HIP_CHECK(hipStreamSynchronize(s));
  }
  return v ? 1 : 0;
}

}  // extern "C"
