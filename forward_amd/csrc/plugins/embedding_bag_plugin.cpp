// Host side of the EmbeddingBag plugin: field parsing, shape / format rules, table upload,
// enqueue dispatch to the C-ABI launchers, (de)serialisation.  Reference behaviour cited per
// method (paths under source/trt_engine/trt_network_crt/plugins/embedding_bag_plugin/).
#include "embedding_bag_plugin.h"

namespace fwdmi {

namespace {

bool is_reduce_op(int v) { return v == 0 || v == 1 || v == 2 || v == 3 || v == 999; }

const fwdmi_bag_ext make_ext(const EmbeddingBagOptions& o, const void* psw, int32_t* oob, void* square_out = nullptr) {
  fwdmi_bag_ext x{};
  x.table_dtype = o.table_dtype;
  x.index_dtype = o.index_dtype;
  x.out_dtype = o.out_dtype;
  x.include_last_offset = o.include_last_offset;
  x.per_sample_weights = psw;
  x.max_indices = nullptr;
  x.out_row_stride = 0;
  x.oob_flag = oob;
  x.flags = 0;
  x.square_sum_out = square_out;
  return x;
}

}  // namespace

EmbeddingBagPlugin::EmbeddingBagPlugin(std::shared_ptr<HostDeviceBlob> table, int dim, int count, int offset,
                                       ReduceOperation op, const EmbeddingBagOptions& opt, bool version_ext)
    : dim_(dim), count_(count), data_offset_(offset), op_(op), opt_(opt), version_ext_(version_ext),
      table_(std::move(table)) {}

EmbeddingBagPlugin::~EmbeddingBagPlugin() noexcept { terminate(); }

// One output: the reduced bags (embedding_bag_plugin.cpp:55); "002" with with_square_sum: two.
int EmbeddingBagPlugin::getNbOutputs() const noexcept { return opt_.with_square_sum ? 2 : 1; }

// Shape rules of embedding_bag_plugin.cpp:57-100.
//   1 input  [B, L]           -> [B, dim]            (reduce)
//                              -> [B, L, dim]         (GATHER, dim > 1; [B, L] when dim == 1)
//   2 inputs ids [N], offsets [B] or [1, B] -> [B, dim]   (GATHER not allowed)
Dims EmbeddingBagPlugin::getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept {
  clear_error();
  if (outputIndex < 0 || outputIndex >= getNbOutputs() || !inputs || nbInputs < 1 ||
      nbInputs > (opt_.per_sample_weights ? 3 : 2)) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: output %d with %d inputs", outputIndex, nbInputs);
    return error_dims();
  }
  if (nbInputs == 1) {
    if (inputs[0].nbDims != 2) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: a single input must be 2-D, got %d-D", inputs[0].nbDims);
      return error_dims();
    }
    Dims out = inputs[0];
    if (op_ != ReduceOperation::GATHER) {
      out.d[1] = dim_;
    } else if (dim_ > 1) {
      out.nbDims = 3;
      out.d[2] = dim_;
    }
    return out;
  }
  const Dims& off = inputs[1];
  if (!(off.nbDims == 1 || (off.nbDims == 2 && off.d[0] == 1))) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: offsets must be [B] or [1, B]");
    return error_dims();
  }
  if (op_ == ReduceOperation::GATHER) {
    set_error(FWDMI_ERR_UNSUPPORTED, "EmbeddingBag: GATHER with an offsets input is not supported");
    return error_dims();
  }
  const int n_off = off.nbDims == 1 ? off.d[0] : off.d[1], trailing = opt_.include_last_offset ? 1 : 0;
  if (n_off < trailing) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: %d offsets", n_off);
    return error_dims();
  }
  Dims out{};
  out.nbDims = 2;
  out.d[0] = n_off - trailing;
  out.d[1] = dim_;
  return out;
}

// Formats of embedding_bag_plugin.cpp:102-114: integer ids in, float rows out, all linear.
// Version "002" widens the types to what its options name.
bool EmbeddingBagPlugin::supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                                   int nbOutputs) noexcept {
  const int max_inputs = opt_.per_sample_weights ? 3 : 2;
  if (!inOut || nbInputs < 1 || nbInputs > max_inputs || nbOutputs != getNbOutputs() || pos < 0 ||
      pos >= nbInputs + nbOutputs)
    return false;
  const PluginTensorDesc& d = inOut[pos];
  if (d.format != FWDMI_FORMAT_LINEAR) return false;
  if (pos >= nbInputs) return d.type == opt_.out_dtype;
  if (pos == 2) return d.type == opt_.table_dtype;  // per-sample weights
  return d.type == opt_.index_dtype;
}

// Uploads the table once (embedding_bag_plugin.cpp:116-127); clones share the device copy.
int EmbeddingBagPlugin::configurePlugin(const DynamicPluginTensorDesc*, int, const DynamicPluginTensorDesc*,
                                        int) noexcept {
  clear_error();
  if (initialized_) return FWDMI_OK;
  int rc = table_->acquire(&d_data_);
  if (rc != FWDMI_OK) return rc;
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&d_oob_), sizeof(int32_t));
  if (e == hipSuccess) e = hipMemset(d_oob_, 0, sizeof(int32_t));
  if (e != hipSuccess) {
    table_->release();
    d_data_ = nullptr;
    if (d_oob_) (void)hipFree(d_oob_);
    d_oob_ = nullptr;
    return set_error(FWDMI_ERR_HIP, "EmbeddingBag: flag allocation failed: %s", hipGetErrorString(e));
  }
  initialized_ = true;
  return FWDMI_OK;
}

size_t EmbeddingBagPlugin::getWorkspaceSize(const PluginTensorDesc*, int, const PluginTensorDesc*, int) const noexcept {
  return 0;
}

int EmbeddingBagPlugin::initialize() noexcept { return 0; }

void EmbeddingBagPlugin::terminate() noexcept {
  if (!initialized_) return;
  table_->release();
  d_data_ = nullptr;
  if (d_oob_) (void)hipFree(d_oob_);
  d_oob_ = nullptr;
  initialized_ = false;
}

// Dispatch of embedding_bag_plugin.cpp:146-189: 2-D ids -> gather or fixed-length bags,
// 1-D ids -> offsets form; an unsupported id type returns -1.
int EmbeddingBagPlugin::enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc,
                                const void* const* inputs, void* const* outputs, void*, void* hipStream) noexcept {
  clear_error();
  if (!inputDesc || !outputDesc || !inputs || !outputs)
    return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag::enqueue: null argument");
  if (!initialized_) return set_error(FWDMI_ERR_NOT_CONFIGURED, "EmbeddingBag::enqueue before configurePlugin");
  if (inputDesc[0].type != opt_.index_dtype)
    return set_error(FWDMI_ERR_UNSUPPORTED, "Unsupported input data type %d", inputDesc[0].type);

  const Dims& in0 = inputDesc[0].dims;
  if (in0.nbDims != 1 && in0.nbDims != 2)
    return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag::enqueue: ids must be 1-D or 2-D, got %d-D", in0.nbDims);
  if (in0.nbDims > 1) {
    const int64_t batch_size = in0.d[0], bag_len = in0.d[1];
    const fwdmi_bag_ext x = make_ext(opt_, nullptr, d_oob_, opt_.with_square_sum ? outputs[1] : nullptr);
    if (op_ == ReduceOperation::GATHER)
      return fwdmi_gather(inputs[0], outputs[0], batch_size, bag_len, d_data_, count_, dim_, data_offset_, &x,
                          hipStream);
    return fwdmi_embedding_bag_fixed(inputs[0], outputs[0], batch_size, bag_len, d_data_, count_, dim_,
                                     data_offset_, static_cast<int>(op_), &x, hipStream);
  }
  if (op_ == ReduceOperation::GATHER)
    return set_error(FWDMI_ERR_UNSUPPORTED, "EmbeddingBag: GATHER with an offsets input is not supported");
  const int64_t input_size = in0.d[0];
  const Dims& in1 = inputDesc[1].dims;
  if (!(in1.nbDims == 1 || (in1.nbDims == 2 && in1.d[0] == 1)))
    return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag::enqueue: offsets must be [B] or [1, B]");
  const int64_t n_off = in1.nbDims == 1 ? in1.d[0] : in1.d[1];
  const int64_t n_bags = n_off - (opt_.include_last_offset ? 1 : 0);
  const fwdmi_bag_ext x = make_ext(opt_, opt_.per_sample_weights ? inputs[2] : nullptr, d_oob_,
                                   opt_.with_square_sum ? outputs[1] : nullptr);
  return fwdmi_embedding_bag(inputs[0], inputs[1], outputs[0], input_size, n_bags, d_data_, count_, dim_,
                             data_offset_, static_cast<int>(op_), &x, hipStream);
}

// "001" bytes (embedding_bag_plugin.cpp:191-202):
//   int dim | int count | int data_offset | int op | size_t n | float[n]
// "002" bytes:
//   int dim | int count | int data_offset | int op | int table_dtype | int index_dtype |
//   int out_dtype | int include_last_offset | int per_sample_weights | int with_square_sum |
//   size_t n | elem[n]
// A "002" plugin whose table was given by file (`data_file`) writes, in place of the table,
//   size_t SIZE_MAX | size_t path_len | path bytes | uint64 byte offset in the file
// so an engine file stays small and loading maps the table instead of copying it.
size_t EmbeddingBagPlugin::getSerializationSize() const noexcept {
  const size_t head = 4 * sizeof(int) + (version_ext_ ? 6 * sizeof(int) : 0) + sizeof(size_t);
  if (table_->by_reference()) return head + sizeof(size_t) + table_->path().size() + sizeof(uint64_t);
  return head + table_->size();
}

void EmbeddingBagPlugin::serialize(void* buffer) const noexcept {
  ByteWriter w(buffer);
  w.pod<int>(dim_);
  w.pod<int>(count_);
  w.pod<int>(data_offset_);
  w.pod<int>(static_cast<int>(op_));
  if (version_ext_) {
    w.pod<int>(opt_.table_dtype);
    w.pod<int>(opt_.index_dtype);
    w.pod<int>(opt_.out_dtype);
    w.pod<int>(opt_.include_last_offset);
    w.pod<int>(opt_.per_sample_weights);
    w.pod<int>(opt_.with_square_sum);
  }
  if (table_->by_reference()) {
    w.pod<size_t>(SIZE_MAX);
    w.pod<size_t>(table_->path().size());
    w.bytes(table_->path().data(), table_->path().size());
    w.pod<uint64_t>(table_->file_offset());
    return;
  }
  const size_t es = dtype_size(opt_.table_dtype);
  w.pod<size_t>(table_->size() / es);
  w.bytes(table_->data(), table_->size());
}

EmbeddingBagPlugin* EmbeddingBagPlugin::deserialize(const void* data, size_t length, bool version_ext) {
  clear_error();
  ByteReader r(data, length);
  int dim = 0, count = 0, off = 0, op = 0;
  EmbeddingBagOptions opt;
  r.pod(&dim);
  r.pod(&count);
  r.pod(&off);
  r.pod(&op);
  if (version_ext) {
    r.pod(&opt.table_dtype);
    r.pod(&opt.index_dtype);
    r.pod(&opt.out_dtype);
    r.pod(&opt.include_last_offset);
    r.pod(&opt.per_sample_weights);
    r.pod(&opt.with_square_sum);
  }
  if (!r.ok() || !is_float_dtype(opt.table_dtype) || !is_float_dtype(opt.out_dtype) ||
      !is_index_dtype(opt.index_dtype)) {
    set_error(FWDMI_ERR_TRUNCATED, "EmbeddingBag: serialized header truncated or malformed");
    return nullptr;
  }
  if (dim <= 0 || dim > (1 << 24) || count <= 0 || !is_reduce_op(op) ||  // dim: what the launchers accept
      (opt.with_square_sum && (op != FWDMI_OP_SUM || opt.per_sample_weights))) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: serialized fields inconsistent (dim %d, count %d, op %d)", dim, count, op);
    return nullptr;
  }
  const size_t es = dtype_size(opt.table_dtype);
  {
    ByteReader peek = r;
    size_t marker = 0;
    if (version_ext && peek.pod(&marker) && marker == SIZE_MAX) {   // table by reference
      size_t path_len = 0;
      uint64_t file_off = 0;
      std::string path;
      bool ok = peek.pod(&path_len) && path_len <= peek.left();
      if (ok) {
        path.resize(path_len);
        ok = peek.bytes(&path[0], path_len) && peek.pod(&file_off);
      }
      if (!ok) {
        set_error(FWDMI_ERR_TRUNCATED, "EmbeddingBag: serialized table reference truncated");
        return nullptr;
      }
      auto blob = HostDeviceBlob::map_file(path, file_off, (size_t)dim * (size_t)count * es);
      if (!blob) return nullptr;
      return new EmbeddingBagPlugin(std::move(blob), dim, count, off, static_cast<ReduceOperation>(op), opt, true);
    }
  }
  std::vector<uint8_t> bytes;
  size_t n = 0;
  if (!r.vec(&bytes, es, &n)) {
    set_error(FWDMI_ERR_TRUNCATED, "EmbeddingBag: serialized table truncated");
    return nullptr;
  }
  if (n != (size_t)dim * (size_t)count) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: serialized fields inconsistent (dim %d, count %d, op %d, n %zu)",
              dim, count, op, n);
    return nullptr;
  }
  return new EmbeddingBagPlugin(std::make_shared<HostDeviceBlob>(std::move(bytes)), dim, count, off,
                                static_cast<ReduceOperation>(op), opt, version_ext);
}

const char* EmbeddingBagPlugin::getPluginType() const noexcept { return EMBEDDING_BAG_PLUGIN_NAME; }

const char* EmbeddingBagPlugin::getPluginVersion() const noexcept {
  return version_ext_ ? EMBEDDING_BAG_PLUGIN_VERSION_EXT : EMBEDDING_BAG_PLUGIN_VERSION;
}

void EmbeddingBagPlugin::destroy() noexcept { delete this; }

// An independent plugin object over the same table storage (the reference deep-copies the
// host table, embedding_bag_plugin.cpp:212-214; sharing it changes no observable result).
IPluginV2DynamicExt* EmbeddingBagPlugin::clone() const noexcept {
  auto* p = new EmbeddingBagPlugin(table_, dim_, count_, data_offset_, op_, opt_, version_ext_);
  p->namespace_ = namespace_;
  return p;
}

void EmbeddingBagPlugin::setPluginNamespace(const char* pluginNamespace) noexcept {
  namespace_ = pluginNamespace ? pluginNamespace : "";
}

const char* EmbeddingBagPlugin::getPluginNamespace() const noexcept { return namespace_.c_str(); }

DataType EmbeddingBagPlugin::getOutputDataType(int, const DataType*, int) const noexcept {
  return static_cast<DataType>(opt_.out_dtype);
}

// ---- creator -----------------------------------------------------------------------------------
// Declared fields of embedding_bag_plugin.cpp:229-243; "002" lists its optional ones after them.
EmbeddingBagPluginCreator::EmbeddingBagPluginCreator(bool version_ext) : version_ext_(version_ext) {
  declare("dim", PluginFieldType::kINT32);
  declare("count", PluginFieldType::kINT32);
  declare("offset", PluginFieldType::kINT32);
  declare("op", PluginFieldType::kINT32);
  declare("data", PluginFieldType::kFLOAT32);
  if (version_ext_) {
    declare("index_type", PluginFieldType::kINT32);
    declare("output_fp16", PluginFieldType::kINT32);
    declare("include_last_offset", PluginFieldType::kINT32);
    declare("per_sample_weights", PluginFieldType::kINT32);
    declare("with_square_sum", PluginFieldType::kINT32);
    declare("data_file", PluginFieldType::kCHAR);
    declare("data_file_row_offset", PluginFieldType::kINT32);
    declare("table_type", PluginFieldType::kINT32);
  }
}

const char* EmbeddingBagPluginCreator::getPluginName() const noexcept { return EMBEDDING_BAG_PLUGIN_NAME; }

const char* EmbeddingBagPluginCreator::getPluginVersion() const noexcept {
  return version_ext_ ? EMBEDDING_BAG_PLUGIN_VERSION_EXT : EMBEDDING_BAG_PLUGIN_VERSION;
}

// Field contract of embedding_bag_plugin.cpp:257-293: exactly {dim,count,offset,op,data} for
// "001" (a different count or an unknown name is a contract violation; here it yields nullptr
// and an error message instead of abort()).
IPluginV2DynamicExt* EmbeddingBagPluginCreator::createPlugin(const char*, const PluginFieldCollection* fc) noexcept {
  clear_error();
  if (!fc || (fc->nbFields > 0 && !fc->fields)) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: null field collection");
    return nullptr;
  }
  if (!version_ext_ && fc->nbFields != 5) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: expected 5 fields, got %d", fc->nbFields);
    return nullptr;
  }
  int dim = 0, count = 0, offset = 0, op = -1, file_row_offset = 0, table_type = -1;
  bool have[5] = {false, false, false, false, false};
  const PluginField* data = nullptr;
  std::string data_file;
  EmbeddingBagOptions opt;
  for (int i = 0; i < fc->nbFields; ++i) {
    const PluginField& f = fc->fields[i];
    const std::string name = f.name ? f.name : "";
    int* scalar = nullptr;
    int slot = -1;
    if (name == "dim") scalar = &dim, slot = 0;
    else if (name == "count") scalar = &count, slot = 1;
    else if (name == "offset") scalar = &offset, slot = 2;
    else if (name == "op") scalar = &op, slot = 3;
    else if (version_ext_ && name == "include_last_offset") scalar = &opt.include_last_offset;
    else if (version_ext_ && name == "per_sample_weights") scalar = &opt.per_sample_weights;
    else if (version_ext_ && name == "with_square_sum") scalar = &opt.with_square_sum;
    else if (version_ext_ && name == "index_type") scalar = &opt.index_dtype;
    else if (version_ext_ && name == "data_file_row_offset") scalar = &file_row_offset;
    else if (version_ext_ && name == "table_type") scalar = &table_type;
    if (scalar) {
      if (f.type != FWDMI_FIELD_I32 || !f.data) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: field '%s' must be INT32", name.c_str());
        return nullptr;
      }
      *scalar = *static_cast<const int*>(f.data);
      if (slot >= 0) have[slot] = true;
    } else if (version_ext_ && name == "output_fp16") {
      if (f.type != FWDMI_FIELD_I32 || !f.data) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: field 'output_fp16' must be INT32");
        return nullptr;
      }
      opt.out_dtype = *static_cast<const int*>(f.data) ? FWDMI_F16 : FWDMI_F32;
    } else if (version_ext_ && name == "data_file") {
      if (f.type != FWDMI_FIELD_CHAR || !f.data || f.length <= 0) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: field 'data_file' must be a CHAR path");
        return nullptr;
      }
      data_file.assign(static_cast<const char*>(f.data), (size_t)f.length);
      while (!data_file.empty() && data_file.back() == '\0') data_file.pop_back();
      have[4] = true;
    } else if (name == "data") {
      const bool type_ok = f.type == FWDMI_FIELD_F32 || (version_ext_ && f.type == FWDMI_FIELD_F16);
      if (!type_ok || !f.data) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: field 'data' must be FLOAT32%s", version_ext_ ? " or FLOAT16" : "");
        return nullptr;
      }
      data = &f;
      opt.table_dtype = f.type == FWDMI_FIELD_F16 ? FWDMI_F16 : FWDMI_F32;
      have[4] = true;
    } else {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: unknown field '%s'", name.c_str());
      return nullptr;
    }
  }
  for (int i = 0; i < 5; ++i)
    if (!have[i]) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: missing field '%s'", mPluginAttributes[i].name);
      return nullptr;
    }
  if (dim <= 0 || dim > (1 << 24) || count <= 0 || !is_reduce_op(op) || !is_index_dtype(opt.index_dtype)) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: bad field values (dim %d, count %d, op %d, index_type %d)", dim,
              count, op, opt.index_dtype);
    return nullptr;
  }
  if (opt.per_sample_weights && op != FWDMI_OP_SUM) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: per_sample_weights requires op SUM");
    return nullptr;
  }
  if (opt.with_square_sum && (op != FWDMI_OP_SUM || opt.per_sample_weights)) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: with_square_sum requires op SUM without per_sample_weights");
    return nullptr;
  }
  const size_t n = (size_t)dim * (size_t)count;
  if (!data_file.empty()) {
    if (data || !is_float_dtype(table_type) || file_row_offset < 0) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: 'data_file' excludes 'data' and needs 'table_type' (0 fp32 / 1 fp16)");
      return nullptr;
    }
    opt.table_dtype = table_type;
    const size_t es = dtype_size(table_type);
    auto blob = HostDeviceBlob::map_file(data_file, (uint64_t)file_row_offset * dim * es, n * es);
    if (!blob) return nullptr;
    auto* obj = new EmbeddingBagPlugin(std::move(blob), dim, count, offset, static_cast<ReduceOperation>(op), opt, true);
    obj->setPluginNamespace(mNamespace.c_str());
    return obj;
  }
  if (data->length < 0 || (size_t)data->length != n) {
    // The reference copies dim*count floats whatever the field's length says
    // (embedding_bag_plugin.cpp:283-285); its caller passes dim*count
    // (trt_embedding_bag_creator.h:62-64).  Anything else would read past the caller's array.
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBag: 'data' holds %d elements, dim*count = %zu", data->length, n);
    return nullptr;
  }
  auto* obj = new EmbeddingBagPlugin(make_blob(data->data, n * dtype_size(opt.table_dtype)), dim, count, offset,
                                     static_cast<ReduceOperation>(op), opt, version_ext_);
  obj->setPluginNamespace(mNamespace.c_str());
  return obj;
}

IPluginV2DynamicExt* EmbeddingBagPluginCreator::deserializePlugin(const char*, const void* serialData,
                                                                  size_t serialLength) noexcept {
  EmbeddingBagPlugin* obj = EmbeddingBagPlugin::deserialize(serialData, serialLength, version_ext_);
  if (obj) obj->setPluginNamespace(mNamespace.c_str());
  return obj;
}

FWDMI_REGISTER_PLUGIN(EmbeddingBagPluginCreator);
FWDMI_REGISTER_PLUGIN(EmbeddingBagPluginCreatorExt);

}  // namespace fwdmi
