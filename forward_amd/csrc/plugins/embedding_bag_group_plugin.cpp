// Host side of "EmbeddingBagGroup_TRT": the T EmbeddingBag layers and the concatenation of a
// DLRM-style sparse stage as one plugin whose enqueue is one multi-table launch.  The per-table
// rules (id / offsets shapes, index filter, output type) are those of EmbeddingBag_TRT "002";
// reference behaviour cited there (plugins/embedding_bag_plugin/embedding_bag_plugin.cpp).
#include <cmath>

#include "embedding_bag_plugin.h"

namespace fwdmi {

namespace {

bool is_group_op(int v) { return v == 0 || v == 1 || v == 2 || v == 3; }

// Field-level consistency shared by createPlugin and deserialize.  Returns an empty string if fine.
std::string check_spec(const EmbeddingBagGroupSpec& s) {
  const int T = s.n_tables();
  if (T < 1 || T > kMaxGroupTables) return "needs 1.." + std::to_string(kMaxGroupTables) + " tables";
  if (s.dim <= 0 || s.dim > (1 << 24)) return "dim out of range";
  if (!is_group_op(static_cast<int>(s.op))) return "op must be 0 (sum), 1 (mean), 2 (max) or 3 (square sum)";
  if ((int)s.offset.size() != T || (int)s.cost.size() != T) return "'offset' / 'table_cost' must have one entry per table";
  for (int t = 0; t < T; ++t) {
    if (s.count[t] <= 0) return "every 'count' must be positive";
    if (!(s.cost[t] > 0.0f) || !std::isfinite(s.cost[t])) return "every 'table_cost' must be positive and finite";
  }
  if (!is_float_dtype(s.opt.table_dtype) || !is_float_dtype(s.opt.out_dtype) || !is_index_dtype(s.opt.index_dtype))
    return "unsupported table / index / output type";
  if ((int64_t)T * s.dim > INT32_MAX) return "output row too wide";
  // at most 2^41 rows of at most 2^24 elements: the byte count must stay far inside 64 bits
  if (s.total_rows() > ((size_t)1 << 48) / ((size_t)s.dim * 4)) return "tables too large";
  if (s.opt.per_sample_weights && s.op != ReduceOperation::SUM) return "per_sample_weights requires op 0 (sum)";
  return "";
}

size_t table_bytes(const EmbeddingBagGroupSpec& s, int t) {
  return (size_t)s.count[t] * (size_t)s.dim * dtype_size(s.opt.table_dtype);
}

void default_cost(EmbeddingBagGroupSpec* s) {
  const int T = s->n_tables();
  std::vector<int64_t> bytes(T);
  for (int t = 0; t < T; ++t) bytes[t] = (int64_t)table_bytes(*s, t);
  s->cost.assign(T, 1.0f);
  (void)fwdmi_bag_table_cost(bytes.data(), T, s->cost.data());
}

}  // namespace

EmbeddingBagGroupPlugin::EmbeddingBagGroupPlugin(std::shared_ptr<HostDeviceBlob> tables, EmbeddingBagGroupSpec spec)
    : spec_(std::move(spec)), tables_(std::move(tables)) {}

EmbeddingBagGroupPlugin::~EmbeddingBagGroupPlugin() noexcept { terminate(); }

int EmbeddingBagGroupPlugin::getNbOutputs() const noexcept { return 1; }

// Per table ids_t [N_t], offsets_t [B] or [1, B] (the two-input form of
// embedding_bag_plugin.cpp:84-99) and, with per_sample_weights, weights_t [N_t] -> [B, T*dim].
Dims EmbeddingBagGroupPlugin::getOutputDimensions(int outputIndex, const Dims* inputs, int nbInputs) noexcept {
  clear_error();
  const int T = spec_.n_tables();
  const int per = inputs_per_table();
  if (outputIndex != 0 || !inputs || nbInputs != per * T) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: output %d with %d inputs (%d tables need %d)", outputIndex,
              nbInputs, T, per * T);
    return error_dims();
  }
  int64_t n_off = -1;
  for (int t = 0; t < T; ++t) {
    const Dims& ids = inputs[per * t];
    const Dims& off = inputs[per * t + 1];
    if (ids.nbDims != 1 || !(off.nbDims == 1 || (off.nbDims == 2 && off.d[0] == 1))) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: table %d needs ids [N] and offsets [B] or [1, B]", t);
      return error_dims();
    }
    if (per == 3 && (inputs[per * t + 2].nbDims != 1 || inputs[per * t + 2].d[0] != ids.d[0])) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: table %d needs one weight per id", t);
      return error_dims();
    }
    const int64_t n = off.nbDims == 1 ? off.d[0] : off.d[1];
    if (n_off >= 0 && n != n_off) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: table %d has %lld offsets, table 0 has %lld", t, (long long)n,
                (long long)n_off);
      return error_dims();
    }
    n_off = n;
  }
  Dims out{};
  out.nbDims = 2;
  out.d[0] = (int32_t)(n_off - (spec_.opt.include_last_offset ? 1 : 0));
  out.d[1] = T * spec_.dim;
  return out;
}

bool EmbeddingBagGroupPlugin::supportsFormatCombination(int pos, const PluginTensorDesc* inOut, int nbInputs,
                                                        int nbOutputs) noexcept {
  const int per = inputs_per_table();
  if (!inOut || nbInputs != per * spec_.n_tables() || nbOutputs != 1 || pos < 0 || pos >= nbInputs + nbOutputs)
    return false;
  const PluginTensorDesc& d = inOut[pos];
  if (d.format != FWDMI_FORMAT_LINEAR) return false;
  if (pos >= nbInputs) return d.type == spec_.opt.out_dtype;
  return d.type == (pos % per == 2 ? spec_.opt.table_dtype : spec_.opt.index_dtype);
}

// One upload of all tables (one device allocation); clones share it.
int EmbeddingBagGroupPlugin::configurePlugin(const DynamicPluginTensorDesc*, int, const DynamicPluginTensorDesc*,
                                             int) noexcept {
  clear_error();
  if (initialized_) return FWDMI_OK;
  int rc = tables_->acquire(&d_data_);
  if (rc != FWDMI_OK) return rc;
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&d_oob_), sizeof(int32_t));
  if (e == hipSuccess) e = hipMemset(d_oob_, 0, sizeof(int32_t));
  if (e != hipSuccess) {
    tables_->release();
    d_data_ = nullptr;
    if (d_oob_) (void)hipFree(d_oob_);
    d_oob_ = nullptr;
    return set_error(FWDMI_ERR_HIP, "EmbeddingBagGroup: flag allocation failed: %s", hipGetErrorString(e));
  }
  initialized_ = true;
  return FWDMI_OK;
}

size_t EmbeddingBagGroupPlugin::getWorkspaceSize(const PluginTensorDesc*, int, const PluginTensorDesc*,
                                                 int) const noexcept {
  return ((size_t)spec_.n_tables() * sizeof(fwdmi_bag_table) + 255) & ~(size_t)255;
}

int EmbeddingBagGroupPlugin::initialize() noexcept { return 0; }

void EmbeddingBagGroupPlugin::terminate() noexcept {
  if (!initialized_) return;
  tables_->release();
  d_data_ = nullptr;
  if (d_oob_) (void)hipFree(d_oob_);
  d_oob_ = nullptr;
  initialized_ = false;
}

// Reduces all tables in one launch.  This call's table descriptors travel with that launch as
// kernel arguments (up to FWDMI_BAG_INLINE_TABLES tables) or are written into the workspace by
// small launches before it (more tables); either way nothing is staged on the host and the call
// stays stream-ordered.
int EmbeddingBagGroupPlugin::enqueue(const PluginTensorDesc* inputDesc, const PluginTensorDesc* outputDesc,
                                     const void* const* inputs, void* const* outputs, void* workspace,
                                     void* hipStream) noexcept {
  clear_error();
  if (!inputDesc || !outputDesc || !inputs || !outputs)
    return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: null argument");
  if (!initialized_) return set_error(FWDMI_ERR_NOT_CONFIGURED, "EmbeddingBagGroup::enqueue before configurePlugin");
  if (!workspace)
    return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue needs getWorkspaceSize() bytes of workspace");
  const int T = spec_.n_tables();
  const int per = inputs_per_table();
  const size_t es = dtype_size(spec_.opt.table_dtype);
  fwdmi_bag_table* const d_tables = static_cast<fwdmi_bag_table*>(workspace);

  int64_t n_off = -1, total_ids = 0;
  constexpr int kMaxLenHints = 64;  // per-table mean bag lengths are a sizing hint for at most this many tables
  float avg_len_t[kMaxLenHints];
  size_t row0 = 0;
  constexpr int kChunk = 64;
  static_assert(kChunk >= FWDMI_BAG_INLINE_TABLES, "one chunk holds every table of the inline form");
  fwdmi_bag_table chunk[kChunk];
  for (int t0 = 0; t0 < T; t0 += kChunk) {
    const int n = std::min(kChunk, T - t0);
    for (int k = 0; k < n; ++k) {
      const int t = t0 + k;
      if (inputDesc[per * t].type != spec_.opt.index_dtype || inputDesc[per * t + 1].type != spec_.opt.index_dtype)
        return set_error(FWDMI_ERR_UNSUPPORTED, "Unsupported input data type %d", inputDesc[per * t].type);
      const Dims& ids = inputDesc[per * t].dims;
      const Dims& off = inputDesc[per * t + 1].dims;
      if (ids.nbDims != 1 || !(off.nbDims == 1 || (off.nbDims == 2 && off.d[0] == 1)))
        return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: table %d needs ids [N], offsets [B] or [1, B]", t);
      const int64_t no = off.nbDims == 1 ? off.d[0] : off.d[1];
      if (n_off >= 0 && no != n_off)
        return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: tables disagree on the number of bags");
      n_off = no;
      if (ids.d[0] < 0) return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: negative id count");
      total_ids += ids.d[0];
      if (t < kMaxLenHints) avg_len_t[t] = (float)ids.d[0];  // divided by the bag count below
      fwdmi_bag_table& d = chunk[k];
      d.data = static_cast<const char*>(d_data_) + row0 * (size_t)spec_.dim * es;
      d.input = inputs[per * t];
      d.input_2 = inputs[per * t + 1];
      d.weights = nullptr;
      if (per == 3) {
        const PluginTensorDesc& w = inputDesc[per * t + 2];
        if (w.type != spec_.opt.table_dtype || w.dims.nbDims != 1 || w.dims.d[0] != ids.d[0])
          return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: table %d needs one weight per id in the table's type", t);
        d.weights = inputs[per * t + 2];
        if (ids.d[0] > 0 && !d.weights)
          return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: null weights (table %d)", t);
      }
      d.count = spec_.count[t];
      d.input_size = ids.d[0];
      d.data_offset = spec_.offset[t];
      d.out_col = (int64_t)t * spec_.dim;
      if (ids.d[0] > 0 && !d.input) return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: null ids (table %d)", t);
      if (!d.input_2) return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: null offsets (table %d)", t);
      row0 += (size_t)spec_.count[t];
    }
    if (T > FWDMI_BAG_INLINE_TABLES) {  // fewer travel with the launch itself (below)
      const int rc = fwdmi_bag_tables_fill(chunk, n, d_tables + t0, hipStream);
      if (rc != FWDMI_OK) return rc;
    }
  }
  const int64_t n_bags = n_off - (spec_.opt.include_last_offset ? 1 : 0);
  if (n_bags < 0) return set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup::enqueue: offsets input is empty");
  if (n_bags == 0) return FWDMI_OK;

  fwdmi_bag_ext x{};
  x.table_dtype = spec_.opt.table_dtype;
  x.index_dtype = spec_.opt.index_dtype;
  x.out_dtype = spec_.opt.out_dtype;
  x.include_last_offset = spec_.opt.include_last_offset;
  x.out_row_stride = (int64_t)T * spec_.dim;
  x.oob_flag = d_oob_;
  x.flags = (spec_.xcd_affinity ? FWDMI_BAG_XCD_TABLE_AFFINITY : 0) | (per == 3 ? FWDMI_BAG_TABLE_WEIGHTS : 0);
  x.table_cost = spec_.cost.data();
  if (T <= kMaxLenHints) {
    for (int t = 0; t < T; ++t) avg_len_t[t] /= (float)n_bags;
    x.table_avg_len = avg_len_t;
    x.flags |= FWDMI_BAG_TABLE_AVG_LEN;
  }
  const double avg_len = (double)total_ids / ((double)n_bags * T);
  if (T <= FWDMI_BAG_INLINE_TABLES)  // `chunk` holds them all: the descriptors are kernel arguments of the one launch
    return fwdmi_embedding_bag_multi_host(chunk, T, nullptr, n_bags, outputs[0], spec_.dim, static_cast<int>(spec_.op),
                                          avg_len, &x, hipStream);
  return fwdmi_embedding_bag_multi(d_tables, T, n_bags, outputs[0], spec_.dim, static_cast<int>(spec_.op), avg_len,
                                   &x, hipStream);
}

// Bytes:
//   int dim | int op | int T | int table_dtype | int index_dtype | int out_dtype |
//   int include_last_offset | int xcd_affinity | int per_sample_weights |
//   int count[T] | int offset[T] | float cost[T] |
//   size_t n | elem[n]                      (all tables back to back), or, for tables given by file,
//   size_t SIZE_MAX | size_t path_len | path bytes | uint64 byte offset in the file
size_t EmbeddingBagGroupPlugin::getSerializationSize() const noexcept {
  const size_t head = 9 * sizeof(int) + (size_t)spec_.n_tables() * (2 * sizeof(int) + sizeof(float)) + sizeof(size_t);
  if (tables_->by_reference()) return head + sizeof(size_t) + tables_->path().size() + sizeof(uint64_t);
  return head + tables_->size();
}

void EmbeddingBagGroupPlugin::serialize(void* buffer) const noexcept {
  ByteWriter w(buffer);
  w.pod<int>(spec_.dim);
  w.pod<int>(static_cast<int>(spec_.op));
  w.pod<int>(spec_.n_tables());
  w.pod<int>(spec_.opt.table_dtype);
  w.pod<int>(spec_.opt.index_dtype);
  w.pod<int>(spec_.opt.out_dtype);
  w.pod<int>(spec_.opt.include_last_offset);
  w.pod<int>(spec_.xcd_affinity);
  w.pod<int>(spec_.opt.per_sample_weights);
  w.bytes(spec_.count.data(), spec_.count.size() * sizeof(int));
  w.bytes(spec_.offset.data(), spec_.offset.size() * sizeof(int));
  w.bytes(spec_.cost.data(), spec_.cost.size() * sizeof(float));
  if (tables_->by_reference()) {
    w.pod<size_t>(SIZE_MAX);
    w.pod<size_t>(tables_->path().size());
    w.bytes(tables_->path().data(), tables_->path().size());
    w.pod<uint64_t>(tables_->file_offset());
    return;
  }
  w.pod<size_t>(tables_->size() / dtype_size(spec_.opt.table_dtype));
  w.bytes(tables_->data(), tables_->size());
}

EmbeddingBagGroupPlugin* EmbeddingBagGroupPlugin::deserialize(const void* data, size_t length) {
  clear_error();
  ByteReader r(data, length);
  EmbeddingBagGroupSpec s;
  int op = 0, T = 0;
  r.pod(&s.dim);
  r.pod(&op);
  r.pod(&T);
  r.pod(&s.opt.table_dtype);
  r.pod(&s.opt.index_dtype);
  r.pod(&s.opt.out_dtype);
  r.pod(&s.opt.include_last_offset);
  r.pod(&s.xcd_affinity);
  r.pod(&s.opt.per_sample_weights);
  if (!r.ok() || T < 1 || T > kMaxGroupTables || r.left() < (size_t)T * (2 * sizeof(int) + sizeof(float))) {
    set_error(FWDMI_ERR_TRUNCATED, "EmbeddingBagGroup: serialized header truncated or malformed");
    return nullptr;
  }
  s.op = static_cast<ReduceOperation>(op);
  s.count.resize(T);
  s.offset.resize(T);
  s.cost.resize(T);
  r.bytes(s.count.data(), (size_t)T * sizeof(int));
  r.bytes(s.offset.data(), (size_t)T * sizeof(int));
  r.bytes(s.cost.data(), (size_t)T * sizeof(float));
  const std::string why = check_spec(s);
  if (!why.empty()) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: serialized fields inconsistent: %s", why.c_str());
    return nullptr;
  }
  const size_t es = dtype_size(s.opt.table_dtype);
  const size_t n_elems = s.total_rows() * (size_t)s.dim;
  {
    ByteReader peek = r;
    size_t marker = 0;
    if (peek.pod(&marker) && marker == SIZE_MAX) {  // tables by reference
      size_t path_len = 0;
      uint64_t file_off = 0;
      std::string path;
      bool ok = peek.pod(&path_len) && path_len <= peek.left();
      if (ok) {
        path.resize(path_len);
        ok = peek.bytes(&path[0], path_len) && peek.pod(&file_off);
      }
      if (!ok) {
        set_error(FWDMI_ERR_TRUNCATED, "EmbeddingBagGroup: serialized table reference truncated");
        return nullptr;
      }
      auto blob = HostDeviceBlob::map_file(path, file_off, n_elems * es);
      if (!blob) return nullptr;
      return new EmbeddingBagGroupPlugin(std::move(blob), std::move(s));
    }
  }
  std::vector<uint8_t> bytes;
  size_t n = 0;
  if (!r.vec(&bytes, es, &n)) {
    set_error(FWDMI_ERR_TRUNCATED, "EmbeddingBagGroup: serialized tables truncated");
    return nullptr;
  }
  if (n != n_elems) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: serialized tables hold %zu elements, dim * sum(count) = %zu", n,
              n_elems);
    return nullptr;
  }
  return new EmbeddingBagGroupPlugin(std::make_shared<HostDeviceBlob>(std::move(bytes)), std::move(s));
}

const char* EmbeddingBagGroupPlugin::getPluginType() const noexcept { return EMBEDDING_BAG_GROUP_PLUGIN_NAME; }
const char* EmbeddingBagGroupPlugin::getPluginVersion() const noexcept { return EMBEDDING_BAG_GROUP_PLUGIN_VERSION; }
void EmbeddingBagGroupPlugin::destroy() noexcept { delete this; }

IPluginV2DynamicExt* EmbeddingBagGroupPlugin::clone() const noexcept {
  auto* p = new EmbeddingBagGroupPlugin(tables_, spec_);
  p->namespace_ = namespace_;
  return p;
}

void EmbeddingBagGroupPlugin::setPluginNamespace(const char* pluginNamespace) noexcept {
  namespace_ = pluginNamespace ? pluginNamespace : "";
}

const char* EmbeddingBagGroupPlugin::getPluginNamespace() const noexcept { return namespace_.c_str(); }

DataType EmbeddingBagGroupPlugin::getOutputDataType(int, const DataType*, int) const noexcept {
  return static_cast<DataType>(spec_.opt.out_dtype);
}

// ---- creator -----------------------------------------------------------------------------------
// Field names follow EmbeddingBag_TRT (embedding_bag_plugin.cpp:229-243); `count` and `offset`
// become arrays with one entry per table and `data` holds the tables back to back.
EmbeddingBagGroupPluginCreator::EmbeddingBagGroupPluginCreator() {
  declare("dim", PluginFieldType::kINT32);
  declare("op", PluginFieldType::kINT32);
  declare("count", PluginFieldType::kINT32);
  declare("offset", PluginFieldType::kINT32);
  declare("data", PluginFieldType::kFLOAT32);
  declare("index_type", PluginFieldType::kINT32);
  declare("output_fp16", PluginFieldType::kINT32);
  declare("include_last_offset", PluginFieldType::kINT32);
  declare("data_file", PluginFieldType::kCHAR);
  declare("data_file_row_offset", PluginFieldType::kINT32);
  declare("table_type", PluginFieldType::kINT32);
  declare("per_sample_weights", PluginFieldType::kINT32);
  declare("table_cost", PluginFieldType::kFLOAT32);
  declare("xcd_affinity", PluginFieldType::kINT32);
}

const char* EmbeddingBagGroupPluginCreator::getPluginName() const noexcept { return EMBEDDING_BAG_GROUP_PLUGIN_NAME; }
const char* EmbeddingBagGroupPluginCreator::getPluginVersion() const noexcept {
  return EMBEDDING_BAG_GROUP_PLUGIN_VERSION;
}

IPluginV2DynamicExt* EmbeddingBagGroupPluginCreator::createPlugin(const char*,
                                                                  const PluginFieldCollection* fc) noexcept {
  clear_error();
  if (!fc || (fc->nbFields > 0 && !fc->fields)) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: null field collection");
    return nullptr;
  }
  EmbeddingBagGroupSpec s;
  int op = -1, file_row_offset = 0, table_type = -1;
  bool have_dim = false, have_op = false;
  const PluginField* data = nullptr;
  std::string data_file;
  for (int i = 0; i < fc->nbFields; ++i) {
    const PluginField& f = fc->fields[i];
    const std::string name = f.name ? f.name : "";
    int* scalar = nullptr;
    std::vector<int>* ints = nullptr;
    if (name == "dim") scalar = &s.dim, have_dim = true;
    else if (name == "op") scalar = &op, have_op = true;
    else if (name == "include_last_offset") scalar = &s.opt.include_last_offset;
    else if (name == "per_sample_weights") scalar = &s.opt.per_sample_weights;
    else if (name == "index_type") scalar = &s.opt.index_dtype;
    else if (name == "data_file_row_offset") scalar = &file_row_offset;
    else if (name == "table_type") scalar = &table_type;
    else if (name == "xcd_affinity") scalar = &s.xcd_affinity;
    else if (name == "count") ints = &s.count;
    else if (name == "offset") ints = &s.offset;
    if (scalar || ints) {
      if (f.type != FWDMI_FIELD_I32 || !f.data || f.length < 1 || (ints && f.length > kMaxGroupTables)) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: field '%s' must be INT32%s", name.c_str(),
                  ints ? " with one entry per table" : "");
        return nullptr;
      }
      const int* v = static_cast<const int*>(f.data);
      if (scalar)
        *scalar = v[0];
      else
        ints->assign(v, v + f.length);
    } else if (name == "output_fp16") {
      if (f.type != FWDMI_FIELD_I32 || !f.data) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: field 'output_fp16' must be INT32");
        return nullptr;
      }
      s.opt.out_dtype = *static_cast<const int*>(f.data) ? FWDMI_F16 : FWDMI_F32;
    } else if (name == "table_cost") {
      if (f.type != FWDMI_FIELD_F32 || !f.data || f.length < 1 || f.length > kMaxGroupTables) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: field 'table_cost' must be FLOAT32 with one entry per table");
        return nullptr;
      }
      const float* v = static_cast<const float*>(f.data);
      s.cost.assign(v, v + f.length);
    } else if (name == "data_file") {
      if (f.type != FWDMI_FIELD_CHAR || !f.data || f.length <= 0) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: field 'data_file' must be a CHAR path");
        return nullptr;
      }
      data_file.assign(static_cast<const char*>(f.data), (size_t)f.length);
      while (!data_file.empty() && data_file.back() == '\0') data_file.pop_back();
    } else if (name == "data") {
      if ((f.type != FWDMI_FIELD_F32 && f.type != FWDMI_FIELD_F16) || !f.data) {
        set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: field 'data' must be FLOAT32 or FLOAT16");
        return nullptr;
      }
      data = &f;
      s.opt.table_dtype = f.type == FWDMI_FIELD_F16 ? FWDMI_F16 : FWDMI_F32;
    } else {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: unknown field '%s'", name.c_str());
      return nullptr;
    }
  }
  if (!have_dim || !have_op || s.count.empty() || (!data && data_file.empty())) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: fields 'dim', 'op', 'count' and 'data' (or 'data_file') are required");
    return nullptr;
  }
  s.op = static_cast<ReduceOperation>(op);
  if (s.offset.empty()) s.offset.assign(s.count.size(), 0);
  if (!data_file.empty()) {
    if (data || !is_float_dtype(table_type) || file_row_offset < 0) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: 'data_file' excludes 'data' and needs 'table_type' (0 fp32 / 1 fp16)");
      return nullptr;
    }
    s.opt.table_dtype = table_type;
  }
  const bool own_cost = s.cost.empty();
  if (own_cost) s.cost.assign(s.count.size(), 1.0f);
  const std::string why = check_spec(s);
  if (!why.empty()) {
    set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: %s", why.c_str());
    return nullptr;
  }
  if (own_cost) default_cost(&s);
  const size_t es = dtype_size(s.opt.table_dtype);
  const size_t n = s.total_rows() * (size_t)s.dim;
  std::shared_ptr<HostDeviceBlob> blob;
  if (!data_file.empty()) {
    blob = HostDeviceBlob::map_file(data_file, (uint64_t)file_row_offset * s.dim * es, n * es);
    if (!blob) return nullptr;
  } else {
    if (data->length < 0 || (size_t)data->length != n) {
      set_error(FWDMI_ERR_BAD_ARG, "EmbeddingBagGroup: 'data' holds %d elements, dim * sum(count) = %zu", data->length, n);
      return nullptr;
    }
    blob = make_blob(data->data, n * es);
  }
  auto* obj = new EmbeddingBagGroupPlugin(std::move(blob), std::move(s));
  obj->setPluginNamespace(mNamespace.c_str());
  return obj;
}

IPluginV2DynamicExt* EmbeddingBagGroupPluginCreator::deserializePlugin(const char*, const void* serialData,
                                                                       size_t serialLength) noexcept {
  EmbeddingBagGroupPlugin* obj = EmbeddingBagGroupPlugin::deserialize(serialData, serialLength);
  if (obj) obj->setPluginNamespace(mNamespace.c_str());
  return obj;
}

FWDMI_REGISTER_PLUGIN(EmbeddingBagGroupPluginCreator);

}  // namespace fwdmi
