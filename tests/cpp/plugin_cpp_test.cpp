// C++ host test of the plugin interface in fwdmi_plugin.h, written the way the reference's
// layer creator and TensorRT drive a plugin (source/trt_engine/trt_network_crt/layer_creators/
// trt_embedding_bag_creator.h:44-85 for creation; build-time calls getOutputDimensions,
// supportsFormatCombination, configurePlugin, serialize; run-time call enqueue).
//
//   plugin_cpp_test host   registry, fields, shapes, formats, serialized bytes (no GPU needed)
//   plugin_cpp_test gpu    the above plus configure + enqueue on device buffers, checked against
//                          sums computed on the host in double precision
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "fwdmi_plugin.h"

#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::printf("FAIL %s:%d: %s  [%s]\n", __FILE__, __LINE__, #cond, fwdmi_last_error()); \
      return 1;                                                            \
    }                                                                      \
  } while (0)

using namespace fwdmi;

static PluginTensorDesc desc(std::initializer_list<int> dims, int type) {
  PluginTensorDesc d{};
  d.dims.nbDims = (int)dims.size();
  int i = 0;
  for (int v : dims) d.dims.d[i++] = v;
  d.type = type;
  d.format = FWDMI_FORMAT_LINEAR;
  d.scale = 1.0f;
  return d;
}

int main(int argc, char** argv) {
  const bool gpu = argc > 1 && std::string(argv[1]) == "gpu";
  const int dim = 8, count = 50;
  std::vector<float> table(dim * count);
  for (int i = 0; i < dim * count; ++i) table[i] = std::sin(0.37f * i) * 0.5f;
  const int offset = 0, op = 0;

  // ---- what the layer creator does ----------------------------------------------------------
  IPluginCreator* creator = getPluginRegistry()->getPluginCreator("EmbeddingBag_TRT", "001");
  CHECK(creator != nullptr);
  CHECK(std::string(creator->getPluginName()) == "EmbeddingBag_TRT");
  CHECK(creator->getFieldNames()->nbFields == 5);
  std::vector<PluginField> field_data;
  field_data.push_back({"dim", &dim, FWDMI_FIELD_I32, 1});
  field_data.push_back({"count", &count, FWDMI_FIELD_I32, 1});
  field_data.push_back({"offset", &offset, FWDMI_FIELD_I32, 1});
  field_data.push_back({"op", &op, FWDMI_FIELD_I32, 1});
  field_data.push_back({"data", table.data(), FWDMI_FIELD_F32, dim * count});
  const PluginFieldCollection plugin_data{(int32_t)field_data.size(), field_data.data()};
  IPluginV2DynamicExt* plugin = creator->createPlugin("embedding_bag", &plugin_data);
  CHECK(plugin != nullptr);
  // a wrong field count is a contract violation: nullptr + message instead of abort()
  const PluginFieldCollection four{4, field_data.data()};
  CHECK(creator->createPlugin("embedding_bag", &four) == nullptr);
  CHECK(std::strstr(fwdmi_last_error(), "expected 5 fields") != nullptr);

  // ---- what TensorRT does at build time -----------------------------------------------------
  const std::vector<int32_t> ids = {1, 0, 3, 1, 4, 49, 7, 7, 7, 12};
  const std::vector<int32_t> offs = {0, 0, 5, 6};  // bags: empty, 5 ids, 1 id, 4 ids
  Dims in_dims[2] = {desc({(int)ids.size()}, FWDMI_I32).dims, desc({(int)offs.size()}, FWDMI_I32).dims};
  const Dims out_dims = plugin->getOutputDimensions(0, in_dims, 2);
  CHECK(out_dims.nbDims == 2 && out_dims.d[0] == 4 && out_dims.d[1] == dim);
  PluginTensorDesc io[3] = {desc({(int)ids.size()}, FWDMI_I32), desc({(int)offs.size()}, FWDMI_I32),
                            desc({4, dim}, FWDMI_F32)};
  for (int pos = 0; pos < 3; ++pos) CHECK(plugin->supportsFormatCombination(pos, io, 2, 1));
  io[2].type = FWDMI_F16;
  CHECK(!plugin->supportsFormatCombination(2, io, 2, 1));
  io[2].type = FWDMI_F32;
  CHECK(plugin->getWorkspaceSize(io, 2, io + 2, 1) == 0);
  CHECK(plugin->getNbOutputs() == 1);
  const DataType in_types[2] = {DataType::kINT32, DataType::kINT32};
  CHECK(plugin->getOutputDataType(0, in_types, 2) == DataType::kFLOAT);

  std::vector<char> blob(plugin->getSerializationSize());
  plugin->serialize(blob.data());
  CHECK(blob.size() == 24 + sizeof(float) * dim * count);
  CHECK(std::memcmp(blob.data() + 24, table.data(), sizeof(float) * dim * count) == 0);
  IPluginV2DynamicExt* loaded = creator->deserializePlugin("embedding_bag", blob.data(), blob.size());
  CHECK(loaded != nullptr);
  CHECK(creator->deserializePlugin("embedding_bag", blob.data(), blob.size() - 1) == nullptr);
  IPluginV2DynamicExt* clone = loaded->clone();
  CHECK(clone != nullptr && std::string(clone->getPluginType()) == "EmbeddingBag_TRT");

  // the LayerNorm family is reachable the same way
  CHECK(getPluginRegistry()->getPluginCreator("ForwardLayerNormPluginDynamic", "1") != nullptr);
  CHECK(getPluginRegistry()->getPluginCreator("CustomSkipLayerNormPluginDynamic", "1") != nullptr);
  CHECK(getPluginRegistry()->getPluginCreator("CustomEmbLayerNormPluginDynamic", "1") != nullptr);
  CHECK(getPluginRegistry()->getPluginCreator("EmbeddingBag_TRT", "9") == nullptr);

  // ---- damaged engine bytes: every truncation and a sweep of byte flips of every plugin's blob
  //      must come back as nullptr or as a plugin that can be destroyed, never as a crash ------
  {
    std::vector<float> gamma(16, 1.0f), beta(16, 0.0f), word(5 * 16, 0.25f), pos(4 * 16, 0.5f), tok(2 * 16, 0.125f);
    const int ld = 16, type_id = FWDMI_F16, fp16 = 1, mha = FWDMI_F16;
    std::vector<PluginField> ln = {{"ld", &ld, FWDMI_FIELD_I32, 1},           {"type_id", &type_id, FWDMI_FIELD_I32, 1},
                                   {"beta", beta.data(), FWDMI_FIELD_F32, 16}, {"gamma", gamma.data(), FWDMI_FIELD_F32, 16},
                                   {"bias", beta.data(), FWDMI_FIELD_F32, 16}};
    std::vector<PluginField> emb = {{"bert_embeddings_layernorm_beta", beta.data(), FWDMI_FIELD_F32, 16},
                                    {"bert_embeddings_layernorm_gamma", gamma.data(), FWDMI_FIELD_F32, 16},
                                    {"bert_embeddings_word_embeddings", word.data(), FWDMI_FIELD_F32, 5 * 16},
                                    {"bert_embeddings_token_type_embeddings", tok.data(), FWDMI_FIELD_F32, 2 * 16},
                                    {"bert_embeddings_position_embeddings", pos.data(), FWDMI_FIELD_F32, 4 * 16},
                                    {"output_fp16", &fp16, FWDMI_FIELD_I32, 1},
                                    {"mha_type_id", &mha, FWDMI_FIELD_I32, 1}};
    const int g_dim = 4, g_op = 0, g_counts[3] = {2, 5, 1};
    std::vector<float> g_rows(8 * 4, 0.5f);
    std::vector<PluginField> group = {{"dim", &g_dim, FWDMI_FIELD_I32, 1},
                                      {"op", &g_op, FWDMI_FIELD_I32, 1},
                                      {"count", g_counts, FWDMI_FIELD_I32, 3},
                                      {"data", g_rows.data(), FWDMI_FIELD_F32, 8 * 4}};
    struct Case {
      const char* name;
      const char* version;
      std::vector<PluginField>* fields;
    } cases[] = {{"EmbeddingBag_TRT", "001", &field_data},
                 {"EmbeddingBagGroup_TRT", "001", &group},
                 {"EmbeddingBag_TRT", "002", &field_data},
                 {"ForwardLayerNormPluginDynamic", "1", &ln},
                 {"CustomSkipLayerNormPluginDynamic", "1", &ln},
                 {"CustomEmbLayerNormPluginDynamic", "1", &emb}};
    for (const Case& c : cases) {
      IPluginCreator* cr = getPluginRegistry()->getPluginCreator(c.name, c.version);
      CHECK(cr != nullptr);
      const PluginFieldCollection fc{(int32_t)c.fields->size(), c.fields->data()};
      IPluginV2DynamicExt* p = cr->createPlugin("layer", &fc);
      CHECK(p != nullptr);
      std::vector<char> good(p->getSerializationSize());
      p->serialize(good.data());
      p->destroy();
      IPluginV2DynamicExt* again = cr->deserializePlugin("layer", good.data(), good.size());
      CHECK(again != nullptr && again->getSerializationSize() == good.size());
      again->destroy();
      for (size_t n = 0; n < good.size(); n += (n < 64 ? 1 : 37)) {
        std::vector<char> cut(good.begin(), good.begin() + n);  // exact-size heap copy: overreads show up
        IPluginV2DynamicExt* q = cr->deserializePlugin("layer", cut.data(), cut.size());
        if (q) q->destroy();
      }
      unsigned state = 12345;
      for (int trial = 0; trial < 400; ++trial) {
        std::vector<char> bad(good);
        state = state * 1664525u + 1013904223u;
        const size_t at = (trial < 200 ? state % std::min<size_t>(bad.size(), 48) : state % bad.size());
        state = state * 1664525u + 1013904223u;
        bad[at] = (char)(state >> 24);
        IPluginV2DynamicExt* q = cr->deserializePlugin("layer", bad.data(), bad.size());
        if (q) {
          std::vector<char> out(q->getSerializationSize());
          q->serialize(out.data());
          q->destroy();
        }
      }
    }
  }

  // enqueue before configurePlugin is refused with a status
  {
    const void* ins[2] = {nullptr, nullptr};
    void* outs[1] = {nullptr};
    CHECK(plugin->enqueue(io, io + 2, ins, outs, nullptr, nullptr) == FWDMI_ERR_NOT_CONFIGURED);
  }

  if (gpu) {
    // ---- what TensorRT does at run time -----------------------------------------------------
    int32_t *d_ids = nullptr, *d_offs = nullptr;
    float* d_out = nullptr;
    CHECK(hipMalloc(&d_ids, ids.size() * 4) == hipSuccess);
    CHECK(hipMalloc(&d_offs, offs.size() * 4) == hipSuccess);
    CHECK(hipMalloc(&d_out, 4 * dim * 4) == hipSuccess);
    CHECK(hipMemcpy(d_ids, ids.data(), ids.size() * 4, hipMemcpyHostToDevice) == hipSuccess);
    CHECK(hipMemcpy(d_offs, offs.data(), offs.size() * 4, hipMemcpyHostToDevice) == hipSuccess);
    hipStream_t stream;
    CHECK(hipStreamCreate(&stream) == hipSuccess);
    std::vector<double> want(4 * dim, 0.0);
    const int ends[4] = {0, 5, 6, (int)ids.size()};
    for (int b = 0; b < 4; ++b)
      for (int i = offs[b]; i < ends[b]; ++i)
        for (int c = 0; c < dim; ++c) want[b * dim + c] += table[ids[i] * dim + c];

    IPluginV2DynamicExt* runs[3] = {plugin, loaded, clone};
    for (IPluginV2DynamicExt* p : runs) {
      DynamicPluginTensorDesc din[2] = {{io[0], io[0].dims, io[0].dims}, {io[1], io[1].dims, io[1].dims}};
      DynamicPluginTensorDesc dout[1] = {{io[2], io[2].dims, io[2].dims}};
      CHECK(p->configurePlugin(din, 2, dout, 1) == FWDMI_OK);
      CHECK(p->configurePlugin(din, 2, dout, 1) == FWDMI_OK);  // idempotent
      CHECK(hipMemsetAsync(d_out, 0xff, 4 * dim * 4, stream) == hipSuccess);
      const void* ins[2] = {d_ids, d_offs};
      void* outs[1] = {d_out};
      CHECK(p->enqueue(io, io + 2, ins, outs, nullptr, stream) == 0);
      std::vector<float> got(4 * dim);
      CHECK(hipMemcpyAsync(got.data(), d_out, got.size() * 4, hipMemcpyDeviceToHost, stream) == hipSuccess);
      CHECK(hipStreamSynchronize(stream) == hipSuccess);
      for (int i = 0; i < 4 * dim; ++i) CHECK(std::fabs(got[i] - want[i]) <= 1e-6 * (1.0 + std::fabs(want[i])));
      for (int c = 0; c < dim; ++c) CHECK(got[c] == 0.0f);  // the empty bag
    }
    // int64 ids are refused by the "001" contract with -1 (embedding_bag_plugin.cpp:182-185)
    PluginTensorDesc bad = io[0];
    bad.type = FWDMI_I64;
    const void* ins[2] = {d_ids, d_offs};
    void* outs[1] = {d_out};
    PluginTensorDesc bad_io[2] = {bad, io[1]};
    CHECK(plugin->enqueue(bad_io, io + 2, ins, outs, nullptr, stream) == FWDMI_ERR_UNSUPPORTED);
    loaded->destroy();   // the clone shares the device table and must keep working
    CHECK(clone->enqueue(io, io + 2, ins, outs, nullptr, stream) == 0);
    CHECK(hipStreamSynchronize(stream) == hipSuccess);
    clone->destroy();
    plugin->terminate();
    plugin->destroy();
    (void)hipFree(d_ids);
    (void)hipFree(d_offs);
    (void)hipFree(d_out);
    (void)hipStreamDestroy(stream);
  } else {
    loaded->destroy();
    clone->destroy();
    plugin->destroy();
  }
  std::printf("PASS (%s)\n", gpu ? "gpu" : "host");
  return 0;
}
