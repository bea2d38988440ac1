/*
 * fwdmi.h -- C ABI of the MI355X (gfx950) embedding-side plugin path.
 *
 * Two layers are exported from libfwdmi.so, both `extern "C"`, plain pointers and sizes only:
 *
 *  1. kernel launchers: one per kernel family, the functions a plugin's enqueue() calls.  They
 *     take DEVICE pointers, enqueue work on the given HIP stream and return without
 *     synchronising or allocating.
 *  2. plugin objects: an opaque-handle view of the C++ plugin classes (creator lookup, field
 *     parsing, shape inference, format negotiation, configure, enqueue, serialize, clone) for
 *     hosts that cannot include the C++ header (Python ctypes, cgo, JNI).
 *
 * Every function returns an int status unless noted: 0 ok, negative on error (never aborts).
 * Paths in "replaces" notes are relative to the reference tree (Tencent/Forward).
 */
#ifndef FWDMI_H_
#define FWDMI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes ---------------------------------------------------------------------- */
#define FWDMI_OK 0
#define FWDMI_ERR_UNSUPPORTED (-1) /* dtype / format the path does not handle (reference: enqueue returns -1,
                                      embedding_bag_plugin.cpp:182-185) */
#define FWDMI_ERR_BAD_ARG (-2)     /* null pointer, negative size, shape mismatch */
#define FWDMI_ERR_HIP (-3)         /* a HIP runtime call failed; fwdmi_last_error() has the text */
#define FWDMI_ERR_NOT_CONFIGURED (-4)
#define FWDMI_ERR_TRUNCATED (-5)   /* serialized blob shorter than its own header says */

/* ---- element types: values follow nvinfer1::DataType; I64 is an extension ---------------- */
#define FWDMI_F32 0
#define FWDMI_F16 1
#define FWDMI_I8 2
#define FWDMI_I32 3
#define FWDMI_BOOL 4
#define FWDMI_I64 10

/* ---- plugin field types: values follow nvinfer1::PluginFieldType -------------------------- */
#define FWDMI_FIELD_F16 0
#define FWDMI_FIELD_F32 1
#define FWDMI_FIELD_F64 2
#define FWDMI_FIELD_I8 3
#define FWDMI_FIELD_I16 4
#define FWDMI_FIELD_I32 5
#define FWDMI_FIELD_CHAR 6
#define FWDMI_FIELD_DIMS 7
#define FWDMI_FIELD_UNKNOWN 8

/* ---- tensor format: nvinfer1::TensorFormat::kLINEAR ---------------------------------------- */
#define FWDMI_FORMAT_LINEAR 0

/* ---- bag reduction codes: ReduceOperation, embedding_bag_plugin.h:39 ----------------------- */
#define FWDMI_OP_SUM 0
#define FWDMI_OP_MEAN 1
#define FWDMI_OP_MAX 2
#define FWDMI_OP_SQUARE_SUM 3
#define FWDMI_OP_GATHER 999

const char* fwdmi_version(void);
/* Text of the most recent failure on the calling thread ("" if none). */
const char* fwdmi_last_error(void);
/* Number of HIP devices visible (0 without a GPU; never an error). */
int fwdmi_device_count(void);

/* ========================================================================================= *
 *  1. Kernel launchers
 * ========================================================================================= */

/*
 * Options beyond what the reference launchers take.  NULL means the reference's contract:
 * fp32 table, int32 indices, fp32 output rows packed at stride `dim`.
 */
typedef struct fwdmi_bag_ext {
  int32_t table_dtype;         /* FWDMI_F32 | FWDMI_F16 */
  int32_t index_dtype;         /* FWDMI_I32 | FWDMI_I64 (indices, offsets, max_indices) */
  int32_t out_dtype;           /* FWDMI_F32 | FWDMI_F16 */
  int32_t include_last_offset; /* offsets has n_bags+1 entries */
  const void* per_sample_weights; /* device, table dtype, [n_indices]; SUM only; may be NULL */
  void* max_indices;           /* device, index dtype, [n_bags, dim]; MAX only; may be NULL */
  int64_t out_row_stride;      /* elements between output rows; 0 = dim (lets several tables
                                  write column blocks of one concatenated matrix) */
  int32_t* oob_flag;           /* device int, set to 1 (sticky) when an id falls outside
                                  [data_offset, data_offset+count); may be NULL */
  int32_t flags;               /* FWDMI_BAG_* bits, 0 for none */
  const float* table_cost;     /* HOST array [n_tables] or NULL: relative cost of one bag of each
                                  table, used by FWDMI_BAG_XCD_TABLE_AFFINITY */
  void* square_sum_out;        /* device, out dtype, laid out like the output (same row stride and
                                  column blocks); op SUM without weights only; may be NULL.  When
                                  given, the same pass also writes the sum of squares of every
                                  bag: the two reductions a factorisation-machine term needs
                                  (the reference builds them as two plugins over two copies of
                                  the table, source/fwd_tf/tf_cvt/tf_desc_creators/tf_embedding_bag_creator.h:43-95) */
  const float* table_avg_len;  /* read only with FWDMI_BAG_TABLE_AVG_LEN in `flags`.  HOST array [n_tables]
                                  or NULL: mean ids per bag of each table of a multi-table launch.  With
                                  it, a table's share of the XCD segments (FWDMI_BAG_XCD_TABLE_AFFINITY)
                                  follows its bags' length as well as table_cost, and in launches of at
                                  most 64 tables those whose means differ by half or more get runs of
                                  their own size; without it every table counts as avg_bag_len long.  A
                                  sizing hint only: results do not depend on it */
  /* Layout of library version 0.2 (fwdmi_version()).  Members added after it are announced by a
   * bit in `flags` and read only when that bit is set, so a caller built against this layout
   * keeps working with later libraries. */
} fwdmi_bag_ext;

/* Multi-table launches only: renumber workgroups so that each of the 8 XCDs (one L2 each)
 * works through whole tables (a table's hot rows are then fetched into one L2 instead of all
 * eight).  The table-major work list is cut into eight segments of equal estimated cost;
 * `table_cost` supplies the estimate (large tables whose rows come from HBM cost more per bag
 * than small cache-resident ones), without it all tables count the same. */
#define FWDMI_BAG_XCD_TABLE_AFFINITY 1
/* Multi-table launches only (op SUM): every table's descriptor carries a `weights` pointer
 * (per-sample weights in the table's type, one per id); a table whose pointer is NULL uses
 * weight 1 for all of its ids. */
#define FWDMI_BAG_TABLE_WEIGHTS 2
/* ext->table_avg_len is present and may be read (see there). */
#define FWDMI_BAG_TABLE_AVG_LEN 4

/*
 * Variable-length bags: bag b = input[input_2[b] .. input_2[b+1]), last bag ends at input_size.
 * replaces EmbeddingBag(), embedding_bag_plugin.h:47-49 / embedding_bag_plugin.cu:198-206.
 *   input    [input_size] ids          input_2 [block_size] offsets (block_size = number of bags)
 *   output   [block_size, dim]         data    [count, dim] table, row-major
 * Ids outside [data_offset, data_offset+count) are skipped (embedding_bag_plugin.cu:94).
 * op_type MEAN divides by the bag length, MAX keeps the first maximum; empty bags give zeros.
 */
int fwdmi_embedding_bag(const void* input, const void* input_2, void* output, int64_t input_size,
                        int64_t block_size, const void* data, int64_t count, int32_t dim,
                        int64_t data_offset, int32_t op_type, const fwdmi_bag_ext* ext, void* stream);

/*
 * Fixed-length bags: input is [batch_size, offset] ids, bag b = row b.
 * replaces EmbeddingBagWithFixedOffset(), embedding_bag_plugin.h:43-45 / .cu:190-196.
 */
int fwdmi_embedding_bag_fixed(const void* input, void* output, int64_t batch_size, int64_t offset,
                              const void* data, int64_t count, int32_t dim, int64_t data_offset,
                              int32_t op_type, const fwdmi_bag_ext* ext, void* stream);

/*
 * Plain row gather (op 999): output[i, :] = data[input[i] - data_offset, :] for the
 * batch_size*offset ids; out-of-range ids produce zero rows.
 * replaces Gather(), embedding_bag_plugin.h:40-41 / .cu:182-188.
 */
int fwdmi_gather(const void* input, void* output, int64_t batch_size, int64_t offset,
                 const void* data, int64_t count, int32_t dim, int64_t data_offset,
                 const fwdmi_bag_ext* ext, void* stream);

/*
 * One table of a multi-table batch.  The array of these lives in DEVICE memory.
 */
typedef struct fwdmi_bag_table {
  const void* data;    /* [count, dim], 16-byte aligned when dim * element size is a multiple of 16;
                          must address count * dim elements.  count <= 0 is an empty table: data
                          is not read (may be NULL), every id counts as out of range and the
                          table's output block is zeros */
  const void* input;   /* [input_size] ids */
  const void* input_2; /* [n_bags] offsets (+1 with include_last_offset) */
  int64_t count;
  int64_t input_size;
  int64_t data_offset;
  int64_t out_col;     /* first output column of this table's block (t * dim for a plain
                          concatenation); with dim a multiple of 16 bytes of elements it must be
                          one too */
  const void* weights; /* [input_size] per-sample weights, table dtype; read only with
                          FWDMI_BAG_TABLE_WEIGHTS; may be NULL */
} fwdmi_bag_table;

/*
 * All tables of a DLRM-style sparse stage in one launch: every table reduces the same number
 * of bags with the same dim / dtypes and writes its [n_bags, dim] block at column out_col of
 * one [n_bags, out_row_stride] matrix.  Equivalent to n_tables calls of fwdmi_embedding_bag
 * with ext->out_row_stride set (the reference issues one plugin enqueue per table,
 * embedding_bag_plugin.cpp:146-189, and concatenates afterwards).
 * `avg_bag_len` (>0) is a sizing hint: the mean ids per bag over the batch.  At most 2^20 tables per launch.
 * Per-sample weights come through the descriptors (FWDMI_BAG_TABLE_WEIGHTS), not through
 * ext->per_sample_weights; max_indices is not available in this form.
 */
int fwdmi_embedding_bag_multi(const fwdmi_bag_table* tables_dev, int32_t n_tables, int64_t n_bags,
                              void* output, int32_t dim, int32_t op_type, double avg_bag_len,
                              const fwdmi_bag_ext* ext, void* stream);

/*
 * fwdmi_embedding_bag_multi for callers that hold the descriptors in HOST memory and rebuild them per
 * call (a plugin's enqueue: new id / offset buffers every time).  Up to FWDMI_BAG_INLINE_TABLES tables travel with the launch
 * itself, as kernel arguments: one launch, nothing staged, `tables_dev` is not used and may be NULL.
 * More tables are written to `tables_dev` (a device array of n_tables descriptors, required then) by
 * fwdmi_bag_tables_fill on the same stream first.  The descriptors are checked on the host (data /
 * ids / offsets present, column block inside the output row, 16-byte alignment where rows are read as
 * slices) and, for at most 64 tables, every table's mean bag length is taken from them unless
 * ext->table_avg_len is given (more tables run with avg_bag_len for all of them).
 * Results equal those of fwdmi_embedding_bag_multi bit for bit.
 */
#define FWDMI_BAG_INLINE_TABLES 40
int fwdmi_embedding_bag_multi_host(const fwdmi_bag_table* tables_host, int32_t n_tables, fwdmi_bag_table* tables_dev,
                                   int64_t n_bags, void* output, int32_t dim, int32_t op_type, double avg_bag_len,
                                   const fwdmi_bag_ext* ext, void* stream);

/*
 * fwdmi_embedding_bag_multi for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  The descriptors are given in HOST memory; the library copies them (as kernel
 * arguments, on `stream`) into a descriptor buffer that is part of its own code object, then
 * launches exactly what fwdmi_embedding_bag_multi launches, so results are bit-identical.
 * It calls no hipMalloc / hipFree or any other allocating routine; inputs and outputs are the
 * caller's.  Limits: at most 1024 tables per call (more is FWDMI_ERR_BAD_ARG; the buffer holds
 * 64 KiB per GPU for the life of the process).  Calls of at most FWDMI_BAG_INLINE_TABLES tables
 * carry their descriptors among the launch's own arguments and share nothing.  Larger calls on
 * one GPU share that GPU's buffer: a call's descriptor writes and its launch are enqueued under
 * one lock, so calls on the same stream, from any number of host threads, are ordered by the
 * stream; calls that overlap on one GPU (different streams without an ordering between them)
 * race and must not be made.  The first such call on a device looks the buffer's address up
 * (hipGetSymbolAddress); make that call outside a graph capture.
 */
int fwdmi_embedding_bag_multi_noalloc(const fwdmi_bag_table* tables_host, int32_t n_tables, int64_t n_bags,
                                      void* output, int32_t dim, int32_t op_type, double avg_bag_len,
                                      const fwdmi_bag_ext* ext, void* stream);

/*
 * Writes n_tables descriptors from HOST memory into the DEVICE array a later
 * fwdmi_embedding_bag_multi on the same stream reads.  The descriptors travel as kernel
 * arguments: stream-ordered, no host synchronisation, no pinned staging buffer, and the host
 * array may be reused as soon as the call returns.  For callers whose id / offset buffers change
 * from call to call (a plugin's enqueue).  (No counterpart in the reference, which launches one
 * kernel per table.)
 */
int fwdmi_bag_tables_fill(const fwdmi_bag_table* tables_host, int32_t n_tables, fwdmi_bag_table* tables_dev,
                          void* stream);

/*
 * Cost estimate for fwdmi_bag_ext.table_cost from the tables' sizes: cost[t] = 1 for a table
 * small enough to stay in one XCD's L2, growing with log(size) to about 1.45 for a table of
 * 512 MiB or more, whose rows mostly come from HBM.  (No counterpart in the reference, which
 * launches one kernel per table.)
 */
int fwdmi_bag_table_cost(const int64_t* table_bytes, int32_t n_tables, float* cost);

/*
 * What the bag launches know of the current device, as the runtime reports it: compute units and
 * XCDs (accelerator dies, one L2 each; 1 when the device is one die or the runtime does not say).
 * Run sizes follow the CU count; FWDMI_BAG_XCD_TABLE_AFFINITY is honoured with 2 .. 8 XCDs and is
 * the plain table-major order otherwise.  (No counterpart in the reference.)
 */
int fwdmi_bag_device_topology(int32_t* cus, int32_t* xcds);

/*
 * out = gamma * (x - mean) * rsqrt(var + eps) + beta,  x = input (+ bias), per row of ld.
 * n = total elements (rows = n / ld).  gamma/beta/bias: device fp32 [ld]; bias may be NULL.
 * dtype: FWDMI_F32 | FWDMI_F16 for input and output.  The reference has no eps (pass 0).
 * replaces computeLayerNorm<T,hasBias>(), layer_norm_plugin.h:37-39 / layer_norm_kernel.cu:278-305.
 */
int fwdmi_layer_norm(void* stream, int32_t ld, int64_t n, const void* input, const float* beta,
                     const float* gamma, void* output, const float* bias, int32_t dtype, float eps);

/*
 * out = LN(input + skip (+ bias)): the arithmetic of "CustomSkipLayerNormPluginDynamic" v1 as
 * the reference wires it (trt_bert_creator.h:199-239, inputs {input, skip}).
 */
int fwdmi_skip_layer_norm(void* stream, int32_t ld, int64_t n, const void* input, const void* skip,
                          const float* beta, const float* gamma, void* output, const float* bias,
                          int32_t dtype, float eps);

/*
 * BERT embedding lookup fused with LayerNorm: the arithmetic of
 * "CustomEmbLayerNormPluginDynamic" v1 as the reference wires it (trt_bert_creator.h:113-155).
 *   input_ids, segment_ids, input_mask : int32 [S, B]   (token t = s*B + b)
 *   word [word_count, ld], pos [pos_count, ld], tok [tok_count, ld] in `dtype`
 *   output [S, B, ld] in `dtype`;  mask_idx int32 [B] = first s with input_mask[s,b]==0, else S
 *   (mask_idx / input_mask may both be NULL).  Out-of-table ids add a zero row and raise
 *   *oob_flag (may be NULL).
 */
int fwdmi_emb_layer_norm(void* stream, int32_t S, int32_t B, int32_t ld, const int32_t* input_ids,
                         const int32_t* segment_ids, const int32_t* input_mask, const float* beta,
                         const float* gamma, const void* word, const void* pos, const void* tok,
                         int32_t word_count, int32_t pos_count, int32_t tok_count, void* output,
                         int32_t* mask_idx, int32_t dtype, float eps, int32_t* oob_flag);

/*
 * Options of fwdmi_emb_layer_norm_ex (NULL = the plain call above).
 *   batch_major: ids / mask are [B, S] and the output is [B, S, ld] (the reference transposes to
 *     [S, B] before the plugin and back after it, trt_bert_creator.h:64-71,106-109).
 *   skip != NULL fuses the SkipLayerNorm that consumes the embedding in the same pass:
 *     first  = LN(word + pos + tok) rounded to `dtype` (also stored to emb_output if given)
 *     output = LN2(first + skip (+ bias2)) with gamma2 / beta2 / eps2
 *   which equals fwdmi_emb_layer_norm followed by fwdmi_skip_layer_norm bit for bit.
 */
typedef struct fwdmi_emb_ext {
  int32_t batch_major;
  float eps2;
  const void* skip;      /* [rows, ld] in `dtype`, row order as the output */
  const float* gamma2;   /* fp32 [ld] */
  const float* beta2;    /* fp32 [ld] */
  const float* bias2;    /* fp32 [ld] or NULL */
  void* emb_output;      /* [rows, ld] or NULL */
} fwdmi_emb_ext;

int fwdmi_emb_layer_norm_ex(void* stream, int32_t S, int32_t B, int32_t ld, const int32_t* input_ids,
                            const int32_t* segment_ids, const int32_t* input_mask, const float* beta,
                            const float* gamma, const void* word, const void* pos, const void* tok,
                            int32_t word_count, int32_t pos_count, int32_t tok_count, void* output,
                            int32_t* mask_idx, int32_t dtype, float eps, int32_t* oob_flag,
                            const fwdmi_emb_ext* ext);

/* ========================================================================================= *
 *  2. Plugin objects (opaque handles over the C++ classes in fwdmi_plugin.h)
 * ========================================================================================= */

typedef struct fwdmi_plugin fwdmi_plugin;   /* an IPluginV2DynamicExt */
typedef struct fwdmi_creator fwdmi_creator; /* an IPluginCreator (owned by the registry) */

typedef struct fwdmi_dims {
  int32_t nbDims;
  int32_t d[8];
} fwdmi_dims; /* nvinfer1::Dims */

typedef struct fwdmi_tensor_desc {
  fwdmi_dims dims;
  int32_t type;   /* FWDMI_F32 ... */
  int32_t format; /* FWDMI_FORMAT_LINEAR */
  float scale;
} fwdmi_tensor_desc; /* nvinfer1::PluginTensorDesc */

typedef struct fwdmi_plugin_field {
  const char* name;
  const void* data; /* borrowed: the plugin copies what it keeps */
  int32_t type;     /* FWDMI_FIELD_* */
  int32_t length;   /* element count */
} fwdmi_plugin_field; /* nvinfer1::PluginField */

/* getPluginRegistry()->getPluginCreator(name, version), trt_embedding_bag_creator.h:54-55.
 * Registered: "EmbeddingBag_TRT"/"001" (the reference contract) and "002" (fp16 tables, int64 ids,
 * fp16 output, include_last_offset, per-sample weights, a second output with the sums of squares,
 * tables by file reference),
 * "EmbeddingBagGroup_TRT"/"001" (T tables + their concatenation, one launch per enqueue; needs
 * getWorkspaceSize bytes of workspace), "CustomEmbLayerNormPluginDynamic"/"1",
 * "CustomSkipLayerNormPluginDynamic"/"1", "ForwardLayerNormPluginDynamic"/"1". NULL if absent. */
fwdmi_creator* fwdmi_get_plugin_creator(const char* name, const char* version);
int fwdmi_registry_size(void);
fwdmi_creator* fwdmi_registry_at(int i);

const char* fwdmi_creator_name(fwdmi_creator* c);
const char* fwdmi_creator_version(fwdmi_creator* c);
int fwdmi_creator_num_fields(fwdmi_creator* c);
/* name / type of declared field i (IPluginCreator::getFieldNames). */
const char* fwdmi_creator_field_name(fwdmi_creator* c, int i);
int fwdmi_creator_field_type(fwdmi_creator* c, int i);
/* IPluginCreator::createPlugin; NULL on a contract violation (fwdmi_last_error says which). */
fwdmi_plugin* fwdmi_creator_create_plugin(fwdmi_creator* c, const char* name,
                                          const fwdmi_plugin_field* fields, int n_fields);
/* IPluginCreator::deserializePlugin; NULL on a truncated / malformed blob. */
fwdmi_plugin* fwdmi_creator_deserialize_plugin(fwdmi_creator* c, const char* name, const void* data,
                                               size_t length);

int fwdmi_plugin_get_nb_outputs(fwdmi_plugin* p);
/* getOutputDimensions on concrete dims; writes *out. */
int fwdmi_plugin_get_output_dimensions(fwdmi_plugin* p, int output_index, const fwdmi_dims* inputs,
                                       int nb_inputs, fwdmi_dims* out);
/* 1 supported, 0 not, negative on bad arguments. */
int fwdmi_plugin_supports_format_combination(fwdmi_plugin* p, int pos, const fwdmi_tensor_desc* in_out,
                                             int nb_inputs, int nb_outputs);
/* configurePlugin: uploads tables / parameters to the current device (needs a GPU). */
int fwdmi_plugin_configure(fwdmi_plugin* p, const fwdmi_tensor_desc* in, int nb_inputs,
                           const fwdmi_tensor_desc* out, int nb_outputs);
size_t fwdmi_plugin_get_workspace_size(fwdmi_plugin* p, const fwdmi_tensor_desc* in, int nb_inputs,
                                       const fwdmi_tensor_desc* out, int nb_outputs);
int fwdmi_plugin_initialize(fwdmi_plugin* p);
void fwdmi_plugin_terminate(fwdmi_plugin* p);
/* enqueue: device pointers, stream-ordered, no host sync, no allocation. */
int fwdmi_plugin_enqueue(fwdmi_plugin* p, const fwdmi_tensor_desc* in_desc,
                         const fwdmi_tensor_desc* out_desc, const void* const* inputs,
                         void* const* outputs, void* workspace, void* stream);
size_t fwdmi_plugin_get_serialization_size(fwdmi_plugin* p);
int fwdmi_plugin_serialize(fwdmi_plugin* p, void* buffer);
const char* fwdmi_plugin_get_type(fwdmi_plugin* p);
const char* fwdmi_plugin_get_version(fwdmi_plugin* p);
void fwdmi_plugin_set_namespace(fwdmi_plugin* p, const char* ns);
const char* fwdmi_plugin_get_namespace(fwdmi_plugin* p);
int fwdmi_plugin_get_output_data_type(fwdmi_plugin* p, int index, const int32_t* input_types,
                                      int nb_inputs);
fwdmi_plugin* fwdmi_plugin_clone(fwdmi_plugin* p);
void fwdmi_plugin_destroy(fwdmi_plugin* p);
/* Reads and clears the plugin's sticky "an id was out of range" device flag (synchronises the
 * stream; diagnostic, not part of the reference contract). Returns 0/1 or a negative status. */
int fwdmi_plugin_take_oob_flag(fwdmi_plugin* p, void* stream);

/* ========================================================================================= *
 *  3. Plan files: the plugins of an engine in one file + the "<file>.meta" JSON sidecar
 *     replaces the plugin part of TrtForwardEngine::Save / Load
 *     (source/trt_engine/trt_engine/trt_fwd_engine.cpp:156-209) and the sidecar of
 *     source/trt_engine/trt_common/trt_meta_data.cpp:42-97: keys infer_mode (int, the InferMode of
 *     source/common/fwd_common.h:40-46: 0 float, 1 half, 2 int8, 3 int8_calib), opt_batch_size,
 *     max_batch_size (ints), unused_input_indices, output_indices (int arrays), torch_module_path
 *     (string), written in the reference's text form so that either side loads the other's file.
 * ========================================================================================= */
typedef struct fwdmi_plan fwdmi_plan;

/* Serializes n plugins (with the layer names they were created under) into `path`;
 * meta_json (may be NULL) is checked as a sidecar (every key above present with its type, else
 * FWDMI_ERR_BAD_ARG and nothing is written) and goes to "<path>.meta" in the reference's form. */
int fwdmi_plan_save(const char* path, fwdmi_plugin* const* plugins, const char* const* layer_names, int n,
                    const char* meta_json);
/* Reads a plan back: every entry is re-created through its registered creator's
 * deserializePlugin.  NULL on a missing / truncated file, an unknown (type, version) or a sidecar
 * that is present but malformed (a plan without a sidecar loads, with no settings). */
fwdmi_plan* fwdmi_plan_load(const char* path);
int fwdmi_plan_size(fwdmi_plan* plan);
const char* fwdmi_plan_layer_name(fwdmi_plan* plan, int i);
/* Hands entry i to the caller (who destroys it); a second call for the same i returns NULL. */
fwdmi_plugin* fwdmi_plan_take_plugin(fwdmi_plan* plan, int i);
/* The sidecar as JSON text in the reference's form ("" if the sidecar is absent). */
const char* fwdmi_plan_meta(fwdmi_plan* plan);
void fwdmi_plan_close(fwdmi_plan* plan);

/* The sidecar by itself, typed: EngineMetaData of source/trt_engine/trt_common/trt_meta_data.h:37-90.
 * A new object holds the reference's defaults (infer_mode 0, batch sizes -1, empty arrays and path). */
typedef struct fwdmi_meta fwdmi_meta;
fwdmi_meta* fwdmi_meta_new(void);
/* EngineMetaData::LoadMetaData, trt_meta_data.cpp:49-79.  NULL when the file cannot be opened, is
 * not JSON, lacks infer_mode / opt_batch_size / max_batch_size / torch_module_path or holds a
 * value of the wrong type (fwdmi_last_error says which); absent index arrays read as empty. */
fwdmi_meta* fwdmi_meta_load(const char* meta_file);
/* The same from JSON text. */
fwdmi_meta* fwdmi_meta_parse(const char* json_text);
/* A copy of a loaded plan's sidecar; NULL if the plan has none.  Freed with fwdmi_meta_free. */
fwdmi_meta* fwdmi_plan_meta_data(fwdmi_plan* plan);
/* EngineMetaData::SaveMetaData, trt_meta_data.cpp:81-97: keys in alphabetical order, four-space
 * indentation, one array element per line, trailing newline. */
int fwdmi_meta_save(fwdmi_meta* m, const char* meta_file);
/* The text fwdmi_meta_save writes (valid until the next call on `m`). */
const char* fwdmi_meta_json(fwdmi_meta* m);
int32_t fwdmi_meta_infer_mode(fwdmi_meta* m);
int32_t fwdmi_meta_opt_batch_size(fwdmi_meta* m);
int32_t fwdmi_meta_max_batch_size(fwdmi_meta* m);
const char* fwdmi_meta_torch_module_path(fwdmi_meta* m);
/* Element count; *data (may be NULL) points at the elements, ascending for the unused inputs
 * (a set in the reference), valid until the next call of the same getter on `m`. */
int32_t fwdmi_meta_unused_input_indices(fwdmi_meta* m, const int32_t** data);
int32_t fwdmi_meta_output_indices(fwdmi_meta* m, const int32_t** data);
/* Sets every member at once (arrays are copied; torch_module_path NULL = ""). */
int fwdmi_meta_set(fwdmi_meta* m, int32_t infer_mode, int32_t opt_batch_size, int32_t max_batch_size,
                   const int32_t* unused_input_indices, int32_t n_unused, const int32_t* output_indices,
                   int32_t n_outputs, const char* torch_module_path);
void fwdmi_meta_free(fwdmi_meta* m);

#ifdef __cplusplus
}
#endif
#endif /* FWDMI_H_ */
