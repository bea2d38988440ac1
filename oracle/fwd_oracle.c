/*
 * fwd_oracle.c -- CPU restatement of the embedding-side plugin path of Tencent/Forward.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the parity tests, the smoke test and
 * the bench's cpu_baseline leg compare the HIP path against.  It is never linked into, loaded
 * by, or called from the product library.
 *
 * What it restates (paths relative to the reference tree):
 *   source/trt_engine/trt_network_crt/plugins/embedding_bag_plugin/embedding_bag_plugin.cu
 *     :80-86    bag bounds: offsets[b] .. offsets[b+1], last bag ends at input_size
 *     :94       index filter: rows outside [data_offset, data_offset+count) are skipped
 *     :95       row address = dim * (idx - data_offset)
 *     :135-136  fixed-length bags: start = L*b, end = start+L
 *     :170-181  plain gather (op 999)
 *   source/trt_engine/trt_network_crt/plugins/embedding_bag_plugin/embedding_bag_plugin.h:39
 *     op codes SUM=0 MEAN=1 MAX=2 SQUARE_SUM=3 GATHER=999
 *   source/trt_engine/trt_network_crt/plugins/layer_norm_plugin/layer_norm_kernel.cu
 *     :153-198  out = gamma * (x - mu) * rsigma + beta, x = in (+ bias)
 *   source/trt_engine/trt_network_crt/layer_creators/trt_bert_creator.h:113-155,199-239
 *     operand order of the two BERT plugins ([S,B] ids, [S,B,H] activations)
 *   python/bert_helpers/modeling.py:426,489-495,513-528
 *     embedding = word[id] + token_type[seg] + position[s], then LayerNorm
 *
 * Where the reference kernel's arithmetic is wrong or unspecified the oracle follows the
 * ground truth the reference's own tests use (libtorch CPU,
 * source/unit_test/unit_test_torch_helper.h:82-87):
 *   - MEAN divides the bag SUM by the bag length (the reference kernel swaps the op codes of
 *     mean and max inside atomicOp, embedding_bag_plugin.cu:52-63,111-112);
 *   - MAX is a true maximum with "first occurrence wins" (strict >, NaN never replaces a
 *     value, a NaN first element stays), argmax reports the ROW ID, empty bag -> 0 / 0;
 *   - sums are sequential in bag order in fp32 using fused multiply-add for weighted terms
 *     (the reference's shared-memory atomics have no defined order).
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   embedding bag sum        pinned: reference-held tables + inputs (embedding_bag.pth,
 *                            dlrm.pth), numpy gather+sum, libtorch CPU
 *   mean / max / weights     pinned: libtorch CPU on seeded inputs, hand-worked NaN/tie cases
 *                            (equal bit for bit, fp32 and fp16 tables, except the mean over an
 *                            fp16 table: libtorch's CPU kernel rounds the sum to fp16 and divides
 *                            that, this file divides the fp32 sum and rounds once; at most one
 *                            fp16 unit apart, inside the fp16 bar)
 *   fixed-length / gather    pinned: numpy fancy indexing
 *   layer norm family        pinned: float64 closed form (numpy), libtorch CPU layer_norm,
 *                            standardisation invariants
 *   emb-layer-norm / skip    arithmetic pinned as above; the NVIDIA plugins that the
 *                            reference loads by name are absent from the tree, so their
 *                            exact rounding is "parity unpinned"
 *   mask index               pinned: closed form (first zero of the mask column)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

enum { DT_F32 = 0, DT_F16 = 1, DT_I32 = 3, DT_I64 = 10 };
enum { OP_SUM = 0, OP_MEAN = 1, OP_MAX = 2, OP_SQUARE_SUM = 3, OP_GATHER = 999 };

/* ---- IEEE binary16 <-> binary32, exact / round-to-nearest-even ------------------------ */
static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: renormalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? (0x200u | ((absx >> 13) & 0x3ffu)) : 0));
  }
  if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x33000001u) { /* below half of the smallest subnormal -> 0 */
    return (uint16_t)sign;
  }
  int e = (int)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (e < -14) { /* subnormal half */
    shift = 13 + (-14 - e);
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
  return (uint16_t)(sign | (base + q)); /* a mantissa carry correctly bumps the exponent */
}

void oracle_half_to_float(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = half_to_float(in[i]);
}
void oracle_float_to_half(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = float_to_half(in[i]);
}

static inline float load_elem(const void* p, int dtype, int64_t i) {
  return dtype == DT_F16 ? half_to_float(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
static inline int64_t load_index(const void* p, int dtype, int64_t i) {
  return dtype == DT_I64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}
static inline void store_elem(void* p, int dtype, int64_t i, float v) {
  if (dtype == DT_F16)
    ((uint16_t*)p)[i] = float_to_half(v);
  else
    ((float*)p)[i] = v;
}
static inline void store_index(void* p, int dtype, int64_t i, int64_t v) {
  if (dtype == DT_I64)
    ((int64_t*)p)[i] = v;
  else
    ((int32_t*)p)[i] = (int32_t)v;
}

void oracle_set_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n > 0 ? n : 1);
#else
  (void)n;
#endif
}
int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/*
 * Bag reduction over an indices + offsets layout.
 *   fixed_len > 0 : indices is [n_bags, fixed_len], offsets ignored (embedding_bag_plugin.cu:135-136)
 *   fixed_len == 0: bag b covers offsets[b] .. offsets[b+1]; without include_last_offset the
 *                   offsets array has n_bags entries and the last bag ends at n_indices
 *                   (embedding_bag_plugin.cu:80-86)
 * psw (nullable): per-sample weights in the table dtype, SUM only.
 * max_indices (nullable): [n_bags, dim] in the index dtype, MAX only.
 * out_row_stride in elements (>= dim) lets several tables write one concatenated matrix.
 * Returns the number of indices that fell outside [data_offset, data_offset+count).
 */
int64_t oracle_embedding_bag(const void* indices, const void* offsets, void* output, int64_t n_indices,
                             int64_t n_bags, const void* table, int64_t count, int dim,
                             int64_t data_offset, int op, int table_dtype, int index_dtype,
                             int out_dtype, const void* psw, int include_last_offset,
                             int64_t fixed_len, int64_t out_row_stride, void* max_indices) {
  int64_t oob_total = 0;
  if (out_row_stride <= 0) out_row_stride = dim;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : oob_total)
  for (int64_t b = 0; b < n_bags; ++b) {
    int64_t start, end;
    if (fixed_len > 0) {
      start = b * fixed_len;
      end = start + fixed_len;
    } else {
      start = load_index(offsets, index_dtype, b);
      end = (b + 1 < n_bags || include_last_offset) ? load_index(offsets, index_dtype, b + 1)
                                                    : n_indices;
    }
    float acc[4096];
    int64_t arg[4096];
    for (int c0 = 0; c0 < dim; c0 += 4096) {
      int cw = dim - c0 < 4096 ? dim - c0 : 4096;
      for (int c = 0; c < cw; ++c) {
        acc[c] = 0.0f;
        arg[c] = 0;
      }
      int first = 1;
      for (int64_t i = start; i < end; ++i) {
        int64_t id = load_index(indices, index_dtype, i);
        int64_t row = id - data_offset;
        if (row < 0 || row >= count) {
          if (c0 == 0) ++oob_total;
          continue;
        }
        float w = psw ? load_elem(psw, table_dtype, i) : 1.0f;
        int64_t base = row * (int64_t)dim + c0;
        for (int c = 0; c < cw; ++c) {
          float x = load_elem(table, table_dtype, base + c);
          switch (op) {
            case OP_MAX:
              if (first || x > acc[c]) {
                acc[c] = x;
                arg[c] = id;
              }
              break;
            case OP_SQUARE_SUM:
              acc[c] = fmaf(x, x, acc[c]);
              break;
            default:
              acc[c] = psw ? fmaf(w, x, acc[c]) : acc[c] + x;
          }
        }
        first = 0;
      }
      int64_t len = end - start;
      for (int c = 0; c < cw; ++c) {
        float v = acc[c];
        if (op == OP_MEAN && len > 0) v = v / (float)len;
        store_elem(output, out_dtype, b * out_row_stride + c0 + c, v);
        if (max_indices) store_index(max_indices, index_dtype, b * (int64_t)dim + c0 + c, arg[c]);
      }
    }
  }
  return oob_total;
}

/*
 * Plain row gather, op 999 (embedding_bag_plugin.cu:170-181): out[i, :] = table[id_i - data_offset, :].
 * The reference leaves rows with out-of-range ids unwritten; the restatement (and the HIP
 * path) define them as zero rows, which is one of the outcomes the reference allows.
 */
int64_t oracle_gather(const void* indices, void* output, int64_t n_indices, const void* table,
                      int64_t count, int dim, int64_t data_offset, int table_dtype, int index_dtype,
                      int out_dtype) {
  int64_t oob = 0;
#pragma omp parallel for schedule(static) reduction(+ : oob)
  for (int64_t i = 0; i < n_indices; ++i) {
    int64_t row = load_index(indices, index_dtype, i) - data_offset;
    int ok = row >= 0 && row < count;
    if (!ok) ++oob;
    for (int c = 0; c < dim; ++c)
      store_elem(output, out_dtype, i * (int64_t)dim + c,
                 ok ? load_elem(table, table_dtype, row * (int64_t)dim + c) : 0.0f);
  }
  return oob;
}

/* One row of LayerNorm in float64, two-pass (the closed form every LN kernel is checked against). */
static void ln_row(const double* x, int ld, const float* gamma, const float* beta, double eps,
                   void* out, int out_dtype, int64_t out_base) {
  double mu = 0.0;
  for (int i = 0; i < ld; ++i) mu += x[i];
  mu /= ld;
  double var = 0.0;
  for (int i = 0; i < ld; ++i) var += (x[i] - mu) * (x[i] - mu);
  var /= ld;
  double rs = 1.0 / sqrt(var + eps);
  for (int i = 0; i < ld; ++i)
    store_elem(out, out_dtype, out_base + i,
               (float)((double)gamma[i] * (x[i] - mu) * rs + (double)beta[i]));
}

/*
 * out = LN(input (+ skip) (+ bias)); n = total elements, rows = n / ld
 * (layer_norm_kernel.cu:278-305 with the optional second operand of the skip plugin,
 * trt_bert_creator.h:233-235).  gamma/beta/bias are fp32 arrays of ld entries.
 */
int oracle_skip_layer_norm(int ld, int64_t n, const void* input, const void* skip, const float* beta,
                           const float* gamma, void* output, const float* bias, int dtype,
                           double eps) {
  if (ld <= 0 || n % ld != 0) return -2;
  int64_t rows = n / ld;
  int failed = 0;
#pragma omp parallel
  {
    double* x = (double*)malloc(sizeof(double) * (size_t)ld); /* one row, per thread */
    if (!x) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
      if (!x) continue;
      for (int i = 0; i < ld; ++i) {
        double v = load_elem(input, dtype, r * ld + i);
        if (skip) v += load_elem(skip, dtype, r * ld + i);
        if (bias) v += bias[i];
        x[i] = v;
      }
      ln_row(x, ld, gamma, beta, eps, output, dtype, r * (int64_t)ld);
    }
    free(x);
  }
  return failed ? -3 : 0;
}

/*
 * BERT embedding + LayerNorm on [S,B] ids (trt_bert_creator.h:64-71 transposes to [S,B]):
 * token t = s*B + b;  x = word[input_ids[t]] + pos[s] + tok[segment_ids[t]];  out[t,:] = LN(x).
 * mask_idx[b] = index of the first 0 in input_mask[:, b], or S when the column has none
 * (equals the valid length for prefix masks).  Ids outside their table contribute a zero row
 * and are counted in the return value.
 */
int64_t oracle_emb_layer_norm(int S, int B, int ld, const int32_t* input_ids,
                              const int32_t* segment_ids, const int32_t* input_mask,
                              const float* beta, const float* gamma, const void* word,
                              const void* pos, const void* tok, int word_count, int pos_count,
                              int tok_count, void* output, int32_t* mask_idx, int dtype,
                              double eps) {
  int64_t oob = 0;
  if (ld <= 0) return -2;
  int failed = 0;
#pragma omp parallel reduction(+ : oob)
  {
  double* x = (double*)malloc(sizeof(double) * (size_t)ld); /* one row, per thread */
  if (!x) {
#pragma omp atomic write
    failed = 1;
  }
#pragma omp for schedule(static)
  for (int64_t t = 0; t < (int64_t)S * B; ++t) {
    if (!x) continue;
    int s = (int)(t / B);
    int64_t w = input_ids[t], g = segment_ids[t];
    int wok = w >= 0 && w < word_count, gok = g >= 0 && g < tok_count, pok = s < pos_count;
    if (!wok) ++oob;
    if (!gok) ++oob;
    if (!pok) ++oob;
    for (int i = 0; i < ld; ++i) {
      double v = 0.0;
      if (wok) v += load_elem(word, dtype, w * ld + i);
      if (pok) v += load_elem(pos, dtype, (int64_t)s * ld + i);
      if (gok) v += load_elem(tok, dtype, g * ld + i);
      x[i] = v;
    }
    ln_row(x, ld, gamma, beta, eps, output, dtype, t * (int64_t)ld);
  }
  free(x);
  }
  if (failed) return -3;
  if (mask_idx && input_mask) {
    for (int b = 0; b < B; ++b) {
      int first = S;
      for (int s = 0; s < S; ++s)
        if (input_mask[(int64_t)s * B + b] == 0) {
          first = s;
          break;
        }
      mask_idx[b] = first;
    }
  }
  return oob;
}
