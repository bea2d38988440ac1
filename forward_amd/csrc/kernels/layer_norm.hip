// LayerNorm family for gfx950: plain LayerNorm with optional pre-bias, SkipLayerNorm
// (input + skip (+ bias)) and the BERT embedding lookup fused with LayerNorm (+ mask index).
//
// One wavefront owns one row.  Each lane keeps its 128-bit slices of the row in registers
// (row read once), computes its own mean and centred sum of squares, and the 64 partial
// (count, mean, M2) triples are merged with a butterfly of DPP row operations and two
// cross-row shuffles (Chan's parallel Welford update), all in fp32.  gamma / beta (/ bias)
// live in registers and are reused for every row the wavefront processes.
//
// Rows of at most 512 bytes share a wavefront (64/G rows at a time, G lanes each); rows too long
// for one wavefront's registers take a workgroup per row, and so do rows whose length or
// alignment rule out 128-bit access and do not fit a wavefront (one element per lane per slice).
// Rows beyond a workgroup's registers are streamed twice by a workgroup (the second time from
// cache).  What is left (embedding rows of more than 512 elements without 128-bit access) takes
// the strided kernel: one element per lane per step, row read twice.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../common.h"
#include "device_util.h"

// No implicit multiply-add fusion in this file: the fused kernel and the separate launches must
// round identically, so every fused operation is written as an explicit fma.
#pragma clang fp contract(off)

namespace fwdmi {
namespace {

// Row-processing workgroups per CU.  With 4 (16 wavefronts per CU) a wavefront of the 8192-token
// configuration handles two rows, so the second row's loads overlap the first row's arithmetic and
// store; measured best among 2 / 4 / 6 / 8 / 16.
#ifndef FWDMI_LN_BLOCKS_PER_CU
#define FWDMI_LN_BLOCKS_PER_CU 4
#endif
constexpr int kWG = 256;
constexpr int kWavesPerWG = kWG / 64;

enum Mode { kLayerNorm = 0, kSkip = 1, kEmb = 2, kEmbSkip = 3 };
constexpr bool is_emb(int mode) { return mode == kEmb || mode == kEmbSkip; }

struct LnLaunch {
  const void* input;  // kLayerNorm / kSkip: [rows, ld]; kEmb: word table
  const void* skip;   // kSkip: [rows, ld]
  const void* pos;    // kEmb
  const void* tok;    // kEmb
  const float* gamma;
  const float* beta;
  const float* bias;  // nullable
  const float* gamma2;  // kEmbSkip: parameters of the second LayerNorm
  const float* beta2;
  const float* bias2;   // nullable
  void* emb_output;     // kEmbSkip: optional copy of the first-stage result
  void* output;
  const int32_t* input_ids;
  const int32_t* segment_ids;
  const int32_t* input_mask;
  int32_t* mask_idx;
  int32_t* oob_flag;
  int64_t rows;
  int32_t ld;
  int32_t S, B;
  int32_t word_count, pos_count, tok_count;
  int32_t row_blocks;  // workgroups that process rows; the rest compute mask indices
  int32_t total_waves; // row-processing wavefronts in the grid
  float eps;
  float eps2;
  float one;  // 1.0f, as a run-time value (see the row sum in ln_rows_kernel)
  int32_t batch_major;  // kEmb*: ids / mask are [B,S] and rows are ordered b*S + s
};

// Rounds an fp32 result to the I/O type in a step of its own.  Without the barrier the compiler
// may fold the preceding fma and the conversion into one mixed-precision instruction that rounds
// once; whether it does depends on the surrounding code, and the fused and the two-launch forms
// of the same arithmetic would then differ in the last bit.
template <typename T>
__device__ __forceinline__ T round_to(float y) {
  asm volatile("" : "+v"(y));
  return (T)y;
}

struct Welford {
  float n, mean, m2;
};

__device__ __forceinline__ Welford merge(const Welford a, const Welford b) {
  Welford r;
  r.n = a.n + b.n;
  // counts are small integers: the hardware reciprocal (1 ulp) is ample here
  const float inv = r.n > 0.0f ? __builtin_amdgcn_rcpf(r.n) : 0.0f;
  const float d = b.mean - a.mean;
  r.mean = a.mean + d * (b.n * inv);
  r.m2 = a.m2 + b.m2 + d * d * (a.n * b.n * inv);
  return r;
}

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}

template <int CTRL>
__device__ __forceinline__ Welford dpp(const Welford w) {
  return Welford{dpp<CTRL>(w.n), dpp<CTRL>(w.mean), dpp<CTRL>(w.m2)};
}

__device__ __forceinline__ Welford xor_lanes(const Welford w, int mask) {
  return Welford{__shfl_xor(w.n, mask), __shfl_xor(w.mean, mask), __shfl_xor(w.m2, mask)};
}

// After this every lane holds the statistics of all 64 lanes.
__device__ __forceinline__ Welford wave_allreduce(Welford w) {
  w = merge(w, dpp<0xB1>(w));   // quad_perm [1,0,3,2]: lane ^ 1
  w = merge(w, dpp<0x4E>(w));   // quad_perm [2,3,0,1]: lane ^ 2
  w = merge(w, dpp<0x141>(w));  // row_half_mirror: the other quad of each 8
  w = merge(w, dpp<0x140>(w));  // row_mirror: the other half of each row of 16
  w = merge(w, xor_lanes(w, 16));
  w = merge(w, xor_lanes(w, 32));
  // Lanes agree up to rounding (merge is not bitwise symmetric); take lane 0's value everywhere.
  w.n = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(w.n)));
  w.mean = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(w.mean)));
  w.m2 = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(w.m2)));
  return w;
}

// The same when every lane starts with the same count `n0`: the two sides of every merge then
// hold equal counts, which turns the update into mean = (a + b) / 2 and
// M2 = M2a + M2b + (b - a)^2 * n / 2 with n known at compile time per level.
struct MeanM2 {
  float mean, m2;
};
__device__ __forceinline__ MeanM2 merge_equal(const MeanM2 a, const MeanM2 b, float half_n) {
  const float d = b.mean - a.mean;
  return MeanM2{__builtin_fmaf(d, 0.5f, a.mean), __builtin_fmaf(d * d, half_n, a.m2 + b.m2)};
}
template <int CTRL>
__device__ __forceinline__ MeanM2 dpp(const MeanM2 w) {
  return MeanM2{dpp<CTRL>(w.mean), dpp<CTRL>(w.m2)};
}
__device__ __forceinline__ Welford wave_allreduce_equal(float mean, float m2, float n0) {
  MeanM2 w{mean, m2};
  w = merge_equal(w, dpp<0xB1>(w), 0.5f * n0);
  w = merge_equal(w, dpp<0x4E>(w), 1.0f * n0);
  w = merge_equal(w, dpp<0x141>(w), 2.0f * n0);
  w = merge_equal(w, dpp<0x140>(w), 4.0f * n0);
  w = merge_equal(w, MeanM2{__shfl_xor(w.mean, 16), __shfl_xor(w.m2, 16)}, 8.0f * n0);
  w = merge_equal(w, MeanM2{__shfl_xor(w.mean, 32), __shfl_xor(w.m2, 32)}, 16.0f * n0);
  Welford r;
  r.n = 64.0f * n0;
  r.mean = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(w.mean)));
  r.m2 = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(w.m2)));
  return r;
}

__device__ __forceinline__ int wave_min(int v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = min(v, __shfl_xor(v, m));
  return v;
}

// Index of the first zero of the mask of batch row b, S when there is none.
__device__ __forceinline__ void mask_index_wave(const LnLaunch& L, int b, int lane) {
  int first = L.S;
  const int64_t base = L.batch_major ? (int64_t)b * L.S : b;
  const int64_t step = L.batch_major ? 1 : L.B;
  // Eight positions per lane are read before the first is looked at: one trip to memory for
  // sequences of up to 512 positions instead of one per 64 (the kernel lasts as long as its slowest
  // wavefront, and in sequence-major layout every one of these loads is a cache line of its own).
  constexpr int kAhead = 8;
  for (int s0 = lane; s0 < L.S; s0 += 64 * kAhead) {
    int v[kAhead];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
      const int s = s0 + 64 * k;
      v[k] = s < L.S ? L.input_mask[base + (int64_t)s * step] : 1;
    }
#pragma unroll
    for (int k = kAhead - 1; k >= 0; --k)
      if (v[k] == 0) first = s0 + 64 * k;  // descending: the earliest position is assigned last
    if (__builtin_amdgcn_ballot_w64(first != L.S) != 0) break;  // a zero in this block: none earlier remains unseen
  }
  first = wave_min(first);
  if (lane == 0) L.mask_idx[b] = first;
}

// Register image of one row's operands: up to three 16-byte slices per chunk.
template <typename T, int VEC, int NV, int MODE>
struct RowRegs {
  Pack<T, VEC> a[NV];                        // input / word row
  Pack<T, VEC> b[MODE == kLayerNorm ? 1 : NV];  // skip / position row
  Pack<T, VEC> c[is_emb(MODE) ? NV : 1];     // token-type row
  Pack<T, VEC> d[MODE == kEmbSkip ? NV : 1]; // residual of the fused second stage
  bool ok0, ok1, ok2;
};

// FULL: ld == 64 * VEC * NV, i.e. every lane owns NV live slices (no masking, equal counts).
template <typename T, int VEC, int NV, int MODE, bool FULL>
__global__ __launch_bounds__(kWG) void ln_rows_kernel(const LnLaunch L) {
  const int lane = threadIdx.x & 63;
  const int wave_in_wg = threadIdx.x >> 6;
  if ((int)blockIdx.x >= L.row_blocks) {
    if (is_emb(MODE)) {
      const int b = ((int)blockIdx.x - L.row_blocks) * kWavesPerWG + wave_in_wg;
      if (b < L.B) mask_index_wave(L, b, lane);
    }
    return;
  }
  // The row a wavefront works on is the same in all of its lanes; saying so keeps row addresses
  // in scalar registers (uniform base + per-lane column offset) and lets the ids of an embedding
  // row come through the scalar unit.
  const int wave = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * kWavesPerWG + wave_in_wg));
  const T FWDMI_GLOBAL* const in0 = gconst<T>(L.input);
  const T FWDMI_GLOBAL* const in1 = gconst<T>(is_emb(MODE) ? L.pos : L.skip);
  const T FWDMI_GLOBAL* const in3 = gconst<T>(L.skip);
  const T FWDMI_GLOBAL* const in2 = gconst<T>(L.tok);

  // Per-lane column slices: chunk j covers elements (j*64 + lane)*VEC .. +VEC.
  bool live[NV];
  int col[NV];
  float cnt = 0.0f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = (j * 64 + lane) * VEC;
    live[j] = FULL || c < L.ld;
    col[j] = live[j] ? c : 0;
    if (live[j]) cnt += (float)VEC;
  }
  const float inv_cnt = cnt > 0.0f ? 1.0f / cnt : 0.0f;

  using Regs = RowRegs<T, VEC, NV, MODE>;
  // Issues the loads of row r (no use of the data yet).
  auto fetch = [&](int64_t r, Regs& R) {
    if (is_emb(MODE)) {
      const int s = L.batch_major ? (int)(r % L.S) : (int)(r / L.B);
      typedef const int32_t __attribute__((address_space(4))) * ConstIds;  // read-only for the whole launch
      const int64_t w = ((ConstIds)L.input_ids)[r], sg = ((ConstIds)L.segment_ids)[r];
      R.ok0 = w >= 0 && w < L.word_count;
      R.ok1 = s < L.pos_count;
      R.ok2 = sg >= 0 && sg < L.tok_count;
      const T FWDMI_GLOBAL* wp = in0 + (R.ok0 ? w : 0) * L.ld;
      const T FWDMI_GLOBAL* pp = in1 + (int64_t)(R.ok1 ? s : 0) * L.ld;
      const T FWDMI_GLOBAL* tp = in2 + (R.ok2 ? sg : 0) * L.ld;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        R.a[j] = gload<T, VEC>(wp + col[j]);
        R.b[j] = gload<T, VEC>(pp + col[j]);
        R.c[j] = gload<T, VEC>(tp + col[j]);
        if (MODE == kEmbSkip) R.d[j] = gload<T, VEC>(in3 + r * L.ld + col[j]);
      }
    } else {
      R.ok0 = R.ok1 = R.ok2 = true;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        R.a[j] = gload<T, VEC>(in0 + r * L.ld + col[j]);
        if (MODE == kSkip) R.b[j] = gload<T, VEC>(in1 + r * L.ld + col[j]);
      }
    }
  };

  // gamma / beta / bias stay in registers for every row this wavefront handles.
  float g[NV][VEC], be[NV][VEC], bi[NV][VEC];
  Regs cur, nxt;
  int64_t r = wave;
  if (r < L.rows) fetch(r, cur);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const Pack<float, VEC> pg = gload<float, VEC>(gconst<float>(L.gamma) + col[j]);
    const Pack<float, VEC> pb = gload<float, VEC>(gconst<float>(L.beta) + col[j]);
    Pack<float, VEC> pi{};
    if (L.bias) pi = gload<float, VEC>(gconst<float>(L.bias) + col[j]);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      g[j][e] = pg.v[e];
      be[j][e] = pb.v[e];
      bi[j][e] = L.bias ? pi.v[e] : 0.0f;
    }
  }

  bool oob = false;
  const float one = L.one;
  for (; r < L.rows; r += L.total_waves) {
    // the next row's loads are in flight while this row is reduced
    const int64_t rn = r + L.total_waves;
    if (rn < L.rows) fetch(rn, nxt);

    float x[NV][VEC];
    if (is_emb(MODE) && !(cur.ok0 && cur.ok1 && cur.ok2)) {  // uniform and rare: an id outside its table
      oob = true;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        if (!cur.ok0) cur.a[j] = Pack<T, VEC>{};
        if (!cur.ok1) cur.b[j] = Pack<T, VEC>{};
        if (!cur.ok2) cur.c[j] = Pack<T, VEC>{};
      }
    }
    // fma(b, 1, a) rounds exactly like a + b and lets half-precision operands enter the sum
    // without conversions of their own (mixed-precision FMA); `one` is a kernel argument so that
    // the multiplication is not folded away.
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float v = (float)cur.a[j].v[e];
        if (MODE != kLayerNorm) v = __builtin_fmaf((float)cur.b[j].v[e], one, v);
        if (is_emb(MODE)) v = __builtin_fmaf((float)cur.c[j].v[e], one, v);
        x[j][e] = is_emb(MODE) ? v : v + bi[j][e];
      }

    // lane-local statistics, then the wave-wide merge: returns (mean, 1/sigma)
    auto stats = [&](float eps, float& mu, float& rs) {
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int e = 0; e < VEC; ++e) sum += (FULL || live[j]) ? x[j][e] : 0.0f;
      Welford w{cnt, sum * inv_cnt, 0.0f};
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = (FULL || live[j]) ? x[j][e] - w.mean : 0.0f;
          w.m2 = __builtin_fmaf(d, d, w.m2);
        }
      w = FULL ? wave_allreduce_equal(w.mean, w.m2, (float)(NV * VEC)) : wave_allreduce(w);
      mu = w.mean;
      // hardware reciprocal and reciprocal square root (1 ulp each) instead of the IEEE sequences
      rs = __builtin_amdgcn_rsqf(__builtin_fmaf(w.m2, __builtin_amdgcn_rcpf(w.n), eps));
    };
    float mu, rs;
    stats(L.eps, mu, rs);

    if (MODE != kEmbSkip) {
      T FWDMI_GLOBAL* op = gmut<T>(L.output) + r * L.ld;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        if (live[j]) {
          Pack<T, VEC> o;
#pragma unroll
          for (int e = 0; e < VEC; ++e) o.v[e] = round_to<T>(__builtin_fmaf(g[j][e], (x[j][e] - mu) * rs, be[j][e]));
          gstore<T, VEC>(op + col[j], o);
        }
      }
    } else {
      // Fused second stage: the first result is rounded to the I/O type exactly as if it had
      // been stored and read back, then out = LN2(first + residual (+ bias2)).
      T FWDMI_GLOBAL* ep = L.emb_output ? gmut<T>(L.emb_output) + r * L.ld : nullptr;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        Pack<T, VEC> o;
        Pack<float, VEC> b2{};
        if (L.bias2) b2 = gload<float, VEC>(gconst<float>(L.bias2) + col[j]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          o.v[e] = round_to<T>(__builtin_fmaf(g[j][e], (x[j][e] - mu) * rs, be[j][e]));
          x[j][e] = __builtin_fmaf((float)cur.d[j].v[e], one, (float)o.v[e]) + (L.bias2 ? b2.v[e] : 0.0f);
        }
        if (ep && live[j]) gstore<T, VEC>(ep + col[j], o);
      }
      stats(L.eps2, mu, rs);
      T FWDMI_GLOBAL* op = gmut<T>(L.output) + r * L.ld;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        if (live[j]) {
          const Pack<float, VEC> g2 = gload<float, VEC>(gconst<float>(L.gamma2) + col[j]);
          const Pack<float, VEC> be2 = gload<float, VEC>(gconst<float>(L.beta2) + col[j]);
          Pack<T, VEC> o;
#pragma unroll
          for (int e = 0; e < VEC; ++e) o.v[e] = round_to<T>(__builtin_fmaf(g2.v[e], (x[j][e] - mu) * rs, be2.v[e]));
          gstore<T, VEC>(op + col[j], o);
        }
      }
    }
    cur = nxt;
  }
  if (oob && L.oob_flag) atomicOr(L.oob_flag, 1);
}

// Narrow rows (at most 32 lanes of 16 bytes): a wavefront works on 64/G rows at a time, G lanes
// per row, so that short rows still fill the 64 lanes.  kLayerNorm / kSkip / kEmb.
template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kWG) void ln_narrow_kernel(const LnLaunch L, const int log2_g) {
  const int lane = threadIdx.x & 63;
  if (MODE == kEmb && (int)blockIdx.x >= L.row_blocks) {
    const int b = ((int)blockIdx.x - L.row_blocks) * kWavesPerWG + (threadIdx.x >> 6);
    if (b < L.B) mask_index_wave(L, b, lane);
    return;
  }
  const int G = 1 << log2_g;
  const int rows_per_wave = 64 >> log2_g;
  const int sub = lane >> log2_g;
  const int gl = lane & (G - 1);
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerWG + (threadIdx.x >> 6);
  const T FWDMI_GLOBAL* const in0 = gconst<T>(L.input);
  const T FWDMI_GLOBAL* const in1 = gconst<T>(MODE == kEmb ? L.pos : L.skip);
  const T FWDMI_GLOBAL* const in2 = gconst<T>(L.tok);
  const bool live = gl * VEC < L.ld;
  const int col = live ? gl * VEC : 0;
  const float cnt = live ? (float)VEC : 0.0f;
  bool oob = false;
  float g[VEC], be[VEC], bi[VEC];
  {
    const Pack<float, VEC> pg = gload<float, VEC>(gconst<float>(L.gamma) + col);
    const Pack<float, VEC> pb = gload<float, VEC>(gconst<float>(L.beta) + col);
    Pack<float, VEC> pi{};
    if (L.bias) pi = gload<float, VEC>(gconst<float>(L.bias) + col);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      g[e] = pg.v[e];
      be[e] = pb.v[e];
      bi[e] = L.bias ? pi.v[e] : 0.0f;
    }
  }
  const float one = L.one;
  const int64_t stride = (int64_t)L.total_waves * rows_per_wave;
  for (int64_t r0 = wave * rows_per_wave; r0 < L.rows; r0 += stride) {
    const int64_t r = r0 + sub;
    const bool row_ok = r < L.rows;
    const int64_t rr = row_ok ? r : L.rows - 1;  // lanes past the last row repeat it and store nothing
    Pack<T, VEC> a{}, b{}, c{};
    if (MODE == kEmb) {
      // word + position + token-type rows of token rr; an id outside its table contributes zeros
      const int s = L.batch_major ? (int)(rr % L.S) : (int)(rr / L.B);
      const int64_t w = L.input_ids[rr], sg = L.segment_ids[rr];
      const bool ok0 = w >= 0 && w < L.word_count, ok1 = s < L.pos_count, ok2 = sg >= 0 && sg < L.tok_count;
      oob |= row_ok && !(ok0 && ok1 && ok2);
      if (ok0) a = gload<T, VEC>(in0 + w * L.ld + col);
      if (ok1) b = gload<T, VEC>(in1 + (int64_t)s * L.ld + col);
      if (ok2) c = gload<T, VEC>(in2 + sg * L.ld + col);
    } else {
      a = gload<T, VEC>(in0 + rr * L.ld + col);
      if (MODE == kSkip) b = gload<T, VEC>(in1 + rr * L.ld + col);
    }
    float x[VEC], sum = 0.0f;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float v = (float)a.v[e];
      if (MODE != kLayerNorm) v = __builtin_fmaf((float)b.v[e], one, v);
      if (MODE == kEmb) v = __builtin_fmaf((float)c.v[e], one, v);
      x[e] = MODE == kEmb ? v : v + bi[e];
      sum += live ? x[e] : 0.0f;
    }
    Welford w{cnt, sum * (1.0f / (float)VEC), 0.0f};
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float d = live ? x[e] - w.mean : 0.0f;
      w.m2 = __builtin_fmaf(d, d, w.m2);
    }
    for (int m = 1; m < G; m <<= 1) w = merge(w, xor_lanes(w, m));
    // the lanes of a row agree up to rounding: all take the value of the row's first lane
    w.n = __shfl(w.n, 0, G);
    w.mean = __shfl(w.mean, 0, G);
    w.m2 = __shfl(w.m2, 0, G);
    const float mu = w.mean;
    const float rs = __builtin_amdgcn_rsqf(__builtin_fmaf(w.m2, __builtin_amdgcn_rcpf(w.n), L.eps));
    if (row_ok && live) {
      Pack<T, VEC> o;
#pragma unroll
      for (int e = 0; e < VEC; ++e) o.v[e] = round_to<T>(__builtin_fmaf(g[e], (x[e] - mu) * rs, be[e]));
      gstore<T, VEC>(gmut<T>(L.output) + r * L.ld + col, o);
    }
  }
  if (MODE == kEmb && oob && L.oob_flag) atomicOr(L.oob_flag, 1);
}

// Wide rows (more than 8 slices per lane of a wavefront): a workgroup of 256 lanes owns a row,
// NV slices per lane in registers (row read once), wavefront statistics merged through LDS.
// gamma / beta / bias are re-read per row (from cache).  kLayerNorm / kSkip only.
template <typename T, int VEC, int NV, int MODE>
__global__ __launch_bounds__(kWG) void ln_block_kernel(const LnLaunch L) {
  __shared__ float s_part[kWavesPerWG][4];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_in_wg = tid >> 6;
  const T FWDMI_GLOBAL* const in0 = gconst<T>(L.input);
  const T FWDMI_GLOBAL* const in1 = gconst<T>(L.skip);
  bool live[NV];
  int col[NV];
  float cnt = 0.0f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = (j * kWG + tid) * VEC;
    live[j] = c < L.ld;
    col[j] = live[j] ? c : 0;
    if (live[j]) cnt += (float)VEC;
  }
  const float inv_cnt = cnt > 0.0f ? 1.0f / cnt : 0.0f;
  const float one = L.one;
  for (int64_t r = blockIdx.x; r < L.rows; r += gridDim.x) {
    Pack<T, VEC> a[NV], b[MODE == kSkip ? NV : 1];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      a[j] = gload<T, VEC>(in0 + r * L.ld + col[j]);
      if (MODE == kSkip) b[j] = gload<T, VEC>(in1 + r * L.ld + col[j]);
    }
    float x[NV][VEC], sum = 0.0f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      Pack<float, VEC> pi{};
      if (L.bias) pi = gload<float, VEC>(gconst<float>(L.bias) + col[j]);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float v = (float)a[j].v[e];
        if (MODE == kSkip) v = __builtin_fmaf((float)b[j].v[e], one, v);
        x[j][e] = v + (L.bias ? pi.v[e] : 0.0f);
        sum += live[j] ? x[j][e] : 0.0f;
      }
    }
    Welford w{cnt, sum * inv_cnt, 0.0f};
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = live[j] ? x[j][e] - w.mean : 0.0f;
        w.m2 = __builtin_fmaf(d, d, w.m2);
      }
    w = wave_allreduce(w);
    if (lane == 0) {
      s_part[wave_in_wg][0] = w.n;
      s_part[wave_in_wg][1] = w.mean;
      s_part[wave_in_wg][2] = w.m2;
    }
    __syncthreads();
    Welford t{s_part[0][0], s_part[0][1], s_part[0][2]};
#pragma unroll
    for (int k = 1; k < kWavesPerWG; ++k) t = merge(t, Welford{s_part[k][0], s_part[k][1], s_part[k][2]});
    __syncthreads();  // s_part is rewritten for the next row
    const float mu = t.mean;
    const float rs = __builtin_amdgcn_rsqf(__builtin_fmaf(t.m2, __builtin_amdgcn_rcpf(t.n), L.eps));
    T FWDMI_GLOBAL* op = gmut<T>(L.output) + r * L.ld;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      if (live[j]) {
        const Pack<float, VEC> pg = gload<float, VEC>(gconst<float>(L.gamma) + col[j]);
        const Pack<float, VEC> pb = gload<float, VEC>(gconst<float>(L.beta) + col[j]);
        Pack<T, VEC> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o.v[e] = round_to<T>(__builtin_fmaf(pg.v[e], (x[j][e] - mu) * rs, pb.v[e]));
        gstore<T, VEC>(op + col[j], o);
      }
    }
  }
}

// Rows beyond a workgroup's registers: a workgroup per row, two passes over the row in slices of
// VEC elements per lane.  The first pass accumulates sums of (x - x0) and (x - x0)^2 with x0 the
// row's first element (the shifted form keeps the cancellation of the one-pass variance small),
// the second pass re-reads the row (from cache) and writes the result.  kLayerNorm / kSkip only.
template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kWG) void ln_stream_kernel(const LnLaunch L) {
  __shared__ float s_part[kWavesPerWG][4];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_in_wg = tid >> 6;
  const T FWDMI_GLOBAL* const in0 = gconst<T>(L.input);
  const T FWDMI_GLOBAL* const in1 = gconst<T>(L.skip);
  const float one = L.one;
  auto value = [&](int64_t base, int c, float* x) {
    const Pack<T, VEC> a = gload<T, VEC>(in0 + base + c);
    Pack<T, VEC> b{};
    if (MODE == kSkip) b = gload<T, VEC>(in1 + base + c);
    Pack<float, VEC> pi{};
    if (L.bias) pi = gload<float, VEC>(gconst<float>(L.bias) + c);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float v = (float)a.v[e];
      if (MODE == kSkip) v = __builtin_fmaf((float)b.v[e], one, v);
      x[e] = v + (L.bias ? pi.v[e] : 0.0f);
    }
  };
  for (int64_t r = blockIdx.x; r < L.rows; r += gridDim.x) {
    const int64_t base = r * L.ld;
    float x0;
    {
      float v = (float)in0[base];
      if (MODE == kSkip) v = __builtin_fmaf((float)in1[base], one, v);
      x0 = v + (L.bias ? L.bias[0] : 0.0f);
    }
    float n = 0.0f, s1 = 0.0f, s2 = 0.0f;
    for (int c = tid * VEC; c < L.ld; c += kWG * VEC) {
      float x[VEC];
      value(base, c, x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = x[e] - x0;
        s1 += d;
        s2 = __builtin_fmaf(d, d, s2);
      }
      n += (float)VEC;
    }
    Welford w{n, 0.0f, 0.0f};
    if (n > 0.0f) {
      const float inv = 1.0f / n;
      w.mean = x0 + s1 * inv;
      w.m2 = fmaxf(s2 - s1 * s1 * inv, 0.0f);
    }
    w = wave_allreduce(w);
    if (lane == 0) {
      s_part[wave_in_wg][0] = w.n;
      s_part[wave_in_wg][1] = w.mean;
      s_part[wave_in_wg][2] = w.m2;
    }
    __syncthreads();
    Welford t{s_part[0][0], s_part[0][1], s_part[0][2]};
#pragma unroll
    for (int k = 1; k < kWavesPerWG; ++k) t = merge(t, Welford{s_part[k][0], s_part[k][1], s_part[k][2]});
    __syncthreads();  // s_part is rewritten for the next row
    const float mu = t.mean;
    const float rs = __builtin_amdgcn_rsqf(__builtin_fmaf(t.m2, __builtin_amdgcn_rcpf(t.n), L.eps));
    T FWDMI_GLOBAL* op = gmut<T>(L.output) + base;
    for (int c = tid * VEC; c < L.ld; c += kWG * VEC) {
      float x[VEC];
      value(base, c, x);
      const Pack<float, VEC> pg = gload<float, VEC>(gconst<float>(L.gamma) + c);
      const Pack<float, VEC> pb = gload<float, VEC>(gconst<float>(L.beta) + c);
      Pack<T, VEC> o;
#pragma unroll
      for (int e = 0; e < VEC; ++e) o.v[e] = round_to<T>(__builtin_fmaf(pg.v[e], (x[e] - mu) * rs, pb.v[e]));
      gstore<T, VEC>(op + c, o);
    }
  }
}

// Any ld, any alignment: one element per lane per step, two passes over the row.
template <typename T, int MODE>
__global__ __launch_bounds__(kWG) void ln_strided_kernel(const LnLaunch L) {
  const int lane = threadIdx.x & 63;
  const int wave_in_wg = threadIdx.x >> 6;
  if ((int)blockIdx.x >= L.row_blocks) {
    if (MODE == kEmb) {
      const int b = ((int)blockIdx.x - L.row_blocks) * kWavesPerWG + wave_in_wg;
      if (b < L.B) mask_index_wave(L, b, lane);
    }
    return;
  }
  const int wave = blockIdx.x * kWavesPerWG + wave_in_wg;
  bool oob = false;
  for (int64_t r = wave; r < L.rows; r += L.total_waves) {
    const T *p0 = nullptr, *p1 = nullptr, *p2 = nullptr;
    bool ok0 = true, ok1 = false, ok2 = false;
    if (MODE == kEmb) {
      const int s = L.batch_major ? (int)(r % L.S) : (int)(r / L.B);
      const int64_t w = L.input_ids[r], sg = L.segment_ids[r];
      ok0 = w >= 0 && w < L.word_count;
      ok1 = s < L.pos_count;
      ok2 = sg >= 0 && sg < L.tok_count;
      oob |= !(ok0 && ok1 && ok2);
      p0 = static_cast<const T*>(L.input) + (ok0 ? w : 0) * L.ld;
      p1 = static_cast<const T*>(L.pos) + (int64_t)(ok1 ? s : 0) * L.ld;
      p2 = static_cast<const T*>(L.tok) + (ok2 ? sg : 0) * L.ld;
    } else {
      p0 = static_cast<const T*>(L.input) + r * L.ld;
      if (MODE == kSkip) {
        p1 = static_cast<const T*>(L.skip) + r * L.ld;
        ok1 = true;
      }
    }
    auto fetch = [&](int i) {
      float v = ok0 ? (float)p0[i] : 0.0f;
      if (MODE != kLayerNorm) v += ok1 ? (float)p1[i] : 0.0f;
      if (MODE == kEmb) v += ok2 ? (float)p2[i] : 0.0f;
      if (MODE != kEmb && L.bias) v += L.bias[i];
      return v;
    };
    Welford w{0.0f, 0.0f, 0.0f};
    for (int i = lane; i < L.ld; i += 64) {
      const float v = fetch(i);
      w.n += 1.0f;
      const float d = v - w.mean;
      w.mean += d / w.n;
      w.m2 = __builtin_fmaf(d, v - w.mean, w.m2);
    }
    w = wave_allreduce(w);
    const float mu = w.mean;
    const float rs = 1.0f / sqrtf(w.m2 / w.n + L.eps);
    T* op = static_cast<T*>(L.output) + r * L.ld;
    for (int i = lane; i < L.ld; i += 64) op[i] = round_to<T>(__builtin_fmaf(L.gamma[i], (fetch(i) - mu) * rs, L.beta[i]));
  }
  if (oob && L.oob_flag) atomicOr(L.oob_flag, 1);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) % 16) == 0; }

template <typename T, int MODE>
int ln_launch(LnLaunch& L, bool vec_ok, hipStream_t stream) {
  constexpr int kVec = 16 / sizeof(T);
  static const int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      return v;
    return 256;
  }();
  // Enough wavefronts to fill the chip; beyond that a wavefront loops over rows so the
  // gamma/beta registers are reused.
  const int64_t max_blocks = (int64_t)cus * FWDMI_LN_BLOCKS_PER_CU;
  const int64_t want = (L.rows + kWavesPerWG - 1) / kWavesPerWG;
  L.row_blocks = (int)std::max<int64_t>(1, std::min(want, max_blocks));
  L.total_waves = L.row_blocks * kWavesPerWG;
  const int mask_blocks = (is_emb(MODE) && L.mask_idx) ? (L.B + kWavesPerWG - 1) / kWavesPerWG : 0;
  const dim3 grid(L.row_blocks + mask_blocks), block(kWG);

  const int chunks = (L.ld + 64 * kVec - 1) / (64 * kVec);
  const bool sliceable = vec_ok && (L.ld % kVec) == 0;
  if constexpr (MODE == kEmb) {
    if (sliceable && L.ld / kVec <= 32) {
      // several tokens per wavefront (hidden sizes of at most 512 bytes)
      int log2_g = 0;
      while ((1 << log2_g) < L.ld / kVec) ++log2_g;
      const int rows_per_wg = kWavesPerWG * (64 >> log2_g);
      const int64_t blocks = std::max<int64_t>(1, std::min((L.rows + rows_per_wg - 1) / rows_per_wg, (int64_t)cus * 8));
      L.row_blocks = (int)blocks;
      L.total_waves = (int)blocks * kWavesPerWG;
      hipLaunchKernelGGL((ln_narrow_kernel<T, kVec, MODE>), dim3((unsigned)(blocks + mask_blocks)), block, 0, stream, L,
                         log2_g);
      FWDMI_HIP_CHECK(hipGetLastError());
      return FWDMI_OK;
    }
  }
  if constexpr (!is_emb(MODE)) {
    if (sliceable && L.ld / kVec <= 32) {
      // several rows per wavefront
      int log2_g = 0;
      while ((1 << log2_g) < L.ld / kVec) ++log2_g;
      const int rows_per_wg = kWavesPerWG * (64 >> log2_g);
      const int64_t blocks = std::max<int64_t>(1, std::min((L.rows + rows_per_wg - 1) / rows_per_wg, (int64_t)cus * 8));
      L.total_waves = (int)blocks * kWavesPerWG;
      hipLaunchKernelGGL((ln_narrow_kernel<T, kVec, MODE>), dim3((unsigned)blocks), block, 0, stream, L, log2_g);
      FWDMI_HIP_CHECK(hipGetLastError());
      return FWDMI_OK;
    }
    if (!sliceable && L.ld <= 32) {
      // rows of at most 32 elements of any alignment (the reference's small-row case,
      // layer_norm_kernel.cu:285-288): one element per lane, 64/G rows per wavefront
      int log2_g = 0;
      while ((1 << log2_g) < L.ld) ++log2_g;
      const int rows_per_wg = kWavesPerWG * (64 >> log2_g);
      const int64_t blocks = std::max<int64_t>(1, std::min((L.rows + rows_per_wg - 1) / rows_per_wg, (int64_t)cus * 8));
      L.total_waves = (int)blocks * kWavesPerWG;
      hipLaunchKernelGGL((ln_narrow_kernel<T, 1, MODE>), dim3((unsigned)blocks), block, 0, stream, L, log2_g);
      FWDMI_HIP_CHECK(hipGetLastError());
      return FWDMI_OK;
    }
    const int block_chunks = (L.ld + kWG * kVec - 1) / (kWG * kVec);
    if (sliceable && chunks > 8 && block_chunks <= 8) {
      // a workgroup per row
      const dim3 bgrid((unsigned)std::max<int64_t>(1, std::min(L.rows, (int64_t)cus * 8)));
      if (block_chunks <= 4)
        hipLaunchKernelGGL((ln_block_kernel<T, kVec, 4, MODE>), bgrid, block, 0, stream, L);
      else
        hipLaunchKernelGGL((ln_block_kernel<T, kVec, 8, MODE>), bgrid, block, 0, stream, L);
      FWDMI_HIP_CHECK(hipGetLastError());
      return FWDMI_OK;
    }
    if (!sliceable && L.ld > 64 * 8 && L.ld <= kWG * 32) {
      const dim3 bgrid((unsigned)std::max<int64_t>(1, std::min(L.rows, (int64_t)cus * 8)));
      if (L.ld <= kWG * 4)
        hipLaunchKernelGGL((ln_block_kernel<T, 1, 4, MODE>), bgrid, block, 0, stream, L);
      else if (L.ld <= kWG * 8)
        hipLaunchKernelGGL((ln_block_kernel<T, 1, 8, MODE>), bgrid, block, 0, stream, L);
      else if (L.ld <= kWG * 16)
        hipLaunchKernelGGL((ln_block_kernel<T, 1, 16, MODE>), bgrid, block, 0, stream, L);
      else
        hipLaunchKernelGGL((ln_block_kernel<T, 1, 32, MODE>), bgrid, block, 0, stream, L);
      FWDMI_HIP_CHECK(hipGetLastError());
      return FWDMI_OK;
    }
  }
  if constexpr (!is_emb(MODE)) {
    const int block_chunks = (L.ld + kWG * kVec - 1) / (kWG * kVec);
    if ((sliceable && block_chunks > 8) || (!sliceable && L.ld > kWG * 32)) {
      // longer than a workgroup's registers hold: two passes, the second from cache
      const dim3 bgrid((unsigned)std::max<int64_t>(1, std::min(L.rows, (int64_t)cus * 8)));
      if (sliceable)
        hipLaunchKernelGGL((ln_stream_kernel<T, kVec, MODE>), bgrid, block, 0, stream, L);
      else
        hipLaunchKernelGGL((ln_stream_kernel<T, 1, MODE>), bgrid, block, 0, stream, L);
      FWDMI_HIP_CHECK(hipGetLastError());
      return FWDMI_OK;
    }
  }
  // Rows that cannot be cut into 16-byte slices (odd length or unaligned operands) are still read
  // once, one element per lane per slice: a wavefront per row up to 512 elements (here, embedding
  // rows included), a workgroup per row up to 8192 (above).
  if constexpr (MODE != kEmbSkip) {
    if (!sliceable && L.ld <= 64 * 8) {
      const int nv1 = L.ld <= 64 ? 1 : L.ld <= 128 ? 2 : L.ld <= 256 ? 4 : 8;
      if (nv1 == 1)
        hipLaunchKernelGGL((ln_rows_kernel<T, 1, 1, MODE, false>), grid, block, 0, stream, L);
      else if (nv1 == 2)
        hipLaunchKernelGGL((ln_rows_kernel<T, 1, 2, MODE, false>), grid, block, 0, stream, L);
      else if (nv1 == 4)
        hipLaunchKernelGGL((ln_rows_kernel<T, 1, 4, MODE, false>), grid, block, 0, stream, L);
      else
        hipLaunchKernelGGL((ln_rows_kernel<T, 1, 8, MODE, false>), grid, block, 0, stream, L);
      FWDMI_HIP_CHECK(hipGetLastError());
      return FWDMI_OK;
    }
  }
  if (sliceable && chunks <= 8) {
    const int nv = chunks <= 1 ? 1 : chunks <= 2 ? 2 : chunks <= 4 ? 4 : 8;
    const bool full = L.ld == 64 * kVec * nv;
#define FWDMI_LN_LAUNCH(NV_)                                                                           \
  if (full)                                                                                            \
    hipLaunchKernelGGL((ln_rows_kernel<T, kVec, NV_, MODE, true>), grid, block, 0, stream, L);         \
  else                                                                                                 \
    hipLaunchKernelGGL((ln_rows_kernel<T, kVec, NV_, MODE, false>), grid, block, 0, stream, L)
    if (nv == 1) {
      FWDMI_LN_LAUNCH(1);
    } else if (nv == 2) {
      FWDMI_LN_LAUNCH(2);
    } else if (nv == 4) {
      FWDMI_LN_LAUNCH(4);
    } else {
      FWDMI_LN_LAUNCH(8);
    }
#undef FWDMI_LN_LAUNCH
  } else if constexpr (MODE == kEmbSkip) {
    return set_error(FWDMI_ERR_UNSUPPORTED, "fused emb+skip layer norm needs 16-byte sliceable rows");
  } else {
    hipLaunchKernelGGL((ln_strided_kernel<T, MODE>), grid, block, 0, stream, L);
  }
  FWDMI_HIP_CHECK(hipGetLastError());
  return FWDMI_OK;
}

// True when rows of `ld` elements of `dtype` take the wavefront-per-row kernel in every mode, so
// that the fused embedding + skip form rounds exactly like its two separate launches.  (Rows of
// at most 512 bytes take the several-rows-per-wavefront kernel when launched separately; their
// fused form is issued as those two launches.)
bool rows_kernel_ok(int ld, int dtype, bool vec_ok) {
  const int vec = 16 / (int)dtype_size(dtype);
  return vec_ok && ld % vec == 0 && ld / vec > 32 && (ld + 64 * vec - 1) / (64 * vec) <= 8;
}

template <int MODE>
int ln_dispatch(LnLaunch& L, int dtype, bool vec_ok, hipStream_t stream) {
  if (dtype == FWDMI_F16) return ln_launch<_Float16, MODE>(L, vec_ok, stream);
  if (dtype == FWDMI_F32) return ln_launch<float, MODE>(L, vec_ok, stream);
  return set_error(FWDMI_ERR_UNSUPPORTED, "layer norm: unsupported dtype %d", dtype);
}

}  // namespace
}  // namespace fwdmi

extern "C" {

int fwdmi_skip_layer_norm(void* stream, int32_t ld, int64_t n, const void* input, const void* skip,
                          const float* beta, const float* gamma, void* output, const float* bias,
                          int32_t dtype, float eps) {
  using namespace fwdmi;
  clear_error();
  if (!is_float_dtype(dtype)) return set_error(FWDMI_ERR_UNSUPPORTED, "layer norm: unsupported dtype %d", dtype);
  FWDMI_REQUIRE(ld > 0 && n >= 0 && n % ld == 0, "layer norm: n=%lld is not a multiple of ld=%d",
                (long long)n, ld);
  if (n == 0) return FWDMI_OK;
  FWDMI_REQUIRE(input && output && beta && gamma, "layer norm: null pointer");
  LnLaunch L{};
  L.one = 1.0f;
  L.input = input;
  L.skip = skip;
  L.gamma = gamma;
  L.beta = beta;
  L.bias = bias;
  L.output = output;
  L.rows = n / ld;
  L.ld = ld;
  L.eps = eps;
  const bool vec_ok = aligned16(input) && aligned16(output) && aligned16(gamma) && aligned16(beta) &&
                      (!bias || aligned16(bias)) && (!skip || aligned16(skip));
  hipStream_t s = static_cast<hipStream_t>(stream);
  return skip ? ln_dispatch<kSkip>(L, dtype, vec_ok, s) : ln_dispatch<kLayerNorm>(L, dtype, vec_ok, s);
}

int fwdmi_layer_norm(void* stream, int32_t ld, int64_t n, const void* input, const float* beta,
                     const float* gamma, void* output, const float* bias, int32_t dtype, float eps) {
  return fwdmi_skip_layer_norm(stream, ld, n, input, nullptr, beta, gamma, output, bias, dtype, eps);
}

int fwdmi_emb_layer_norm_ex(void* stream, int32_t S, int32_t B, int32_t ld, const int32_t* input_ids,
                            const int32_t* segment_ids, const int32_t* input_mask, const float* beta,
                            const float* gamma, const void* word, const void* pos, const void* tok,
                            int32_t word_count, int32_t pos_count, int32_t tok_count, void* output,
                            int32_t* mask_idx, int32_t dtype, float eps, int32_t* oob_flag,
                            const fwdmi_emb_ext* ext) {
  using namespace fwdmi;
  clear_error();
  if (!is_float_dtype(dtype)) return set_error(FWDMI_ERR_UNSUPPORTED, "emb layer norm: unsupported dtype %d", dtype);
  FWDMI_REQUIRE(S >= 0 && B >= 0 && ld > 0, "emb layer norm: S=%d B=%d ld=%d", S, B, ld);
  if ((int64_t)S * B == 0) return FWDMI_OK;
  FWDMI_REQUIRE(input_ids && segment_ids && beta && gamma && word && pos && tok && output,
                "emb layer norm: null pointer");
  FWDMI_REQUIRE(word_count > 0 && pos_count > 0 && tok_count > 0, "emb layer norm: empty table");
  FWDMI_REQUIRE(!mask_idx || input_mask, "emb layer norm: mask_idx requested without input_mask");
  const bool fused = ext && ext->skip;
  FWDMI_REQUIRE(!fused || (ext->gamma2 && ext->beta2), "emb layer norm: fused stage needs gamma2 and beta2");
  LnLaunch L{};
  L.one = 1.0f;
  L.input = word;
  L.pos = pos;
  L.tok = tok;
  L.gamma = gamma;
  L.beta = beta;
  L.output = output;
  L.input_ids = input_ids;
  L.segment_ids = segment_ids;
  L.input_mask = input_mask;
  L.mask_idx = mask_idx;
  L.oob_flag = oob_flag;
  L.rows = (int64_t)S * B;
  L.ld = ld;
  L.S = S;
  L.B = B;
  L.word_count = word_count;
  L.pos_count = pos_count;
  L.tok_count = tok_count;
  L.eps = eps;
  L.batch_major = ext && ext->batch_major;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool tables_ok = aligned16(word) && aligned16(pos) && aligned16(tok) && aligned16(gamma) && aligned16(beta);
  bool vec_ok = tables_ok && aligned16(output);
  if (!fused) return ln_dispatch<kEmb>(L, dtype, vec_ok, s);

  vec_ok = vec_ok && aligned16(ext->skip) && aligned16(ext->gamma2) && aligned16(ext->beta2) &&
           (!ext->bias2 || aligned16(ext->bias2)) && (!ext->emb_output || aligned16(ext->emb_output));
  if (rows_kernel_ok(ld, dtype, vec_ok)) {
    L.skip = ext->skip;
    L.gamma2 = ext->gamma2;
    L.beta2 = ext->beta2;
    L.bias2 = ext->bias2;
    L.eps2 = ext->eps2;
    L.emb_output = ext->emb_output;
    return ln_dispatch<kEmbSkip>(L, dtype, vec_ok, s);
  }
  // every other row shape: the two launches themselves, the second in place over the first result
  void* first = ext->emb_output ? ext->emb_output : output;
  L.output = first;
  int rc = ln_dispatch<kEmb>(L, dtype, tables_ok && aligned16(first), s);
  if (rc != FWDMI_OK) return rc;
  return fwdmi_skip_layer_norm(stream, ld, (int64_t)S * B * ld, first, ext->skip, ext->beta2, ext->gamma2, output,
                               ext->bias2, dtype, ext->eps2);
}

int fwdmi_emb_layer_norm(void* stream, int32_t S, int32_t B, int32_t ld, const int32_t* input_ids,
                         const int32_t* segment_ids, const int32_t* input_mask, const float* beta,
                         const float* gamma, const void* word, const void* pos, const void* tok,
                         int32_t word_count, int32_t pos_count, int32_t tok_count, void* output,
                         int32_t* mask_idx, int32_t dtype, float eps, int32_t* oob_flag) {
  return fwdmi_emb_layer_norm_ex(stream, S, B, ld, input_ids, segment_ids, input_mask, beta, gamma, word, pos, tok,
                                 word_count, pos_count, tok_count, output, mask_idx, dtype, eps, oob_flag, nullptr);
}

}  // extern "C"
