// Bag reduction (sum / mean / max / square-sum, optional per-sample weights), fixed-length
// bags and plain row gather for gfx950.
//
// Work decomposition
//   * A table row is read with 128-bit loads: a row of `dim` elements needs dim*sizeof(T)/16
//     lanes.  G = that number rounded up to a power of two (at most 64) lanes form a
//     sub-wavefront "slot"; a 256-lane workgroup holds 256/G slots, each reducing one bag at
//     a time with fp32 accumulators in registers.  Rows wider than 1 KiB are cut into column
//     slices of 64 lanes and a (bag, slice) pair becomes the unit of work.
//   * A workgroup owns a contiguous run of bags.  Their offsets, and the ids (and weights)
//     they cover, are copied into LDS once with coalesced loads; slots then read ids from
//     LDS as broadcasts, so the only per-row global traffic is the row itself.  For tables of
//     at most 2^24 rows and 4 GiB the copy turns each id (int32 or int64) into a 32-bit row
//     number, so the 64-bit part of the range check happens once per id.
//   * The run's bags are ranked by length in LDS and handed out longest first from an LDS
//     counter: the slots of a wavefront, which execute in lock-step, get bags of nearly equal
//     length, and the long tail of bag lengths is evened out inside a workgroup.
//   * Rows of one bag are added strictly in bag order (eight loads in flight, consumed in
//     order), so fp32 results do not depend on the launch shape.
//   * A multi-table launch can give each of the eight XCDs (one L2 each) its own contiguous
//     part of the table-major work list, cut at equal estimated cost.
//
// Memory safety: offsets are clamped to [0, input_size] and made non-decreasing before use,
// ids outside [data_offset, data_offset+count) never form an address (a table of no rows forms
// none at all), so arbitrary id / offset bytes cannot make the kernel read or write out of bounds.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <cmath>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "../common.h"
#include "bag_plan.h"
#include "device_util.h"

namespace fwdmi {
namespace {

#ifndef FWDMI_BAG_UNROLL
#define FWDMI_BAG_UNROLL 8
#endif
#ifndef FWDMI_BAG_WAVES_PER_EU
#define FWDMI_BAG_WAVES_PER_EU 6  // register budget of 80 VGPRs: measured best on the 26-table configuration
#endif
// argmax tracking and the second accumulator carry more live registers: they keep the looser budget;
// the weighted form sits in between (measured on the 26-table configuration: 4 -> 5 wavefronts 2 % faster)
#define FWDMI_BAG_OCCUPANCY \
  __attribute__((amdgpu_waves_per_eu((KIND == kMax || KIND == kSumSq) ? 4 : KIND == kWeighted ? 5 : FWDMI_BAG_WAVES_PER_EU)))
constexpr int kUnroll = FWDMI_BAG_UNROLL;  // row loads in flight per lane

// Hands elements first[0 .. n) to put(i, value), the workgroup's lanes sharing the work.  Long
// ranges come in with 16-byte loads (a load instruction occupies the CU's memory pipeline for the
// same time whatever its width); the elements before the first 16-byte boundary and behind the
// last one go one by one, so nothing outside the range is read.  `first` is aligned to its type.
// All loads of a lane's share (up to four vectors, the two ends) are issued before the first of
// them is used: the workgroup waits for memory once, not once per vector and once per end (a run of
// 1830 ids is two vectors for most lanes, and most runs start and end off a 16-byte boundary).
// The vectors are loaded with the non-temporal hint: ids and weights are read once, and 111 MB of
// them per launch of the 26-table configuration otherwise displace table rows in L2 (0.4229 -> 0.4220 ms).
template <typename T, typename Put>
__device__ __forceinline__ void stream_in(const T FWDMI_GLOBAL* first, int n, int tid, int lanes, Put put) {
  constexpr int kPer = 16 / (int)sizeof(T);
  constexpr int kAhead = 4;  // vectors a lane has in flight
  if (n < 2 * lanes) {  // uniform over the workgroup: too short for the split to pay; two elements per lane at most
    const int i0 = tid, i1 = tid + lanes;
    T a{}, b{};
    if (i0 < n) a = first[i0];
    if (i1 < n) b = first[i1];
    if (i0 < n) put(i0, a);
    if (i1 < n) put(i1, b);
    return;
  }
  const int misalign = (int)((reinterpret_cast<uintptr_t>(first) & 15) / sizeof(T));
  const int head = (kPer - misalign) & (kPer - 1);
  const int n_vec = (n - head) / kPer;
  const int body_end = head + n_vec * kPer;
  const bool has_head = tid < head, has_tail = body_end + tid < n;
  T at_head{}, at_tail{};
  if (has_head) at_head = first[tid];
  if (has_tail) at_tail = first[body_end + tid];
  for (int v0 = tid; v0 < n_vec; v0 += kAhead * lanes) {
    Pack<T, kPer> p[kAhead];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
      const int v = v0 + k * lanes;
      if (v < n_vec) p[k] = gload_stream<T, kPer>(first + head + v * kPer);
    }
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
      const int v = v0 + k * lanes;
      if (v < n_vec) {
#pragma unroll
        for (int e = 0; e < kPer; ++e) put(head + v * kPer + e, p[k].v[e]);
      }
    }
  }
  if (has_head) put(tid, at_head);
  if (has_tail) put(body_end + tid, at_tail);
}

// EXT: the launch may use what only some multi-table launches need (runs sized per table, descriptors
// among the kernel arguments).  Launches without either run the variant that does not carry that code:
// its presence alone cost 1.2 % on 26 single-table launches of 65536 bags and 0.1 us on a 4096-bag launch.
template <typename TW, typename TI, int VEC, int KIND, bool EXT>
__global__ __launch_bounds__(kWG) FWDMI_BAG_OCCUPANCY void bag_reduce_kernel(const BagLaunch L) {
  // LDS carve-up (dynamic, sized by the host): offsets | ids | weights | lengths | order
  extern __shared__ __attribute__((aligned(16))) unsigned char s_raw[];
  int64_t* const s_off = reinterpret_cast<int64_t*>(s_raw);
  TI* const s_idx = reinterpret_cast<TI*>(s_off + (L.bags_per_wg + 2));
  float* const s_w = reinterpret_cast<float*>(reinterpret_cast<uint32_t*>(s_idx) + L.idx_cap);
  int* const s_len = reinterpret_cast<int*>(s_w + (KIND == kWeighted ? L.idx_cap : 0));
  uint16_t* const s_order = reinterpret_cast<uint16_t*>(s_len + L.bags_per_wg);
  __shared__ int s_next;
  __shared__ int s_hist[kLenBuckets];
  const int wg_lanes = blockDim.x;

  const int tid = threadIdx.x;
  // table, run of the table, bags of a run of this table, quarter of the run (-1: the whole run):
  // uniform over the workgroup
  BagWork W;
  if (!bag_decode<EXT>(L, blockIdx.x, &W)) return;
  const int t = W.table;
  fwdmi_bag_table T;
  if (L.tables) {
    const fwdmi_bag_table FWDMI_GLOBAL* tp = gconst<fwdmi_bag_table>(L.tables) + t;
    T.data = tp->data;
    T.input = tp->input;
    T.input_2 = tp->input_2;
    T.count = tp->count;
    T.input_size = tp->input_size;
    T.data_offset = tp->data_offset;
    T.out_col = tp->out_col;
    T.weights = tp->weights;
  } else {
    T = L.inline_tables[EXT ? t : 0];  // without EXT the one table of a single-table launch
  }

  const int G = 1 << L.log2_g;
  const int slot = tid >> L.log2_g;
  const int gl = tid & (G - 1);
  const int slots = wg_lanes >> L.log2_g;

  int64_t bag0;
  int nb;
  bag_run_range(L, W, &bag0, &nb);
  if (nb <= 0) return;  // a quarter beyond the table's last bag (uniform over the workgroup)
  const TI FWDMI_GLOBAL* __restrict__ ids = gconst<TI>(T.input);
  // per-sample weights: the launch's (single table) or the table's own; none = weight 1
  const TW FWDMI_GLOBAL* __restrict__ psw = gconst<TW>(L.multi ? T.weights : L.psw);
  const bool has_w = KIND == kWeighted && (L.multi ? T.weights : L.psw) != nullptr;  // uniform

  // ---- stage the run's offsets (clamped) ------------------------------------------------
  for (int i = tid; i <= nb; i += wg_lanes) {
    int64_t v;
    if (L.fixed_len >= 0) {
      v = (bag0 + i) * L.fixed_len;
    } else {
      const int64_t b = bag0 + i;
      v = (b < L.n_bags || L.include_last) ? (int64_t)gconst<TI>(T.input_2)[b] : T.input_size;
    }
    s_off[i] = min(max(v, (int64_t)0), T.input_size);
  }
  if (tid == 0) s_next = slots;
  for (int i = tid; i < kLenBuckets; i += wg_lanes) s_hist[i] = 0;
  __syncthreads();

  // A table without rows (count <= 0; its data pointer may be null): every id is outside it, so
  // the run's bags are zeros and no row address is ever formed.  Uniform over the workgroup.
  if (T.count <= 0) {
    bool any = false;
    const int64_t n_el = (int64_t)nb * L.dim;
    for (int64_t i = tid; i < n_el; i += wg_lanes) {
      const int lb = (int)(i / L.dim);
      const int c = (int)(i - (int64_t)lb * L.dim);
      any |= s_off[lb + 1] > s_off[lb];
      const int64_t o = (bag0 + lb) * L.out_stride + T.out_col + c;
      if (L.out_f16) {
        gmut<_Float16>(L.out)[o] = (_Float16)0.0f;
        if (KIND == kSumSq) gmut<_Float16>(L.out2)[o] = (_Float16)0.0f;
      } else {
        gmut<float>(L.out)[o] = 0.0f;
        if (KIND == kSumSq) gmut<float>(L.out2)[o] = 0.0f;
      }
      if (KIND == kMax && L.max_indices) gmut<TI>(L.max_indices)[(bag0 + lb) * (int64_t)L.dim + c] = 0;
    }
    if (any && L.oob_flag) atomicOr(L.oob_flag, 1);
    return;
  }

  // A "compact" table has at most 2^24 rows and 4 GiB: a row number fits 32 bits (whatever the
  // id type) and a row's byte offset is one 24-bit multiply-add on top of a uniform base.
  // Uniform over the workgroup.
  const uint32_t row_bytes = (uint32_t)L.dim * (uint32_t)sizeof(TW);
  const bool compact = T.count <= (1 << 24) && row_bytes < (1u << 24) &&
                       (uint64_t)T.count * row_bytes <= ((uint64_t)1 << 32);
  const uint32_t last32 = (uint32_t)(T.count - 1);
  uint32_t* const s_row = reinterpret_cast<uint32_t*>(s_idx);  // the id window, compact tables

  // ---- stage the ids (and weights) the run covers ----------------------------------------
  // For a compact table the window holds row numbers (id - data_offset; 0xFFFFFFFF for an id
  // outside the table): the 64-bit part of the range check is done once per id here, not once
  // per lane that reads the row.
  const int64_t span0 = s_off[0];
  const int64_t span = s_off[nb] - span0;
  // the window holds 32-bit row numbers of a compact table, ids of the launch's type otherwise
  const int window = compact ? L.idx_cap : L.idx_cap / (int)(sizeof(TI) / 4);
  const bool staged = span >= 0 && span <= window;  // uniform over the workgroup
  if (staged) {
    auto put = [&](int i, TI id) {
      if (compact) {
        const uint64_t row = (uint64_t)((int64_t)id - T.data_offset);
        s_row[i] = row < (uint64_t)T.count ? (uint32_t)row : 0xFFFFFFFFu;
      } else {
        s_idx[i] = id;
      }
    };
    stream_in<TI>(ids + span0, (int)span, tid, wg_lanes, put);
    if (KIND == kWeighted) {
      if (has_w) {
        stream_in<TW>(psw + span0, (int)span, tid, wg_lanes, [&](int i, TW w) { s_w[i] = (float)w; });
      } else {
        for (int i = tid; i < span; i += wg_lanes) s_w[i] = 1.0f;
      }
    }
  }
  // ---- order the run's bags by length, longest first --------------------------------------
  // The slots of one wavefront execute in lock-step, so a wavefront pays for the longest of
  // the bags its slots hold.  Handing out bags in length order gives the slots of a wavefront
  // bags of (nearly) equal length, and starting with the longest evens out the finish.
  // The order changes which slot reduces a bag, never the result.
  const bool sorted = L.fixed_len < 0 && nb > slots;  // with a bag per slot at most there is nothing to order
  if (sorted) {
    // Counting sort on min(length, 255), descending: histogram with LDS atomics, exclusive scan
    // of the 256 buckets by the first wavefront, scatter.  (Order inside a bucket is arbitrary.)
    for (int i = tid; i < nb; i += wg_lanes) {
      const int len = (int)min(max(s_off[i + 1] - s_off[i], (int64_t)0), (int64_t)(kLenBuckets - 1));
      const int bucket = kLenBuckets - 1 - len;
      s_len[i] = (bucket << 16) | atomicAdd(&s_hist[bucket], 1);
    }
    __syncthreads();
    if (tid < 64) {
      constexpr int kPer = kLenBuckets / 64;
      int c[kPer], sum = 0;
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        c[j] = s_hist[tid * kPer + j];
        sum += c[j];
      }
      int incl = sum;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (tid >= d) incl += up;
      }
      int run = incl - sum;
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        s_hist[tid * kPer + j] = run;
        run += c[j];
      }
    }
    __syncthreads();
    for (int i = tid; i < nb; i += wg_lanes) {
      const int packed = s_len[i];
      s_order[s_hist[packed >> 16] + (packed & 0xffff)] = (uint16_t)i;
    }
  }
  __syncthreads();

  const TW FWDMI_GLOBAL* __restrict__ tab = gconst<TW>(T.data);
  const int n_units = nb * L.n_slices;
  const char FWDMI_GLOBAL* const tab_bytes = gconst<char>(T.data);
  bool oob = false;
  const float one = L.one;

  int unit = slot;
  while (unit < n_units) {
    const int ub = L.n_slices == 1 ? unit : unit / L.n_slices;
    const int sl = unit - ub * L.n_slices;
    const int lb = sorted ? (int)s_order[ub] : ub;
    const int64_t start = s_off[lb];
    const int64_t end = max(s_off[lb + 1], start);
    const int col = (sl * G + gl) * VEC;
    const bool col_ok = col < L.dim;
    const TW FWDMI_GLOBAL* __restrict__ tcol = tab + (col_ok ? col : 0);
    const uint32_t col_bytes = (uint32_t)(col_ok ? col : 0) * (uint32_t)sizeof(TW);
    // A run whose offsets decrease can make [start,end) leave the staged window.
    const bool in_lds = staged && start >= span0 && end <= span0 + span;

    float acc[VEC];
    float acc2[KIND == kSumSq ? VEC : 1];
    constexpr bool kIsMax = KIND == kMax || KIND == kMaxValue;
    TI arg[KIND == kMax ? VEC : 1];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
#pragma unroll
    for (int e = 0; e < (KIND == kSumSq ? VEC : 1); ++e) acc2[e] = 0.0f;
#pragma unroll
    for (int e = 0; e < (KIND == kMax ? VEC : 1); ++e) arg[e] = 0;
    bool first = true;

    // Loads UU rows starting at bag position i (all loads issued before the first use), then
    // folds them in bag order.  LDS selects where the ids come from.  COMPACT (implies LDS): the
    // window holds 32-bit row numbers of a table of at most 2^24 rows and 4 GiB, so a row's byte
    // offset is one 24-bit multiply-add on top of a uniform base.
    auto step = [&](auto uu_tag, auto lds_tag, auto compact_tag, auto pred_tag, int64_t i, int cnt) {
      constexpr int UU = decltype(uu_tag)::value;
      constexpr bool LDS = decltype(lds_tag)::value;
      constexpr bool COMPACT = decltype(compact_tag)::value;
      constexpr bool PRED = decltype(pred_tag)::value;  // only the first `cnt` of the UU rows exist
      Pack<TW, VEC> v[UU];
      TI id[UU];
      float w[UU];
      bool ok[UU];
      bool all_ok = true;
      uint32_t r32[COMPACT ? UU : 1];
      if (LDS) {
        // one LDS address per step; the unrolled reads use immediate offsets
        const uint32_t li = (uint32_t)(i - span0);
        const TI* const sp = s_idx + li;
        const uint32_t* const rp = s_row + li;
        const float* const wp = s_w + li;
#pragma unroll
        for (int u = 0; u < UU; ++u) {
          id[u] = 0;
          if (COMPACT) r32[u] = 0;
          w[u] = 0.0f;
          if (!PRED || u < cnt) {
            if (COMPACT)
              r32[u] = rp[u];
            else
              id[u] = sp[u];
            if (KIND == kWeighted) w[u] = wp[u];
          }
        }
      } else {
#pragma unroll
        for (int u = 0; u < UU; ++u) {
          id[u] = 0;
          w[u] = 0.0f;
          if (!PRED || u < cnt) {
            id[u] = ids[i + u];
            if (KIND == kWeighted) w[u] = has_w ? (float)psw[i + u] : 1.0f;
          }
        }
      }
      // a bad id never forms an address: a valid row is fetched instead and discarded below;
      // rows past `cnt` are not fetched at all and enter the fold as zeros
      if (COMPACT) {
        uint32_t worst = 0;
#pragma unroll
        for (int u = 0; u < UU; ++u) {
          const bool valid = !PRED || u < cnt;
          const uint32_t row = r32[u];  // 0 for a row past `cnt`
          worst = max(worst, row);
          const uint32_t off = __umul24(min(row, last32), row_bytes) + col_bytes;
          if (valid) {
            v[u] = gload<TW, VEC>(reinterpret_cast<const TW FWDMI_GLOBAL*>(tab_bytes + off));
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[u].v[e] = (TW)0.0f;
          }
          if (kIsMax) ok[u] = valid && row <= last32;
          if (KIND == kMax) id[u] = (TI)((int64_t)row + T.data_offset);  // argmax reports the id
        }
        all_ok = worst <= last32;
      } else {
#pragma unroll
        for (int u = 0; u < UU; ++u) {
          const bool valid = !PRED || u < cnt;
          const uint64_t row = (uint64_t)((int64_t)id[u] - T.data_offset);
          const bool in_range = row < (uint64_t)T.count;
          ok[u] = valid && in_range;
          if (valid) {
            v[u] = gload<TW, VEC>(tcol + (in_range ? row : 0) * (uint64_t)L.dim);
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[u].v[e] = (TW)0.0f;
          }
          all_ok &= in_range || !valid;
        }
      }
      if (__builtin_expect(!__all(all_ok), 0)) {
        oob |= !all_ok;
#pragma unroll
        for (int u = 0; u < UU; ++u) {
          if (COMPACT) ok[u] = (!PRED || u < cnt) && r32[u] <= last32;
          if (!ok[u]) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[u].v[e] = (TW)0.0f;
            w[u] = 0.0f;
          }
        }
      } else if (COMPACT && !kIsMax) {
#pragma unroll
        for (int u = 0; u < UU; ++u) ok[u] = true;
      }
#pragma unroll
      for (int u = 0; u < UU; ++u) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float x = (float)v[u].v[e];
          if (KIND == kPlain) {
            // fma(x, 1, acc) rounds exactly like acc + x and lets fp16 rows use the
            // mixed-precision FMA (conversion and add in one instruction); `one` arrives as a
            // kernel argument so the multiply is not folded away
            acc[e] = __builtin_fmaf(x, one, acc[e]);
          } else if (KIND == kSquare) {
            acc[e] = __builtin_fmaf(x, x, acc[e]);
          } else if (KIND == kSumSq) {
            acc[e] = __builtin_fmaf(x, one, acc[e]);
            acc2[KIND == kSumSq ? e : 0] = __builtin_fmaf(x, x, acc2[KIND == kSumSq ? e : 0]);
          } else if (KIND == kWeighted) {
            acc[e] = __builtin_fmaf(w[u], x, acc[e]);
          } else {
            if (ok[u] && (first || x > acc[e])) {
              acc[e] = x;
              if (KIND == kMax) arg[e] = id[u];
            }
          }
        }
        if (kIsMax && ok[u]) first = false;
      }
    };
    auto bag = [&](auto lds_tag, auto compact_tag) {
      int64_t i = start;
      for (; i + kUnroll <= end; i += kUnroll)
        step(std::integral_constant<int, kUnroll>{}, lds_tag, compact_tag, std::false_type{}, i, kUnroll);
      // the last 1..7 rows: one predicated step, so a wavefront issues as many loads as its
      // longest remainder needs and no more
      if (i < end)
        step(std::integral_constant<int, kUnroll - 1>{}, lds_tag, compact_tag, std::true_type{}, i, (int)(end - i));
    };
    // Half-precision maximum without conversions: the running maximum stays packed fp16 (max is
    // exact in any format) and one packed instruction handles two columns.  Where the packed
    // maximum could differ from the rule above -- a NaN or an infinity anywhere in the bag's
    // columns of this lane, a maximum of +-0 (the rule keeps the sign that came first), an id
    // outside the table -- the lane redoes the bag with the exact loop below; for ordinary data
    // that never happens.
    bool exact_needed = true;
    if constexpr (KIND == kMaxValue && std::is_same<TW, _Float16>::value && VEC == 8) {
      if (in_lds && compact) {  // uniform over the workgroup, apart from ragged bags
        typedef _Float16 Half2 __attribute__((ext_vector_type(2)));
        const Half2 kNegInf = {-__builtin_inff16(), -__builtin_inff16()};
        const Half2 kZero = {(_Float16)0.0f, (_Float16)0.0f};
        Half2 m[4] = {kNegInf, kNegInf, kNegInf, kNegInf};
        Half2 poison[4] = {kZero, kZero, kZero, kZero};  // turns NaN once a NaN or an infinity went by
        bool bad_id = false;
        auto fast_step = [&](auto uu_tag, auto pred_tag, int i, int cnt) {
          constexpr int UU = decltype(uu_tag)::value;
          constexpr bool PRED = decltype(pred_tag)::value;
          Pack<TW, VEC> v[UU];
          uint32_t worst = 0;
#pragma unroll
          for (int u = 0; u < UU; ++u) {
            const bool valid = !PRED || u < cnt;
            const uint32_t row = valid ? s_row[i + u] : 0u;
            worst = max(worst, row);
            const uint32_t off = __umul24(min(row, last32), row_bytes) + col_bytes;
            if (valid) {
              v[u] = gload<TW, VEC>(reinterpret_cast<const TW FWDMI_GLOBAL*>(tab_bytes + off));
            } else {
#pragma unroll
              for (int e = 0; e < VEC; ++e) v[u].v[e] = -__builtin_inff16();
            }
          }
          bad_id |= worst > last32;
#pragma unroll
          for (int u = 0; u < UU; ++u) {
            Half2 x[4];
            __builtin_memcpy(x, &v[u], sizeof(x));
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              // the instruction itself: the generic maximum would first quiet signalling NaNs
              // of both operands, and NaN is what `poison` already sends to the exact loop
              asm("v_pk_max_f16 %0, %1, %2" : "=v"(m[k]) : "v"(m[k]), "v"(x[k]));
              if (!PRED || u < cnt) poison[k] = x[k] * kZero + poison[k];
            }
          }
        };
        int i = (int)(start - span0);
        const int stop = (int)(end - span0);
        for (; i + kUnroll <= stop; i += kUnroll)
          fast_step(std::integral_constant<int, kUnroll>{}, std::false_type{}, i, kUnroll);
        if (i < stop) fast_step(std::integral_constant<int, kUnroll - 1>{}, std::true_type{}, i, stop - i);
        bool doubt = bad_id;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          uint32_t mb, pb;
          __builtin_memcpy(&mb, &m[k], 4);
          __builtin_memcpy(&pb, &poison[k], 4);
          doubt |= (mb & 0x7fffu) == 0 || (mb & 0x7fff0000u) == 0;          // a maximum of +-0
          doubt |= (pb & 0x7fffu) > 0x7c00u || (pb & 0x7fff0000u) > 0x7c000000u;  // NaN / infinity seen
        }
        if (end == start) doubt = false;  // an empty bag is zeros, set below
        exact_needed = doubt;
        if (!doubt) {
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            acc[2 * k] = end > start ? (float)m[k].x : 0.0f;
            acc[2 * k + 1] = end > start ? (float)m[k].y : 0.0f;
          }
        }
      }
    }
    if constexpr (KIND == kMaxValue && std::is_same<TW, float>::value && VEC == 4) {
      // the same idea for fp32 rows: one v_max_f32 and one poison update per column
      if (in_lds && compact) {
        float m[4], poison[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          m[k] = -__builtin_inff();
          poison[k] = 0.0f;
        }
        bool bad_id = false;
        const float zero = one - one;  // a run-time zero: x * zero must stay a multiplication
        auto fast_step = [&](auto uu_tag, auto pred_tag, int i, int cnt) {
          constexpr int UU = decltype(uu_tag)::value;
          constexpr bool PRED = decltype(pred_tag)::value;
          Pack<TW, VEC> v[UU];
          uint32_t worst = 0;
#pragma unroll
          for (int u = 0; u < UU; ++u) {
            const bool valid = !PRED || u < cnt;
            const uint32_t row = valid ? s_row[i + u] : 0u;
            worst = max(worst, row);
            const uint32_t off = __umul24(min(row, last32), row_bytes) + col_bytes;
            if (valid) {
              v[u] = gload<TW, VEC>(reinterpret_cast<const TW FWDMI_GLOBAL*>(tab_bytes + off));
            } else {
#pragma unroll
              for (int e = 0; e < VEC; ++e) v[u].v[e] = -__builtin_inff();
            }
          }
          bad_id |= worst > last32;
#pragma unroll
          for (int u = 0; u < UU; ++u) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              asm("v_max_f32 %0, %1, %2" : "=v"(m[k]) : "v"(m[k]), "v"(v[u].v[k]));
              if (!PRED || u < cnt) poison[k] = __builtin_fmaf(v[u].v[k], zero, poison[k]);
            }
          }
        };
        int i = (int)(start - span0);
        const int stop = (int)(end - span0);
        for (; i + kUnroll <= stop; i += kUnroll)
          fast_step(std::integral_constant<int, kUnroll>{}, std::false_type{}, i, kUnroll);
        if (i < stop) fast_step(std::integral_constant<int, kUnroll - 1>{}, std::true_type{}, i, stop - i);
        bool doubt = bad_id;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          doubt |= (__float_as_uint(m[k]) & 0x7fffffffu) == 0;             // a maximum of +-0
          doubt |= (__float_as_uint(poison[k]) & 0x7fffffffu) > 0x7f800000u;  // NaN / infinity seen
        }
        if (end == start) doubt = false;
        exact_needed = doubt;
        if (!doubt) {
#pragma unroll
          for (int k = 0; k < 4; ++k) acc[k] = end > start ? m[k] : 0.0f;
        }
      }
    }
    if (exact_needed) {
      if (in_lds) {
        if (compact)
          bag(std::true_type{}, std::true_type{});
        else
          bag(std::true_type{}, std::false_type{});
      } else {
        bag(std::false_type{}, std::false_type{});
      }
    }

    // ---- epilogue: mean scaling, store ---------------------------------------------------
    const int64_t len = end - start;
    if (L.op == FWDMI_OP_MEAN && len > 0) {
      const float flen = (float)len;
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = acc[e] / flen;
    }
    if (col_ok) {
      const int64_t o = (bag0 + lb) * L.out_stride + T.out_col + col;
      if (L.out_f16) {
        _Float16 FWDMI_GLOBAL* op = gmut<_Float16>(L.out) + o;
        if (L.vec_store) {
          Pack<_Float16, VEC> r;
#pragma unroll
          for (int e = 0; e < VEC; ++e) r.v[e] = (_Float16)acc[e];
          if (VEC > 1 && L.vec_store == 2) {
            if constexpr (VEC > 1) gstore_stream<_Float16, VEC>(op, r);
          } else {
            gstore<_Float16, VEC>(op, r);
          }
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) op[e] = (_Float16)acc[e];
        }
      } else {
        float FWDMI_GLOBAL* op = gmut<float>(L.out) + o;
        if (L.vec_store) {
          Pack<float, VEC> r;
#pragma unroll
          for (int e = 0; e < VEC; ++e) r.v[e] = acc[e];
          if (VEC == 8 && L.vec_store == 3) {
            // Eight fp32 results per lane are 32 bytes: stored as they lie, each of the two 16-byte
            // store instructions would write every other 16 bytes of the slot's G * 32.  The lanes
            // trade halves first (lane g takes what lane g/2, then lane G/2 + g/2, holds), so that
            // each instruction writes one contiguous half.  Every lane of the slot is here: the
            // plan asks for this form only when all column slices are full.
            if constexpr (VEC == 8) {
              const int lane = threadIdx.x & 63;
              const int from0 = ((lane & ~(G - 1)) + (gl >> 1)) << 2, from1 = from0 + (G << 1);
              const bool upper = gl & 1;
              Pack<float, 4> h0, h1;
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                const int lo = __float_as_int(r.v[k]), hi = __float_as_int(r.v[4 + k]);
                const int lo0 = __builtin_amdgcn_ds_bpermute(from0, lo), hi0 = __builtin_amdgcn_ds_bpermute(from0, hi);
                const int lo1 = __builtin_amdgcn_ds_bpermute(from1, lo), hi1 = __builtin_amdgcn_ds_bpermute(from1, hi);
                h0.v[k] = __int_as_float(upper ? hi0 : lo0);
                h1.v[k] = __int_as_float(upper ? hi1 : lo1);
              }
              float FWDMI_GLOBAL* const slice = op - gl * VEC;  // the slot's first column of this slice
              gstore_stream<float, 4>(slice + gl * 4, h0);
              gstore_stream<float, 4>(slice + G * 4 + gl * 4, h1);
            }
          } else if (VEC > 1 && L.vec_store == 2) {
            if constexpr (VEC > 1) gstore_stream<float, VEC>(op, r);
          } else {
            gstore<float, VEC>(op, r);
          }
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) op[e] = acc[e];
        }
      }
      if (KIND == kSumSq) {  // second output, same place in its own matrix
        if (L.out_f16) {
          _Float16 FWDMI_GLOBAL* op = gmut<_Float16>(L.out2) + o;
          if (L.vec_store) {
            Pack<_Float16, VEC> r;
#pragma unroll
            for (int e = 0; e < VEC; ++e) r.v[e] = (_Float16)acc2[KIND == kSumSq ? e : 0];
            gstore<_Float16, VEC>(op, r);
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) op[e] = (_Float16)acc2[KIND == kSumSq ? e : 0];
          }
        } else {
          float FWDMI_GLOBAL* op = gmut<float>(L.out2) + o;
          if (L.vec_store) {
            Pack<float, VEC> r;
#pragma unroll
            for (int e = 0; e < VEC; ++e) r.v[e] = acc2[KIND == kSumSq ? e : 0];
            gstore<float, VEC>(op, r);
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) op[e] = acc2[KIND == kSumSq ? e : 0];
          }
        }
      }
      if (KIND == kMax && L.max_indices) {
        TI FWDMI_GLOBAL* mp = gmut<TI>(L.max_indices) + (bag0 + lb) * (int64_t)L.dim + col;
#pragma unroll
        for (int e = 0; e < VEC; ++e) mp[e] = arg[e];
      }
    }

    // ---- next unit of the run ------------------------------------------------------------
    int nxt = 0;
    if (gl == 0) nxt = atomicAdd(&s_next, 1);
    unit = __shfl(nxt, 0, G);
  }

  if (oob && L.oob_flag) atomicOr(L.oob_flag, 1);
}

// Descriptors of a multi-table batch travel to device memory as kernel arguments: no staging
// buffer on the host, no copy engine, ordered on the stream like any launch.
constexpr int kFillChunk = 56;  // 56 x 64 bytes of descriptors per launch, inside the 4 KiB argument limit
struct TableChunk {
  fwdmi_bag_table t[kFillChunk];
};

__global__ __launch_bounds__(64) void bag_tables_fill_kernel(const TableChunk c, int n,
                                                                     fwdmi_bag_table* dst) {
  const int i = threadIdx.x;
  if (i < n) dst[i] = c.t[i];
}

// ---- scratch of the entry point that allocates nothing ---------------------------------------
// The multi-table kernel reads its table descriptors from device memory.  Callers that cannot
// allocate (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc) get
// that memory from this array, which the loaded code object carries: every GPU the library runs
// on holds its own copy, at its own address, until the process ends.
constexpr int kNoAllocMaxTables = 1024;  // 64 KiB of descriptors
static __device__ __align__(256) unsigned char scratch[kNoAllocMaxTables * sizeof(fwdmi_bag_table)];

// In host code `scratch` is only a handle for the runtime, not a device address: the address on
// the current device comes from hipGetSymbolAddress, once per device, and is kept here.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
std::mutex g_noalloc_issue_mu;  // held while a call enqueues its descriptor writes and its launch
void* g_scratch_ptr[kMaxDevices] = {};

int scratch_on_current_device(fwdmi_bag_table** out) {
  int dev = -1;
  FWDMI_HIP_CHECK(hipGetDevice(&dev));
  FWDMI_REQUIRE(dev >= 0 && dev < kMaxDevices, "no-allocation entry point: device index %d beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    FWDMI_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    FWDMI_REQUIRE(p != nullptr, "no-allocation entry point: the scratch array has no address on device %d", dev);
    g_scratch_ptr[dev] = p;
  }
  *out = static_cast<fwdmi_bag_table*>(g_scratch_ptr[dev]);
  return FWDMI_OK;
}

template <typename TW, typename TI, int VEC, bool EXT>
int launch_kind_ext(const BagPlan& P, hipStream_t stream) {
  const dim3 grid(P.grid), block(P.block);
  const BagLaunch& L = P.L;
  switch (P.kind) {
    case kPlain:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kPlain, EXT>), grid, block, P.lds, stream, L);
      break;
    case kSquare:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kSquare, EXT>), grid, block, P.lds, stream, L);
      break;
    case kSumSq:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kSumSq, EXT>), grid, block, P.lds, stream, L);
      break;
    case kWeighted:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kWeighted, EXT>), grid, block, P.lds, stream, L);
      break;
    case kMaxValue:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kMaxValue, EXT>), grid, block, P.lds, stream, L);
      break;
    default:  // argmax: a single table, never the extended form
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kMax, false>), grid, block, P.lds, stream, L);
  }
  FWDMI_HIP_CHECK(hipGetLastError());
  return FWDMI_OK;
}

template <typename TW, typename TI, int VEC>
int launch_kind(const BagPlan& P, hipStream_t stream) {
  return P.ext ? launch_kind_ext<TW, TI, VEC, true>(P, stream) : launch_kind_ext<TW, TI, VEC, false>(P, stream);
}

template <typename TW, typename TI>
int launch_vec(const BagPlan& P, hipStream_t stream) {
  constexpr int kVec = 16 / sizeof(TW);
  return P.vec ? launch_kind<TW, TI, kVec>(P, stream) : launch_kind<TW, TI, 1>(P, stream);
}

// CUs and dies of the current device, asked once per device.  The number of dies is what the
// runtime reports; a runtime that does not know the attribute leaves the device at one die, and
// the launch plan then keeps the plain table-major order.
int device_topology(BagTopology* topo) {
  static std::mutex mu;
  static BagTopology known[kMaxDevices] = {};
  int dev = 0;
  FWDMI_HIP_CHECK(hipGetDevice(&dev));
  const bool cached = dev >= 0 && dev < kMaxDevices;
  std::lock_guard<std::mutex> lock(mu);
  if (cached && known[dev].cus > 0) {
    *topo = known[dev];
    return FWDMI_OK;
  }
  BagTopology t{0, 1};
  FWDMI_HIP_CHECK(hipDeviceGetAttribute(&t.cus, hipDeviceAttributeMultiprocessorCount, dev));
  FWDMI_REQUIRE(t.cus > 0, "device %d reports %d compute units", dev, t.cus);
  int xcds = 0;
  if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, dev) == hipSuccess && xcds > 0)
    t.xcds = xcds;
  else
    (void)hipGetLastError();
  if (cached) known[dev] = t;
  *topo = t;
  return FWDMI_OK;
}

// Plans the launch (bag_plan: pure host arithmetic, tested without a GPU) and issues it.
int bag_dispatch(const fwdmi_bag_table* tables_dev, const fwdmi_bag_table* tables_inline, int n_tables,
                 const fwdmi_bag_table& single,
                 void* output, int64_t n_bags, int64_t fixed_len, int dim, int op, double avg_len,
                 const fwdmi_bag_ext* ext, hipStream_t stream) {
  clear_error();
  // Without a usable device the arguments are still checked first (against a nominal device), so that a
  // caller learns of a bad argument before it learns of the missing GPU; the device's error stands otherwise.
  BagTopology topo{256, 8};
  const int topo_rc = device_topology(&topo);
  BagPlan P;
  if (const int rc = bag_plan(tables_dev, tables_inline, n_tables, single, output, n_bags, fixed_len, dim, op, avg_len,
                              ext, topo, &P))
    return rc;
  if (P.empty) {  // no bags: nothing to launch, with or without a device
    clear_error();
    return FWDMI_OK;
  }
  if (topo_rc) return topo_rc;
  if (P.f16) return P.i64 ? launch_vec<_Float16, int64_t>(P, stream) : launch_vec<_Float16, int32_t>(P, stream);
  return P.i64 ? launch_vec<float, int64_t>(P, stream) : launch_vec<float, int32_t>(P, stream);
}

}  // namespace
}  // namespace fwdmi

extern "C" {

int fwdmi_embedding_bag(const void* input, const void* input_2, void* output, int64_t input_size,
                        int64_t block_size, const void* data, int64_t count, int32_t dim,
                        int64_t data_offset, int32_t op_type, const fwdmi_bag_ext* ext, void* stream) {
  fwdmi_bag_table t{data, input, input_2, count, input_size, data_offset, 0, nullptr};
  const double avg = block_size > 0 ? (double)input_size / (double)block_size : 1.0;
  return fwdmi::bag_dispatch(nullptr, nullptr, 1, t, output, block_size, -1, dim, op_type, avg, ext,
                             static_cast<hipStream_t>(stream));
}

int fwdmi_embedding_bag_fixed(const void* input, void* output, int64_t batch_size, int64_t offset,
                              const void* data, int64_t count, int32_t dim, int64_t data_offset,
                              int32_t op_type, const fwdmi_bag_ext* ext, void* stream) {
  if (offset < 0 || batch_size < 0 || (offset > 0 && batch_size > INT64_MAX / offset))
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "fixed-length bags: batch %lld x length %lld",
                            (long long)batch_size, (long long)offset);
  fwdmi_bag_table t{data, input, nullptr, count, batch_size * offset, data_offset, 0, nullptr};
  return fwdmi::bag_dispatch(nullptr, nullptr, 1, t, output, batch_size, offset, dim, op_type, (double)offset, ext,
                             static_cast<hipStream_t>(stream));
}

int fwdmi_gather(const void* input, void* output, int64_t batch_size, int64_t offset, const void* data,
                 int64_t count, int32_t dim, int64_t data_offset, const fwdmi_bag_ext* ext, void* stream) {
  if (offset < 0 || batch_size < 0 || (offset > 0 && batch_size > INT64_MAX / offset))
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "gather: batch %lld x %lld", (long long)batch_size,
                            (long long)offset);
  // A gather is a sum over bags of exactly one id.
  fwdmi_bag_ext x = ext ? *ext : fwdmi_bag_ext{FWDMI_F32, FWDMI_I32, FWDMI_F32, 0, nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, nullptr};
  x.per_sample_weights = nullptr;
  x.max_indices = nullptr;
  x.square_sum_out = nullptr;
  x.out_row_stride = 0;
  const int64_t n = batch_size * offset;
  fwdmi_bag_table t{data, input, nullptr, count, n, data_offset, 0, nullptr};
  return fwdmi::bag_dispatch(nullptr, nullptr, 1, t, output, n, 1, dim, FWDMI_OP_SUM, 1.0, &x,
                             static_cast<hipStream_t>(stream));
}

int fwdmi_embedding_bag_multi(const fwdmi_bag_table* tables_dev, int32_t n_tables, int64_t n_bags,
                              void* output, int32_t dim, int32_t op_type, double avg_bag_len,
                              const fwdmi_bag_ext* ext, void* stream) {
  if (!tables_dev) return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "multi-table bags: null table array");
  if (ext && ext->per_sample_weights)
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG,
                            "multi-table bags: per-sample weights go into the table descriptors "
                            "(FWDMI_BAG_TABLE_WEIGHTS), not into ext->per_sample_weights");
  fwdmi_bag_table none{};
  return fwdmi::bag_dispatch(tables_dev, nullptr, n_tables, none, output, n_bags, -1, dim, op_type, avg_bag_len, ext,
                             static_cast<hipStream_t>(stream));
}

int fwdmi_bag_tables_fill(const fwdmi_bag_table* tables_host, int32_t n_tables, fwdmi_bag_table* tables_dev,
                          void* stream) {
  fwdmi::clear_error();
  if (n_tables < 0 || (n_tables > 0 && (!tables_host || !tables_dev)))
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "table descriptors: null argument");
  for (int32_t at = 0; at < n_tables; at += fwdmi::kFillChunk) {
    const int n = std::min<int32_t>(fwdmi::kFillChunk, n_tables - at);
    fwdmi::TableChunk c{};
    std::copy(tables_host + at, tables_host + at + n, c.t);
    hipLaunchKernelGGL(fwdmi::bag_tables_fill_kernel, dim3(1), dim3(64), 0,
                       static_cast<hipStream_t>(stream), c, n, tables_dev + at);
    FWDMI_HIP_CHECK(hipGetLastError());
  }
  return FWDMI_OK;
}

namespace {
// What the device-descriptor form leaves to its caller, checked where the descriptors are host memory.
int check_host_tables(const char* what, const fwdmi_bag_table* tables_host, int32_t n_tables, int32_t dim,
                      const fwdmi_bag_ext* ext) {
  const size_t sw = ext ? fwdmi::dtype_size(ext->table_dtype) : sizeof(float);
  const size_t so = ext ? fwdmi::dtype_size(ext->out_dtype) : sizeof(float);
  const int64_t stride = ext && ext->out_row_stride > 0 ? ext->out_row_stride : dim;
  if (ext && (!fwdmi::is_float_dtype(ext->table_dtype) || !fwdmi::is_float_dtype(ext->out_dtype)))  // sizes of 0 below otherwise
    return fwdmi::set_error(FWDMI_ERR_UNSUPPORTED, "%s: unsupported dtype (table %d, out %d)", what, ext->table_dtype,
                            ext->out_dtype);
  for (int32_t t = 0; t < n_tables; ++t) {
    const fwdmi_bag_table& d = tables_host[t];
    FWDMI_REQUIRE(d.count <= 0 || d.data, "%s: table %d has rows but no data", what, t);
    FWDMI_REQUIRE(d.input_size >= 0 && (d.input_size == 0 || d.input) && d.input_2, "%s: table %d lacks ids or offsets", what, t);
    FWDMI_REQUIRE(d.out_col >= 0 && dim > 0 && stride >= dim && d.out_col <= stride - dim,
                  "%s: table %d writes columns %lld.. beyond the row of %lld", what, t, (long long)d.out_col,
                  (long long)stride);
    if (((size_t)dim * sw) % 16 == 0) {  // rows are read (and written) as 16-byte slices
      const size_t store_align = std::min<size_t>(16, 16 / sw * so);
      FWDMI_REQUIRE(reinterpret_cast<uintptr_t>(d.data) % 16 == 0 && ((size_t)d.out_col * so) % store_align == 0,
                    "%s: table %d: data or output column not aligned to its slices", what, t);
    }
  }
  return FWDMI_OK;
}

// Every table's own mean bag length, from host descriptors, unless the caller gave them.
void fill_avg_len(fwdmi_bag_ext* x, float* avg_len_t, const fwdmi_bag_table* tables_host, int32_t n_tables,
                  int64_t n_bags) {
  if ((x->flags & FWDMI_BAG_TABLE_AVG_LEN) || n_tables > fwdmi::kMaxVarTables || n_bags <= 0) return;
  for (int32_t t = 0; t < n_tables; ++t) avg_len_t[t] = (float)((double)tables_host[t].input_size / (double)n_bags);
  x->table_avg_len = avg_len_t;
  x->flags |= FWDMI_BAG_TABLE_AVG_LEN;
}

const fwdmi_bag_ext kPlainExt = {FWDMI_F32, FWDMI_I32, FWDMI_F32, 0, nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, nullptr};
}  // namespace

int fwdmi_embedding_bag_multi_host(const fwdmi_bag_table* tables_host, int32_t n_tables, fwdmi_bag_table* tables_dev,
                                   int64_t n_bags, void* output, int32_t dim, int32_t op_type, double avg_bag_len,
                                   const fwdmi_bag_ext* ext, void* stream) {
  fwdmi::clear_error();
  static const char* const kWhat = "multi-table bags (host descriptors)";
  if (!tables_host || n_tables <= 0) return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "%s: null or empty table array", kWhat);
  if (ext && ext->per_sample_weights)
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG,
                            "multi-table bags: per-sample weights go into the table descriptors "
                            "(FWDMI_BAG_TABLE_WEIGHTS), not into ext->per_sample_weights");
  if (const int rc = check_host_tables(kWhat, tables_host, n_tables, dim, ext)) return rc;
  fwdmi_bag_ext x = ext ? *ext : kPlainExt;
  float avg_len_t[fwdmi::kMaxVarTables];
  fill_avg_len(&x, avg_len_t, tables_host, n_tables, n_bags);
  fwdmi_bag_table none{};
  if (n_tables <= fwdmi::kInlineTables)  // the descriptors are part of the launch: no second launch, no device array
    return fwdmi::bag_dispatch(nullptr, tables_host, n_tables, none, output, n_bags, -1, dim, op_type, avg_bag_len, &x,
                               static_cast<hipStream_t>(stream));
  if (!tables_dev)
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "%s: %d tables need a device array for their descriptors (more than %d)",
                            kWhat, n_tables, fwdmi::kInlineTables);
  if (const int rc = fwdmi_bag_tables_fill(tables_host, n_tables, tables_dev, stream)) return rc;
  return fwdmi::bag_dispatch(tables_dev, nullptr, n_tables, none, output, n_bags, -1, dim, op_type, avg_bag_len, &x,
                             static_cast<hipStream_t>(stream));
}

int fwdmi_embedding_bag_multi_noalloc(const fwdmi_bag_table* tables_host, int32_t n_tables, int64_t n_bags,
                                      void* output, int32_t dim, int32_t op_type, double avg_bag_len,
                                      const fwdmi_bag_ext* ext, void* stream) {
  fwdmi::clear_error();
  static const char* const kWhat = "multi-table bags (no allocation)";
  if (!tables_host || n_tables <= 0) return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "%s: null or empty table array", kWhat);
  if (n_tables > fwdmi::kNoAllocMaxTables)
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG,
                            "multi-table bags (no allocation): %d tables exceed the built-in descriptor "
                            "buffer of %d; use fwdmi_embedding_bag_multi with a descriptor array of your own",
                            n_tables, fwdmi::kNoAllocMaxTables);
  if (ext && ext->per_sample_weights)
    return fwdmi::set_error(FWDMI_ERR_BAD_ARG,
                            "multi-table bags: per-sample weights go into the table descriptors "
                            "(FWDMI_BAG_TABLE_WEIGHTS), not into ext->per_sample_weights");
  // the descriptors are host memory here, so what the device form leaves to its caller is checked
  if (const int rc = check_host_tables(kWhat, tables_host, n_tables, dim, ext)) return rc;
  fwdmi_bag_table none{};
  // the descriptors are on the host here: every table's own mean bag length comes with them
  fwdmi_bag_ext with_len = ext ? *ext : kPlainExt;
  float avg_len_t[fwdmi::kMaxVarTables];
  fill_avg_len(&with_len, avg_len_t, tables_host, n_tables, n_bags);
  // Few enough tables travel with the launch as kernel arguments: nothing is shared between calls then.
  if (n_tables <= fwdmi::kInlineTables)
    return fwdmi::bag_dispatch(nullptr, tables_host, n_tables, none, output, n_bags, -1, dim, op_type, avg_bag_len,
                               &with_len, static_cast<hipStream_t>(stream));
  fwdmi_bag_table* dev_tables = nullptr;
  if (const int rc = fwdmi::scratch_on_current_device(&dev_tables)) return rc;
  // The descriptor writes and the launch that reads them are enqueued under one lock, so that two host
  // threads issuing on the same stream cannot interleave them; stream order then keeps a call's
  // descriptors intact until its launch has read them.  Calls on different streams of one GPU still
  // race unless the caller orders them.
  std::lock_guard<std::mutex> lock(fwdmi::g_noalloc_issue_mu);
  if (const int rc = fwdmi_bag_tables_fill(tables_host, n_tables, dev_tables, stream)) return rc;
  return fwdmi::bag_dispatch(dev_tables, nullptr, n_tables, none, output, n_bags, -1, dim, op_type, avg_bag_len, &with_len,
                             static_cast<hipStream_t>(stream));
}

int fwdmi_bag_device_topology(int32_t* cus, int32_t* xcds) {
  fwdmi::clear_error();
  if (!cus || !xcds) return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "device topology: null argument");
  fwdmi::BagTopology topo{0, 1};
  if (const int rc = fwdmi::device_topology(&topo)) return rc;
  *cus = topo.cus;
  *xcds = topo.xcds;
  return FWDMI_OK;
}

// Measured on the 26-table configuration (tables of 0.25 MB .. 2.5 GB): per-bag cost ratios
// between 1.3 and 1.6 for HBM-resident against L2-resident tables balance the eight XCDs best.
int fwdmi_bag_table_cost(const int64_t* table_bytes, int32_t n_tables, float* cost) {
  if (!table_bytes || !cost || n_tables < 0) return fwdmi::set_error(FWDMI_ERR_BAD_ARG, "table cost: null argument");
  const double small = 2.0 * 1048576.0, large = 512.0 * 1048576.0, beta = 0.45;
  for (int t = 0; t < n_tables; ++t) {
    const double b = (double)std::max<int64_t>(table_bytes[t], 1);
    const double miss = std::min(1.0, std::max(0.0, std::log(b / small) / std::log(large / small)));
    cost[t] = (float)(1.0 + beta * miss);
  }
  return FWDMI_OK;
}

}  // extern "C"
