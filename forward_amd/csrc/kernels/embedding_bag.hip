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
#include "device_util.h"

namespace fwdmi {
namespace {

constexpr int kXcds = 8;           // accelerator complex dies; workgroup b is dispatched to XCD b % 8
constexpr int kWG = 256;           // lanes per workgroup (large batches; small ones use 128 or 64)
#ifndef FWDMI_BAG_IDX_BYTES
#define FWDMI_BAG_IDX_BYTES 16384
#endif
constexpr int kIdxBytes = FWDMI_BAG_IDX_BYTES;   // LDS bytes of the id window per workgroup (4096 row numbers / 2048 64-bit ids)
constexpr int kMaxBagsPerWG = 512; // offsets staged in LDS per workgroup (+1)
constexpr int kLenBuckets = 256;   // bag-length buckets of the in-LDS counting sort
constexpr int kInlineTables = FWDMI_BAG_INLINE_TABLES;  // table descriptors that travel with the launch as kernel arguments
constexpr int kMaxVarTables = 64;  // tables of a launch whose runs may differ in size from table to table
#ifndef FWDMI_BAG_UNROLL
#define FWDMI_BAG_UNROLL 8
#endif
#ifndef FWDMI_BAG_STREAM_BYTES
#define FWDMI_BAG_STREAM_BYTES (8.0 * 1048576.0)  // results of at least this size are stored with the non-temporal hint
#endif
#ifndef FWDMI_BAG_TAIL_RUNS
#define FWDMI_BAG_TAIL_RUNS(resident) ((resident) / 4)  // measured best on the 26-table configuration (16 .. 384 tried)
#endif
#ifndef FWDMI_BAG_WAVES_PER_EU
#define FWDMI_BAG_WAVES_PER_EU 6  // register budget of 80 VGPRs: measured best on the 26-table configuration
#endif
// argmax tracking and the second accumulator carry more live registers: they keep the looser budget;
// the weighted form sits in between (measured on the 26-table configuration: 4 -> 5 wavefronts 2 % faster)
#define FWDMI_BAG_OCCUPANCY \
  __attribute__((amdgpu_waves_per_eu((KIND == kMax || KIND == kSumSq) ? 4 : KIND == kWeighted ? 5 : FWDMI_BAG_WAVES_PER_EU)))
constexpr int kUnroll = FWDMI_BAG_UNROLL;  // row loads in flight per lane

// kMax also tracks the argmax (needs max_indices); kMaxValue is the plugin's case: values only
// kSumSq: the sum and the sum of squares of the same rows in one pass (two outputs)
enum Kind { kPlain = 0, kWeighted = 1, kMax = 2, kSquare = 3, kMaxValue = 4, kSumSq = 5 };

struct BagLaunch {
  const fwdmi_bag_table* tables;  // device array of descriptors, or nullptr -> `inline_tables`
  fwdmi_bag_table inline_tables[kInlineTables];  // a single-table launch uses [0]
  int32_t multi;  // several tables (descriptors in `tables` or inline): weights come with the descriptors
  const void* psw;  // per-sample weights of the single-table form (a table of a batch carries its own)
  void* out;
  void* out2;  // kSumSq: the sums of squares, laid out like `out`
  void* max_indices;
  int32_t* oob_flag;
  int64_t n_bags;
  int64_t out_stride;
  int64_t fixed_len;  // >= 0: bag b covers ids [b*fixed_len, (b+1)*fixed_len); < 0: use offsets
  int32_t dim;
  int32_t op;
  int32_t out_f16;
  int32_t include_last;
  int32_t log2_g;
  int32_t n_slices;
  int32_t bags_per_wg;
  int32_t wgs_per_table;
  int32_t vec_store;  // 0: element stores; 1: 16-byte stores; 2: 16-byte stores with the non-temporal hint
  float one;  // 1.0f
  int32_t xcd_affinity;      // != 0: XCD x works through work items [xcd_start[x], xcd_start[x+1])
  int32_t xcd_start[kXcds + 1];
  int32_t total_wgs;
  int32_t tail_runs;  // XCD mapping only: the last `tail_runs` runs of every XCD's segment are issued as four workgroups each
  int32_t idx_cap;    // 32-bit words of the LDS id window: that many row numbers, or half as many 64-bit ids
  // Multi-table launches whose tables differ in mean bag length: table t's runs hold run_bags[t] bags and
  // are work items [run_start[t], run_start[t + 1]); bags_per_wg is then the largest of them (it sizes LDS).
  int32_t var_runs;
  int32_t run_start[kMaxVarTables + 1];
  uint16_t run_bags[kMaxVarTables];
};

// Hands elements first[0 .. n) to put(i, value), the workgroup's lanes sharing the work.  Long
// ranges come in with 16-byte loads (a load instruction occupies the CU's memory pipeline for the
// same time whatever its width); the elements before the first 16-byte boundary and behind the
// last one go one by one, so nothing outside the range is read.  `first` is aligned to its type.
template <typename T, typename Put>
__device__ __forceinline__ void stream_in(const T FWDMI_GLOBAL* first, int n, int tid, int lanes, Put put) {
  constexpr int kPer = 16 / (int)sizeof(T);
  if (n < 2 * lanes) {  // uniform over the workgroup: too short for the split to pay
    for (int i = tid; i < n; i += lanes) put(i, first[i]);
    return;
  }
  const int misalign = (int)((reinterpret_cast<uintptr_t>(first) & 15) / sizeof(T));
  const int head = (kPer - misalign) & (kPer - 1);
  const int n_vec = (n - head) / kPer;
  const int body_end = head + n_vec * kPer;
  for (int v = tid; v < n_vec; v += lanes) {
    const Pack<T, kPer> p = gload<T, kPer>(first + head + v * kPer);
#pragma unroll
    for (int e = 0; e < kPer; ++e) put(head + v * kPer + e, p.v[e]);
  }
  if (tid < head) put(tid, first[tid]);
  if (body_end + tid < n) put(body_end + tid, first[body_end + tid]);
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
  // Each XCD has its own L2.  On request, a multi-table launch undoes the hardware's round-robin
  // placement (workgroup b runs on XCD b % 8) so that one XCD works through whole tables: a
  // table's hot rows are then fetched into one L2 instead of all eight.
  int work = blockIdx.x;
  int quarter = -1;  // 0..3: this workgroup reduces that quarter of run `work`; -1: the whole run
  if (L.xcd_affinity) {
    // A workgroup lives for about an eighth of the launch, so after an XCD has started its last
    // run its CUs empty out for that long.  The last runs of a segment are therefore cut in four:
    // their workgroups live a quarter as long and the XCD drains that much faster.
    const int x = (int)(blockIdx.x % kXcds);
    const int j = (int)(blockIdx.x / kXcds);
    const int len = L.xcd_start[x + 1] - L.xcd_start[x];
    const int tail = min(len, L.tail_runs);
    const int whole = len - tail;
    if (j < whole) {
      work = L.xcd_start[x] + j;
    } else {
      const int jj = j - whole;
      if (jj >= 4 * tail) return;
      work = L.xcd_start[x] + whole + (jj >> 2);
      quarter = jj & 3;
    }
  }
  int t, wg, bpw;  // table, run of the table, bags of a run of this table: uniform over the workgroup
  if (EXT && L.var_runs) {
    t = 0;
    while (work >= L.run_start[t + 1]) ++t;  // at most kMaxVarTables steps over kernel arguments
    wg = work - L.run_start[t];
    bpw = L.run_bags[t];
  } else {
    t = work / L.wgs_per_table;
    wg = work - t * L.wgs_per_table;
    bpw = L.bags_per_wg;
  }
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

  const int quarter_bags = bpw >> 2;  // the host keeps run sizes multiples of 4 when it cuts runs
  const int64_t bag0 = (int64_t)wg * bpw + (quarter > 0 ? quarter * quarter_bags : 0);
  const int nb = (int)min((int64_t)(quarter < 0 ? bpw : quarter_bags), L.n_bags - bag0);
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
          if (VEC > 1 && L.vec_store == 2) {
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

static_assert(sizeof(BagLaunch) <= 4096, "kernel arguments are limited to 4 KiB");

struct BagShape {
  int grid, block;
  size_t lds;
};

// Bytes of the kernel's LDS carve-up.
size_t bag_lds_bytes(const BagLaunch& L, bool weighted) {
  size_t b = (size_t)(L.bags_per_wg + 2) * sizeof(int64_t) + (size_t)L.idx_cap * sizeof(uint32_t);
  if (weighted) b += (size_t)L.idx_cap * sizeof(float);
  b += (size_t)L.bags_per_wg * (sizeof(int) + sizeof(uint16_t));
  return (b + 15) & ~(size_t)15;
}

template <typename TW, typename TI, int VEC, bool EXT>
int launch_kind_ext(int kind, const BagLaunch& L, const BagShape& sh, hipStream_t stream) {
  const dim3 grid(sh.grid), block(sh.block);
  switch (kind) {
    case kPlain:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kPlain, EXT>), grid, block, sh.lds, stream, L);
      break;
    case kSquare:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kSquare, EXT>), grid, block, sh.lds, stream, L);
      break;
    case kSumSq:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kSumSq, EXT>), grid, block, sh.lds, stream, L);
      break;
    case kWeighted:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kWeighted, EXT>), grid, block, sh.lds, stream, L);
      break;
    case kMaxValue:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kMaxValue, EXT>), grid, block, sh.lds, stream, L);
      break;
    default:
      hipLaunchKernelGGL((bag_reduce_kernel<TW, TI, VEC, kMax, false>), grid, block, sh.lds, stream, L);
  }
  FWDMI_HIP_CHECK(hipGetLastError());
  return FWDMI_OK;
}

template <typename TW, typename TI, int VEC>
int launch_kind(int kind, const BagLaunch& L, const BagShape& sh, hipStream_t stream) {
  const bool ext = L.var_runs || (L.multi && !L.tables);  // per-table run sizes, or descriptors among the arguments
  return ext ? launch_kind_ext<TW, TI, VEC, true>(kind, L, sh, stream)
             : launch_kind_ext<TW, TI, VEC, false>(kind, L, sh, stream);
}

template <typename TW, typename TI>
int launch_vec(bool vec, int kind, const BagLaunch& L, const BagShape& sh, hipStream_t stream) {
  constexpr int kVec = 16 / sizeof(TW);
  return vec ? launch_kind<TW, TI, kVec>(kind, L, sh, stream)
             : launch_kind<TW, TI, 1>(kind, L, sh, stream);
}

int device_cus() {
  static const int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      return v;
    return 256;
  }();
  return cus;
}

int next_pow2(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

// Validates arguments, picks the lane mapping and launches.  `tables_dev` non-null selects the
// multi-table form with descriptors in device memory, `tables_inline` (host, at most kInlineTables)
// the one whose descriptors travel as kernel arguments; with neither, `single` is the table.
int bag_dispatch(const fwdmi_bag_table* tables_dev, const fwdmi_bag_table* tables_inline, int n_tables,
                 const fwdmi_bag_table& single,
                 void* output, int64_t n_bags, int64_t fixed_len, int dim, int op, double avg_len,
                 const fwdmi_bag_ext* ext, hipStream_t stream) {
  clear_error();
  const bool multi = tables_dev || tables_inline;
  static const fwdmi_bag_ext kDefaultExt = {FWDMI_F32, FWDMI_I32, FWDMI_F32, 0, nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, nullptr};
  const fwdmi_bag_ext& x = ext ? *ext : kDefaultExt;

  if (!is_float_dtype(x.table_dtype) || !is_float_dtype(x.out_dtype) || !is_index_dtype(x.index_dtype))
    return set_error(FWDMI_ERR_UNSUPPORTED, "embedding bag: unsupported dtype (table %d, index %d, out %d)",
                     x.table_dtype, x.index_dtype, x.out_dtype);
  if (op != FWDMI_OP_SUM && op != FWDMI_OP_MEAN && op != FWDMI_OP_MAX && op != FWDMI_OP_SQUARE_SUM)
    return set_error(FWDMI_ERR_UNSUPPORTED, "embedding bag: unknown op %d", op);
  // dim: a row's byte size and a run's (bag, slice) count stay far inside 32 bits
  FWDMI_REQUIRE(n_bags >= 0 && dim > 0 && dim <= (1 << 24) && n_tables > 0,
                "embedding bag: n_bags=%lld dim=%d (1 .. 2^24) n_tables=%d", (long long)n_bags, dim, n_tables);
  FWDMI_REQUIRE(!(x.per_sample_weights || (multi && (x.flags & FWDMI_BAG_TABLE_WEIGHTS))) || op == FWDMI_OP_SUM,
                "embedding bag: per_sample_weights needs op SUM (got %d)", op);
  FWDMI_REQUIRE(!x.max_indices || (op == FWDMI_OP_MAX && !multi),
                "embedding bag: max_indices needs op MAX on a single table");
  const int64_t out_stride = x.out_row_stride > 0 ? x.out_row_stride : dim;
  FWDMI_REQUIRE(out_stride >= dim, "embedding bag: out_row_stride %lld < dim %d", (long long)out_stride, dim);
  if (n_bags == 0) return FWDMI_OK;
  FWDMI_REQUIRE(output != nullptr, "embedding bag: null output");
  if (!multi) {
    FWDMI_REQUIRE(single.count > 0 && single.data, "embedding bag: empty table");
    FWDMI_REQUIRE(single.input_size >= 0 && (single.input_size == 0 || single.input),
                  "embedding bag: null ids");
    FWDMI_REQUIRE(fixed_len >= 0 || single.input_2, "embedding bag: null offsets");
    FWDMI_REQUIRE(single.out_col >= 0 && single.out_col + dim <= out_stride, "embedding bag: out_col");
  }

  const size_t sw = dtype_size(x.table_dtype), so = dtype_size(x.out_dtype);
  const int vec_w = (int)(16 / sw);
  // 128-bit row loads need 16-byte row pitch and base; a multi-table launch is checked by its caller.
  bool vec = (dim % vec_w) == 0;
  if (!multi) vec = vec && (reinterpret_cast<uintptr_t>(single.data) % 16) == 0;
  const int VEC = vec ? vec_w : 1;

  BagLaunch L{};
  L.tables = tables_dev;
  L.multi = multi;
  if (tables_inline) {
    FWDMI_REQUIRE(n_tables <= kInlineTables, "embedding bag: %d tables do not fit the launch's arguments (%d)", n_tables,
                  kInlineTables);
    std::copy(tables_inline, tables_inline + n_tables, L.inline_tables);
  } else {
    L.inline_tables[0] = single;
  }
  L.out = output;
  L.max_indices = x.max_indices;
  L.out2 = x.square_sum_out;
  L.oob_flag = x.oob_flag;
  L.n_bags = n_bags;
  L.out_stride = out_stride;
  L.fixed_len = fixed_len;
  L.one = 1.0f;
  L.dim = dim;
  L.op = op;
  L.out_f16 = x.out_dtype == FWDMI_F16;
  L.include_last = x.include_last_offset != 0;
  const int lanes = std::min(64, next_pow2((dim + VEC - 1) / VEC));
  L.log2_g = __builtin_ctz(lanes);
  L.n_slices = (dim + lanes * VEC - 1) / (lanes * VEC);
  if (avg_len < 1.0) avg_len = 1.0;
  // Run length: as many bags as keep the run's ids inside the LDS window, but no more than leaves
  // the chip with ~4 workgroups per CU; small batches also shrink the workgroup (down to one
  // wavefront) so that every CU gets work, but not below one slot per bag of the run: a slot
  // that reduces two bags one after the other doubles the launch's critical path.
  // The id window is sized for 32-bit row numbers unless a single table is known to be too large
  // for them (more than 2^24 rows or 4 GiB): then it holds the launch's 64-bit ids.  (A multi-table
  // launch cannot see its tables' sizes here; a run of such a table that does not fit the window
  // reads its ids from global memory.)
  const bool i64_ids = x.index_dtype == FWDMI_I64;
  const bool wide_ids = i64_ids && !multi &&
                        (single.count > (1 << 24) || (uint64_t)single.count * dim * sw > ((uint64_t)1 << 32));
  const int max_cap = kIdxBytes / (wide_ids ? 8 : 4);
  const int64_t total_bags = n_bags * n_tables;
  const int64_t target_wgs = (int64_t)device_cus() * 4;
  int64_t want_bags = std::max<int64_t>(1, total_bags / target_wgs);
  const int64_t fit_bags = std::max<int64_t>(1, (int64_t)(max_cap / 2.0 / avg_len));
  want_bags = std::min<int64_t>(std::min(want_bags, fit_bags), kMaxBagsPerWG);
  int block = kWG;
  while (block > 64 && block / 2 >= lanes && (int64_t)(block / 2 / lanes) >= want_bags * L.n_slices) block /= 2;
  const int slots = block / lanes;
  // Bags of a run and words of its id window for bags of `avg` ids on average.
  const bool weighted_launch = x.per_sample_weights || (multi && (x.flags & FWDMI_BAG_TABLE_WEIGHTS));
  auto size_run = [&](double avg, int64_t want, int* bags, int* cap) {
    // a whole number of rounds over the slots
    const int64_t units = std::max<int64_t>(slots, want * L.n_slices / slots * slots);
    *bags = (int)std::max<int64_t>(1, std::min<int64_t>(kMaxBagsPerWG, units / L.n_slices));
    *cap = std::min(max_cap, std::max(64, next_pow2((int)std::min<double>(max_cap, avg * *bags * 2.0)))) * (wide_ids ? 2 : 1);
    // With per-sample weights every window slot also holds a weight, and at twice the expected ids the
    // two windows (35 KiB for a run of 112 bags) leave a CU four workgroups.  The expected ids plus 5.5
    // times the spread of a sum of `bags` lengths whose deviation equals their mean keeps all
    // but one run in ten thousand staged (a run that reads its ids unstaged takes several times as
    // long: at 4 spreads, 0.25 % of the runs unstaged, the launch below measures 0.466 ms); measured on
    // the 26-table configuration: 0.490 -> 0.440 ms together with the register budget above.
    if (weighted_launch) {
      const double ids = avg * (*bags + 5.5 * std::sqrt((double)*bags));
      const int tight = ((int)std::min<double>(max_cap, std::max(64.0, ids)) + 63) / 64 * 64 * (wide_ids ? 2 : 1);
      *cap = std::min(*cap, tight);
    }
  };
  size_run(avg_len, want_bags, &L.bags_per_wg, &L.idx_cap);
  // Tables whose mean bag lengths differ (one-hot features beside multi-hot ones) get runs of their
  // own size: sized from the launch's mean, the runs of a long-bag table overflow the id window and
  // those of a one-hot table hold a few ids each.  Measured on 13 one-hot + 13 long-bag tables
  // (28.6 M ids): 0.562 ms with one run size.
  int run_bags[kMaxVarTables];
  bool var_runs = false;
  if (multi && x.table_avg_len && n_tables > 1 && n_tables <= kMaxVarTables) {
    const int64_t want_all = std::min<int64_t>(std::max<int64_t>(1, total_bags / target_wgs), kMaxBagsPerWG);
    int lo = INT_MAX, hi = 0, cap_max = 0;
    for (int t = 0; t < n_tables; ++t) {
      const double a = (double)x.table_avg_len[t];
      FWDMI_REQUIRE(a >= 0.0 && a < 1e30, "embedding bag: table_avg_len must be finite and not negative");
      const double avg_t = std::max(1.0, a);
      const int64_t fit_t = std::max<int64_t>(1, (int64_t)(max_cap / 2.0 / avg_t));
      int cap_t = 0;
      size_run(avg_t, std::min(want_all, fit_t), &run_bags[t], &cap_t);
      lo = std::min(lo, run_bags[t]);
      hi = std::max(hi, run_bags[t]);
      cap_max = std::max(cap_max, cap_t);
    }
    if (2 * hi >= 3 * lo) {  // otherwise one size serves all tables
      var_runs = true;
      L.bags_per_wg = hi;
      L.idx_cap = cap_max;
    }
  }
  const int64_t wgs = (n_bags + L.bags_per_wg - 1) / L.bags_per_wg;
  FWDMI_REQUIRE(wgs * n_tables < (int64_t)1 << 31, "embedding bag: grid too large");
  L.wgs_per_table = (int)wgs;
  int64_t total_runs = wgs * n_tables;
  L.var_runs = 0;
  if (var_runs) {
    total_runs = 0;
    for (int t = 0; t < n_tables; ++t) {
      L.run_start[t] = (int32_t)total_runs;
      L.run_bags[t] = (uint16_t)run_bags[t];
      total_runs += (n_bags + run_bags[t] - 1) / run_bags[t];
      FWDMI_REQUIRE(total_runs < (int64_t)1 << 31, "embedding bag: grid too large");
    }
    L.run_start[n_tables] = (int32_t)total_runs;
    L.var_runs = 1;
  }
  const size_t store_align = std::min<size_t>(16, VEC * so);
  L.vec_store = VEC > 1 && (reinterpret_cast<uintptr_t>(output) % store_align) == 0 &&
                (reinterpret_cast<uintptr_t>(x.square_sum_out) % store_align) == 0 &&
                ((out_stride * so) % store_align) == 0 &&
                (multi || (single.out_col * so) % store_align == 0);

  // A result of several MiB does not survive in the 4 MiB L2 of the XCD that wrote it until somebody
  // reads it (and a reader on another XCD would not find it there anyway); written with the
  // non-temporal hint it does not displace table rows on its way out.  Measured: 2.8 % off the
  // 26-table launch (19 % when every row hits in cache), 3.8 % off 26 single-table launches of
  // 16 MiB results each; a reader of a 16 MiB result right behind the launch costs 2 % more.
  if (L.vec_store && (double)n_bags * n_tables * dim * so >= FWDMI_BAG_STREAM_BYTES) L.vec_store = 2;

  const bool weighted = weighted_launch;
  FWDMI_REQUIRE(!x.square_sum_out || (op == FWDMI_OP_SUM && !weighted),
                "embedding bag: square_sum_out needs op SUM without per-sample weights");
  const int kind = op == FWDMI_OP_MAX      ? (x.max_indices ? kMax : kMaxValue)
                   : op == FWDMI_OP_SQUARE_SUM ? kSquare
                   : weighted                  ? kWeighted
                   : x.square_sum_out          ? kSumSq
                                               : kPlain;
  L.psw = x.per_sample_weights;
  int grid = (int)total_runs;
  L.total_wgs = grid;
  L.xcd_affinity = 0;
  if (multi && n_tables > 1 && (x.flags & FWDMI_BAG_XCD_TABLE_AFFINITY)) {
    // Cut the table-major work list into eight contiguous segments of equal estimated cost
    // (equal length when the caller gives no per-table cost).
    L.xcd_affinity = 1;
    // A bag costs its rows plus a constant (result store, bookkeeping) worth kBagRows rows: fixed-length
    // launches of 1 .. 64 rows per bag fit rows / 36.6 TB/s + result bytes / 3.7 TB/s, and one-hot
    // tables beside tables of 33 ids per bag measure 1 : 4.1 per bag.  With every table's mean bag
    // length known the caller's per-bag cost is scaled by it; without, all tables count as equally long.
    constexpr double kBagRows = 9.6;
    auto cost_of = [&](int u) {
      double c = x.table_cost ? (double)x.table_cost[u] : 1.0;
      if (x.table_avg_len) c *= (std::max(0.0, (double)x.table_avg_len[u]) + kBagRows) / (avg_len + kBagRows);
      return c;
    };
    double total = 0.0;
    for (int t = 0; t < n_tables; ++t) {
      const double c = cost_of(t);
      FWDMI_REQUIRE(c > 0.0 && c < 1e30, "embedding bag: table_cost must be positive and finite");
      const double a = x.table_avg_len ? (double)x.table_avg_len[t] : 0.0;
      FWDMI_REQUIRE(a >= 0.0 && a < 1e30, "embedding bag: table_avg_len must be finite and not negative");
      total += cost_of(t) * (double)wgs;
    }
    int t = 0;
    double before = 0.0;  // cost of the tables before t
    int longest = 0;
    L.xcd_start[0] = 0;
    if (var_runs) {
      // the same cut with runs whose size differs from table to table: a table's cost is its bags' cost
      double all = 0.0;
      for (int u = 0; u < n_tables; ++u) all += cost_of(u) * (double)n_bags;
      for (int k = 1; k <= kXcds; ++k) {
        int cut = grid;
        if (k < kXcds) {
          const double target = all * k / kXcds;
          double c = cost_of(t);
          while (t < n_tables - 1 && before + c * (double)n_bags <= target) {
            before += c * (double)n_bags;
            ++t;
            c = cost_of(t);
          }
          const int64_t runs_t = L.run_start[t + 1] - L.run_start[t];
          const int64_t within =
              std::min<int64_t>(runs_t, std::max<int64_t>(0, (int64_t)((target - before) / (c * run_bags[t]) + 0.5)));
          cut = (int)std::max<int64_t>(L.xcd_start[k - 1], (int64_t)L.run_start[t] + within);
        }
        L.xcd_start[k] = cut;
        longest = std::max(longest, cut - L.xcd_start[k - 1]);
      }
    } else {
      for (int k = 1; k <= kXcds; ++k) {
        int cut = grid;
        if (k < kXcds) {
          const double target = total * k / kXcds;
          double c = cost_of(t);
          while (t < n_tables - 1 && before + c * (double)wgs <= target) {
            before += c * (double)wgs;
            ++t;
            c = cost_of(t);
          }
          const int64_t within = std::min<int64_t>(wgs, std::max<int64_t>(0, (int64_t)((target - before) / c + 0.5)));
          cut = (int)std::max<int64_t>(L.xcd_start[k - 1], (int64_t)t * wgs + within);
        }
        L.xcd_start[k] = cut;
        longest = std::max(longest, cut - L.xcd_start[k - 1]);
      }
    }
    // Runs cut in four at the end of every segment (see the kernel): as many as a quarter of what an XCD holds
    // at once, and only in launches that fill the chip several times over.
    const int resident = device_cus() / kXcds * 6;  // workgroups of 256 lanes an XCD holds at the 6-per-CU occupancy
    L.tail_runs = 0;
    bool can_cut = block == kWG && L.bags_per_wg % 4 == 0 && L.bags_per_wg / 4 >= slots;
    for (int u = 0; var_runs && u < n_tables; ++u) can_cut = can_cut && run_bags[u] % 4 == 0 && run_bags[u] / 4 >= slots;
    if (can_cut && longest >= 4 * resident) L.tail_runs = FWDMI_BAG_TAIL_RUNS(resident);
#ifdef FWDMI_EXP_ENV
    if (const char* e = getenv("FWDMI_EXP_TAIL_RUNS")) L.tail_runs = atoi(e);
#endif
    int most = 0;  // workgroups of the XCD with the most
    for (int k = 0; k < kXcds; ++k) {
      const int len = L.xcd_start[k + 1] - L.xcd_start[k];
      most = std::max(most, len + 3 * std::min(len, L.tail_runs));
    }
    FWDMI_REQUIRE((int64_t)most * kXcds < (int64_t)1 << 31, "embedding bag: grid too large");
    grid = most * kXcds;
  }
  const bool f16 = x.table_dtype == FWDMI_F16, i64 = x.index_dtype == FWDMI_I64;
  const BagShape sh{grid, block, bag_lds_bytes(L, kind == kWeighted)};
  if (f16)
    return i64 ? launch_vec<_Float16, int64_t>(vec, kind, L, sh, stream)
               : launch_vec<_Float16, int32_t>(vec, kind, L, sh, stream);
  return i64 ? launch_vec<float, int64_t>(vec, kind, L, sh, stream)
             : launch_vec<float, int32_t>(vec, kind, L, sh, stream);
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
  for (int32_t t = 0; t < n_tables; ++t) {
    const fwdmi_bag_table& d = tables_host[t];
    FWDMI_REQUIRE(d.count <= 0 || d.data, "%s: table %d has rows but no data", what, t);
    FWDMI_REQUIRE(d.input_size >= 0 && (d.input_size == 0 || d.input) && d.input_2, "%s: table %d lacks ids or offsets", what, t);
    FWDMI_REQUIRE(d.out_col >= 0 && dim > 0 && d.out_col + dim <= stride,
                  "%s: table %d writes columns %lld.. beyond the row of %lld", what, t, (long long)d.out_col,
                  (long long)stride);
    if (sw && ((size_t)dim * sw) % 16 == 0) {  // rows are read (and written) as 16-byte slices
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
  if (x->table_avg_len || n_tables > fwdmi::kMaxVarTables || n_bags <= 0) return;
  for (int32_t t = 0; t < n_tables; ++t) avg_len_t[t] = (float)((double)tables_host[t].input_size / (double)n_bags);
  x->table_avg_len = avg_len_t;
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
  fwdmi_bag_table* dev_tables = nullptr;
  if (const int rc = fwdmi::scratch_on_current_device(&dev_tables)) return rc;
  // stream order keeps a call's descriptors intact until its launch has read them, as long as
  // every call on this GPU uses the same stream (or the caller orders them)
  if (const int rc = fwdmi_bag_tables_fill(tables_host, n_tables, dev_tables, stream)) return rc;
  fwdmi_bag_table none{};
  // the descriptors are on the host here: every table's own mean bag length comes with them
  fwdmi_bag_ext with_len = ext ? *ext : kPlainExt;
  float avg_len_t[fwdmi::kMaxVarTables];
  fill_avg_len(&with_len, avg_len_t, tables_host, n_tables, n_bags);
  return fwdmi::bag_dispatch(dev_tables, nullptr, n_tables, none, output, n_bags, -1, dim, op_type, avg_bag_len, &with_len,
                             static_cast<hipStream_t>(stream));
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
