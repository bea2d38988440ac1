// Launch plan of the bag-reduction kernel: the kernel's argument block, the pure host function
// that fills it (run sizes, LDS carve-up, per-XCD segments, grid) and the mapping from a
// workgroup number to the bags it reduces.  Nothing here touches the GPU: the same code is
// compiled into the library (where the kernel calls bag_decode / bag_run_range) and into a host
// program that walks every workgroup number of a plan and checks that each bag is reduced once.
#pragma once

#include <cstddef>
#include <cstdint>

#include "fwdmi.h"

#if defined(__HIPCC__)
#define FWDMI_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define FWDMI_HD inline
#endif

namespace fwdmi {

constexpr int kMaxXcds = 8;        // accelerator complex dies (one L2 each) a launch plan can tell apart
constexpr int kWG = 256;           // lanes per workgroup (large batches; small ones use 128 or 64)
#ifndef FWDMI_BAG_IDX_BYTES
#define FWDMI_BAG_IDX_BYTES 16384
#endif
constexpr int kIdxBytes = FWDMI_BAG_IDX_BYTES;  // LDS bytes of the id window per workgroup (4096 row numbers / 2048 64-bit ids)
constexpr int kMaxBagsPerWG = 512;  // offsets staged in LDS per workgroup (+1)
constexpr int kLenBuckets = 256;    // bag-length buckets of the in-LDS counting sort
constexpr int kInlineTables = FWDMI_BAG_INLINE_TABLES;  // table descriptors that travel with the launch as kernel arguments
constexpr int kMaxVarTables = 64;   // tables of a launch whose runs may differ in size from table to table
constexpr int kBagLdsLimit = 64 * 1024;  // LDS a workgroup may ask for

// kMax also tracks the argmax (needs max_indices); kMaxValue is the plugin's case: values only
// kSumSq: the sum and the sum of squares of the same rows in one pass (two outputs)
enum Kind { kPlain = 0, kWeighted = 1, kMax = 2, kSquare = 3, kMaxValue = 4, kSumSq = 5 };

// What the device looks like to the plan.  `xcds` is the number of dies the hardware deals
// workgroups to in turn (workgroup b runs on die b % xcds); 1 when the device is one die or the
// runtime cannot tell.
struct BagTopology {
  int cus;
  int xcds;
};

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
  int32_t vec_store;  // 0: element stores; 1: 16-byte stores; 2: 16-byte stores with the non-temporal hint;
                      // 3: as 2 for 32 bytes of results per lane, halves traded between lanes first
  float one;  // 1.0f
  int32_t xcd_affinity;  // != 0: die x works through work items [xcd_start[x], xcd_start[x+1]); then the number of dies
  int32_t xcd_start[kMaxXcds + 1];
  int32_t total_wgs;
  int32_t tail_runs;  // XCD mapping only: the last `tail_runs` runs of every die's segment are issued as four workgroups each
  int32_t idx_cap;    // 32-bit words of the LDS id window: that many row numbers, or half as many 64-bit ids
  // Multi-table launches whose tables differ in mean bag length: table t's runs hold run_bags[t] bags and
  // are work items [run_start[t], run_start[t + 1]); bags_per_wg is then the largest of them (it sizes LDS).
  int32_t var_runs;
  int32_t run_start[kMaxVarTables + 1];
  uint16_t run_bags[kMaxVarTables];
};

static_assert(sizeof(BagLaunch) <= 4096, "kernel arguments are limited to 4 KiB");

// A launch, ready to be issued.
struct BagPlan {
  BagLaunch L;
  int grid, block;
  size_t lds;
  int kind;     // Kind
  bool f16;     // table rows are fp16 (else fp32)
  bool i64;     // ids / offsets are int64 (else int32)
  bool vec;     // rows are read as 16-byte slices
  bool ext;     // the launch needs the kernel variant that knows per-table run sizes / inline descriptors
  bool empty;   // nothing to launch (no bags)
};

// What one workgroup reduces: run `run` of table `table`, whole (quarter < 0) or one quarter of it.
struct BagWork {
  int table;
  int run;
  int run_bags;  // bags in a whole run of this table
  int quarter;
};

// Workgroup number -> its work.  False: the workgroup has nothing to do (padding of the per-die
// numbering).  EXT as in the kernel: launches without per-table run sizes leave that code out.
template <bool EXT>
FWDMI_HD bool bag_decode(const BagLaunch& L, uint32_t block, BagWork* w) {
  int work = (int)block;
  int quarter = -1;
  if (L.xcd_affinity) {
    // Undo the hardware's round-robin placement (workgroup b runs on die b % xcds) so that one die
    // works through whole tables.  A workgroup lives for about an eighth of the launch, so after a
    // die has started its last run its CUs empty out for that long.  The last runs of a segment are
    // therefore cut in four: their workgroups live a quarter as long and the die drains that much faster.
    const uint32_t xcds = (uint32_t)L.xcd_affinity;
    const int x = (int)(block % xcds);
    const int j = (int)(block / xcds);
    const int len = L.xcd_start[x + 1] - L.xcd_start[x];
    const int tail = len < L.tail_runs ? len : L.tail_runs;
    const int whole = len - tail;
    if (j < whole) {
      work = L.xcd_start[x] + j;
    } else {
      const int jj = j - whole;
      if (jj >= 4 * tail) return false;
      work = L.xcd_start[x] + whole + (jj >> 2);
      quarter = jj & 3;
    }
  }
  w->quarter = quarter;
  if (EXT && L.var_runs) {
    int t = 0;
    while (work >= L.run_start[t + 1]) ++t;  // at most kMaxVarTables steps over kernel arguments
    w->table = t;
    w->run = work - L.run_start[t];
    w->run_bags = L.run_bags[t];
  } else {
    const int t = work / L.wgs_per_table;
    w->table = t;
    w->run = work - t * L.wgs_per_table;
    w->run_bags = L.bags_per_wg;
  }
  return true;
}

// Bags [bag0, bag0 + nb) of the table that workgroup `w` reduces; nb <= 0: none (a quarter beyond
// the table's last bag).  The plan keeps run sizes multiples of 4 when it cuts runs.
FWDMI_HD void bag_run_range(const BagLaunch& L, const BagWork& w, int64_t* bag0, int* nb) {
  const int quarter_bags = w.run_bags >> 2;
  const int64_t first = (int64_t)w.run * w.run_bags + (w.quarter > 0 ? w.quarter * quarter_bags : 0);
  const int64_t want = w.quarter < 0 ? w.run_bags : quarter_bags;
  const int64_t left = L.n_bags - first;
  *bag0 = first;
  *nb = (int)(want < left ? want : left);
}

// Bytes of the kernel's LDS carve-up: offsets | ids | weights | lengths | order.
inline size_t bag_lds_bytes(const BagLaunch& L, bool weighted) {
  size_t b = (size_t)(L.bags_per_wg + 2) * sizeof(int64_t) + (size_t)L.idx_cap * sizeof(uint32_t);
  if (weighted) b += (size_t)L.idx_cap * sizeof(float);
  b += (size_t)L.bags_per_wg * (sizeof(int) + sizeof(uint16_t));
  return (b + 15) & ~(size_t)15;
}

// Validates the arguments of a launch and fills `plan`.  `tables_dev` non-null selects the
// multi-table form with descriptors in device memory, `tables_inline` (host, at most
// kInlineTables) the one whose descriptors travel as kernel arguments; with neither, `single` is
// the table.  Pure host arithmetic: no GPU call, pointers are only looked at for alignment.
// Returns FWDMI_OK or an error status with the text recorded for fwdmi_last_error().
int bag_plan(const fwdmi_bag_table* tables_dev, const fwdmi_bag_table* tables_inline, int n_tables,
             const fwdmi_bag_table& single, void* output, int64_t n_bags, int64_t fixed_len, int dim, int op,
             double avg_len, const fwdmi_bag_ext* ext, const BagTopology& topo, BagPlan* plan);

}  // namespace fwdmi
