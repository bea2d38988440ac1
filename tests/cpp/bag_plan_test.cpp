// Host-only check of the bag kernel's launch plan (forward_amd/csrc/kernels/bag_plan.{h,cpp}):
// walks every workgroup number of a plan through the same decode the kernel uses and asserts
// that every bag of every table is reduced exactly once, that nothing reaches past the tables'
// bags or the LDS carve-up, and that the per-die segments are what the plan says.
// Built with g++ and the address / undefined-behaviour sanitizers by tests/test_bag_plan.py.
#include <climits>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "../../forward_amd/csrc/kernels/bag_plan.h"

using namespace fwdmi;

static int g_failures = 0;
static long g_plans = 0;

#define EXPECT(cond, ...)                     \
  do {                                        \
    if (!(cond)) {                            \
      std::fprintf(stderr, "FAIL %s:%d: %s: ", __FILE__, __LINE__, #cond); \
      std::fprintf(stderr, __VA_ARGS__);      \
      std::fprintf(stderr, "\n");             \
      ++g_failures;                           \
      return;                                 \
    }                                         \
  } while (0)

struct Case {
  std::string name;
  int n_tables = 1;
  int64_t n_bags = 0;
  int dim = 128;
  int op = FWDMI_OP_SUM;
  double avg_len = 1.0;
  int table_dtype = FWDMI_F16, index_dtype = FWDMI_I32, out_dtype = FWDMI_F16;
  bool affinity = false, weights = false;
  std::vector<float> cost, len_hint;
  int64_t fixed_len = -1;
  int form = 1;  // 0 single table, 1 descriptors in device memory, 2 descriptors among the arguments
  int64_t single_rows = 1000;
  BagTopology topo{256, 8};
};

// Everything the kernel derives from a workgroup number, checked over the whole grid.
static void walk(const Case& c, const BagPlan& P) {
  const BagLaunch& L = P.L;
  const int n_tables = c.form == 0 ? 1 : c.n_tables;
  EXPECT(P.grid > 0 && P.block > 0, "%s: grid %d block %d", c.name.c_str(), P.grid, P.block);
  EXPECT(P.block == 64 || P.block == 128 || P.block == 256, "%s: block %d", c.name.c_str(), P.block);
  EXPECT((P.block >> L.log2_g) >= 1, "%s: no slot in a workgroup", c.name.c_str());
  EXPECT(L.n_slices >= 1 && (int64_t)L.n_slices * (1 << L.log2_g) * (P.vec ? 16 / (int)(P.f16 ? 2 : 4) : 1) >= c.dim,
         "%s: slices do not cover the row", c.name.c_str());
  EXPECT(P.lds <= (size_t)kBagLdsLimit, "%s: lds %zu", c.name.c_str(), P.lds);
  EXPECT(P.lds >= bag_lds_bytes(L, P.kind == kWeighted), "%s: lds smaller than the carve-up", c.name.c_str());
  EXPECT(L.bags_per_wg >= 1 && L.bags_per_wg <= kMaxBagsPerWG, "%s: bags_per_wg %d", c.name.c_str(), L.bags_per_wg);
  EXPECT(L.idx_cap >= 1 && (size_t)L.idx_cap * 4 <= (size_t)kIdxBytes, "%s: idx_cap %d", c.name.c_str(), L.idx_cap);
  EXPECT(L.n_bags == c.n_bags, "%s: n_bags", c.name.c_str());
  const int per_lane = P.vec ? (P.f16 ? 8 : 4) : 1;  // elements of a table row a lane holds
  EXPECT(L.vec_store >= 0 && L.vec_store <= 3 && (per_lane > 1 || L.vec_store == 0), "%s: vec_store %d with %d elements per lane",
         c.name.c_str(), L.vec_store, per_lane);
  if (L.vec_store == 3) {  // halves traded between the lanes of a slot: every lane of every slice must hold results
    const int g = 1 << L.log2_g;
    EXPECT(per_lane == 8 && !L.out_f16 && g >= 2 && c.dim == L.n_slices * g * 8,
           "%s: traded halves with %d elements per lane, fp16 results %d, slots of %d lanes, %d slices for %d columns",
           c.name.c_str(), per_lane, (int)L.out_f16, g, L.n_slices, c.dim);
  }
  if (L.var_runs) {
    EXPECT(P.ext, "%s: per-table run sizes need the extended kernel", c.name.c_str());
    EXPECT(L.run_start[0] == 0 && L.run_start[n_tables] == L.total_wgs, "%s: run_start ends", c.name.c_str());
    for (int t = 0; t < n_tables; ++t) {
      EXPECT(L.run_bags[t] >= 1 && L.run_bags[t] <= L.bags_per_wg, "%s: run_bags[%d]=%d", c.name.c_str(), t, L.run_bags[t]);
      const int64_t runs = (c.n_bags + L.run_bags[t] - 1) / L.run_bags[t];
      EXPECT(L.run_start[t + 1] - L.run_start[t] == runs, "%s: table %d has %d runs, needs %lld", c.name.c_str(), t,
             L.run_start[t + 1] - L.run_start[t], (long long)runs);
    }
  } else {
    EXPECT((int64_t)L.wgs_per_table * L.bags_per_wg >= c.n_bags, "%s: runs do not cover the bags", c.name.c_str());
    EXPECT((int64_t)L.wgs_per_table * n_tables == L.total_wgs, "%s: total_wgs", c.name.c_str());
  }
  const int xcds = L.xcd_affinity;
  if (xcds) {
    EXPECT(xcds >= 2 && xcds <= kMaxXcds && xcds == c.topo.xcds, "%s: %d dies in the plan", c.name.c_str(), xcds);
    EXPECT(L.xcd_start[0] == 0 && L.xcd_start[xcds] == L.total_wgs, "%s: xcd_start ends", c.name.c_str());
    for (int k = 0; k < xcds; ++k)
      EXPECT(L.xcd_start[k] <= L.xcd_start[k + 1], "%s: xcd_start not monotone at %d", c.name.c_str(), k);
    EXPECT(P.grid % xcds == 0, "%s: grid %d not a multiple of the dies", c.name.c_str(), P.grid);
    if (L.tail_runs > 0) {
      EXPECT(L.bags_per_wg % 4 == 0, "%s: quarter runs of %d bags", c.name.c_str(), L.bags_per_wg);
      for (int t = 0; L.var_runs && t < n_tables; ++t)
        EXPECT(L.run_bags[t] % 4 == 0, "%s: quarter runs of %d bags (table %d)", c.name.c_str(), L.run_bags[t], t);
    }
  } else {
    EXPECT(P.grid == L.total_wgs, "%s: grid %d for %d runs", c.name.c_str(), P.grid, L.total_wgs);
  }
  std::vector<uint8_t> seen((size_t)n_tables * (size_t)c.n_bags, 0);
  for (uint32_t b = 0; b < (uint32_t)P.grid; ++b) {
    BagWork w;
    const bool live = P.ext ? bag_decode<true>(L, b, &w) : bag_decode<false>(L, b, &w);
    if (!live) {
      EXPECT(xcds != 0, "%s: an idle workgroup without the per-die numbering", c.name.c_str());
      continue;
    }
    EXPECT(w.table >= 0 && w.table < n_tables, "%s: block %u -> table %d", c.name.c_str(), b, w.table);
    EXPECT(w.run >= 0 && w.quarter >= -1 && w.quarter <= 3, "%s: block %u", c.name.c_str(), b);
    EXPECT(w.run_bags >= 1 && w.run_bags <= L.bags_per_wg, "%s: block %u run of %d bags (LDS holds %d)", c.name.c_str(), b,
           w.run_bags, L.bags_per_wg);
    if (xcds) {  // a workgroup works inside its die's segment
      const int x = (int)(b % (uint32_t)xcds);
      const int work = L.var_runs ? L.run_start[w.table] + w.run : w.table * L.wgs_per_table + w.run;
      EXPECT(work >= L.xcd_start[x] && work < L.xcd_start[x + 1], "%s: block %u of die %d reduces run %d outside [%d, %d)",
             c.name.c_str(), b, x, work, L.xcd_start[x], L.xcd_start[x + 1]);
    }
    int64_t bag0;
    int nb;
    bag_run_range(L, w, &bag0, &nb);
    EXPECT(bag0 >= 0, "%s: block %u starts at bag %lld", c.name.c_str(), b, (long long)bag0);
    if (w.quarter < 0) EXPECT(nb >= 1, "%s: block %u: a whole run without bags", c.name.c_str(), b);
    for (int i = 0; i < nb; ++i) {
      const int64_t bag = bag0 + i;
      EXPECT(bag < c.n_bags, "%s: block %u reaches bag %lld of %lld", c.name.c_str(), b, (long long)bag, (long long)c.n_bags);
      uint8_t& s = seen[(size_t)w.table * (size_t)c.n_bags + (size_t)bag];
      EXPECT(s == 0, "%s: bag %lld of table %d reduced twice (block %u)", c.name.c_str(), (long long)bag, w.table, b);
      s = 1;
    }
  }
  for (size_t i = 0; i < seen.size(); ++i)
    EXPECT(seen[i] == 1, "%s: bag %zu of table %zu never reduced", c.name.c_str(), i % (size_t)c.n_bags, i / (size_t)c.n_bags);
}

static int make_plan(const Case& c, BagPlan* P) {
  static const int dummy[64] = {};  // pointers are only looked at for alignment
  alignas(16) static char out[16];
  std::vector<fwdmi_bag_table> tabs((size_t)c.n_tables);
  for (int t = 0; t < c.n_tables; ++t)
    tabs[(size_t)t] = fwdmi_bag_table{dummy, dummy, dummy, 1000 + t, (int64_t)(c.avg_len * (double)c.n_bags), 0,
                                      (int64_t)t * c.dim, nullptr};
  fwdmi_bag_ext x{};
  x.table_dtype = c.table_dtype;
  x.index_dtype = c.index_dtype;
  x.out_dtype = c.out_dtype;
  x.out_row_stride = c.form == 0 ? 0 : (int64_t)c.n_tables * c.dim;
  x.flags = (c.affinity ? FWDMI_BAG_XCD_TABLE_AFFINITY : 0) | (c.weights && c.form != 0 ? FWDMI_BAG_TABLE_WEIGHTS : 0) |
            (c.len_hint.empty() ? 0 : FWDMI_BAG_TABLE_AVG_LEN);
  x.table_cost = c.cost.empty() ? nullptr : c.cost.data();
  x.table_avg_len = c.len_hint.empty() ? nullptr : c.len_hint.data();
  if (c.weights && c.form == 0) x.per_sample_weights = dummy;
  fwdmi_bag_table single{dummy, dummy, dummy, c.single_rows, (int64_t)(c.avg_len * (double)c.n_bags), 0, 0, nullptr};
  const fwdmi_bag_table* dev = c.form == 1 ? reinterpret_cast<const fwdmi_bag_table*>(dummy) : nullptr;
  const fwdmi_bag_table* inl = c.form == 2 ? tabs.data() : nullptr;
  ++g_plans;
  return bag_plan(dev, inl, c.form == 0 ? 1 : c.n_tables, single, out, c.n_bags, c.fixed_len, c.dim, c.op, c.avg_len, &x,
                  c.topo, P);
}

static void run_case(const Case& c) {
  BagPlan P;
  const int rc = make_plan(c, &P);
  EXPECT(rc == FWDMI_OK, "%s: bag_plan returned %d (%s)", c.name.c_str(), rc, fwdmi_last_error());
  if (c.n_bags == 0) {
    EXPECT(P.empty, "%s: no bags, but a launch", c.name.c_str());
    return;
  }
  EXPECT(!P.empty, "%s: bags, but no launch", c.name.c_str());
  walk(c, P);
}

static void expect_error(const Case& c, const char* text) {
  BagPlan P;
  const int rc = make_plan(c, &P);
  EXPECT(rc != FWDMI_OK, "%s: accepted", c.name.c_str());
  EXPECT(std::strstr(fwdmi_last_error(), text) != nullptr, "%s: error text '%s' lacks '%s'", c.name.c_str(),
         fwdmi_last_error(), text);
}

int main() {
  // the 26-table configuration the benchmark runs: equal bag lengths, per-table costs, eight dies
  {
    Case c;
    c.name = "config4";
    c.n_tables = 26;
    c.n_bags = 65536;
    c.avg_len = 16.32;
    c.affinity = true;
    for (int t = 0; t < 26; ++t) c.cost.push_back(1.0f + 0.45f * (float)(t % 5) / 4.0f);
    for (int t = 0; t < 26; ++t) c.len_hint.push_back(16.0f + 0.05f * (float)t);
    run_case(c);
    BagPlan P;
    if (make_plan(c, &P) == FWDMI_OK) {
      if (P.L.bags_per_wg != 112 || P.L.tail_runs != 48 || P.L.xcd_affinity != 8 || P.L.var_runs || P.ext) {
        std::fprintf(stderr, "FAIL config4 plan changed: %d bags per run, %d tail runs, %d dies, var_runs %d\n", P.L.bags_per_wg,
                     P.L.tail_runs, P.L.xcd_affinity, P.L.var_runs);
        ++g_failures;
      }
    }
    // the same stage on other devices: one die (a compute partition), four dies, more dies than the plan knows
    const BagTopology topos[] = {{32, 1}, {128, 4}, {64, 2}, {304, 8}, {256, 16}, {80, 8}, {8, 8}, {4, 8}};
    for (const BagTopology& tp : topos) {
      Case d = c;
      d.topo = tp;
      d.name = "config4 on " + std::to_string(tp.cus) + " CUs / " + std::to_string(tp.xcds) + " dies";
      run_case(d);
      BagPlan Q;
      if (make_plan(d, &Q) == FWDMI_OK) {
        const bool want_affinity = tp.xcds >= 2 && tp.xcds <= kMaxXcds && tp.cus >= tp.xcds;
        if ((Q.L.xcd_affinity != 0) != want_affinity || (want_affinity && Q.L.xcd_affinity != tp.xcds)) {
          std::fprintf(stderr, "FAIL %s: per-die numbering %d\n", d.name.c_str(), Q.L.xcd_affinity);
          ++g_failures;
        }
      }
    }
    // one-hot tables beside long-bag tables: runs sized per table
    Case m = c;
    m.name = "mixed bag lengths";
    m.len_hint.clear();
    for (int t = 0; t < 26; ++t) m.len_hint.push_back(t % 2 ? 32.6f : 1.0f);
    m.avg_len = 16.8;
    run_case(m);
    BagPlan Q;
    if (make_plan(m, &Q) == FWDMI_OK && !Q.L.var_runs) {
      std::fprintf(stderr, "FAIL mixed bag lengths: expected per-table run sizes\n");
      ++g_failures;
    }
    m.form = 2;
    m.name = "mixed bag lengths, descriptors among the arguments";
    run_case(m);
    m.weights = true;
    m.name += ", weighted";
    run_case(m);
  }
  // 1 .. 70 tables, ragged batch sizes, with and without length hints / per-die numbering / weights
  std::mt19937_64 rng(20251);
  auto uni = [&](int lo, int hi) { return lo + (int)(rng() % (uint64_t)(hi - lo + 1)); };
  const int64_t batch_sizes[] = {1, 2, 3, 5, 63, 64, 65, 127, 509, 1000, 4096, 4099, 20011, 65536, 100003};
  const int dims[] = {1, 3, 8, 16, 32, 64, 100, 128, 256, 512, 768, 1024, 2048, 5000};
  const BagTopology topos[] = {{256, 8}, {256, 8}, {256, 8}, {32, 1}, {128, 4}, {64, 2}, {304, 8}, {256, 16}, {1, 1}, {7, 7}};
  for (int n_tables = 1; n_tables <= 70; ++n_tables) {
    for (int rep = 0; rep < 12; ++rep) {
      Case c;
      c.n_tables = n_tables;
      c.n_bags = batch_sizes[rng() % (sizeof(batch_sizes) / sizeof(batch_sizes[0]))];
      if ((int64_t)n_tables * c.n_bags > 3000000) c.n_bags = 3000000 / n_tables;
      c.dim = dims[rng() % (sizeof(dims) / sizeof(dims[0]))];
      c.table_dtype = uni(0, 1) ? FWDMI_F16 : FWDMI_F32;
      c.out_dtype = uni(0, 1) ? FWDMI_F16 : FWDMI_F32;
      c.index_dtype = uni(0, 1) ? FWDMI_I64 : FWDMI_I32;
      const int ops[] = {FWDMI_OP_SUM, FWDMI_OP_SUM, FWDMI_OP_MEAN, FWDMI_OP_MAX, FWDMI_OP_SQUARE_SUM};
      c.op = ops[rng() % 5];
      c.weights = c.op == FWDMI_OP_SUM && uni(0, 3) == 0;
      c.avg_len = std::exp(std::log(300.0) * (double)(rng() % 1000) / 1000.0) - 0.5;  // 0.5 .. 300
      c.affinity = uni(0, 2) != 0;
      c.form = n_tables == 1 ? uni(0, 2) : (n_tables <= kInlineTables ? uni(1, 2) : 1);
      c.topo = topos[rng() % (sizeof(topos) / sizeof(topos[0]))];
      if (uni(0, 1)) {
        for (int t = 0; t < n_tables; ++t) c.cost.push_back(1.0f + 0.45f * (float)(rng() % 100) / 100.0f);
      }
      const int hints = uni(0, 3);  // none, equal, mixed, wild
      for (int t = 0; hints && t < n_tables; ++t) {
        const double a = hints == 1 ? c.avg_len : hints == 2 ? (t % 2 ? 2.0 * c.avg_len : 1.0) : std::exp(std::log(400.0) * (double)(rng() % 1000) / 1000.0) - 1.0;
        c.len_hint.push_back((float)a);
      }
      if (c.form == 0 && uni(0, 3) == 0) {
        c.fixed_len = uni(0, 40);
        c.avg_len = (double)c.fixed_len;
      }
      if (c.form == 0 && uni(0, 5) == 0) c.single_rows = (int64_t)1 << 25;  // beyond 32-bit row numbers: 64-bit id window
      c.name = "random " + std::to_string(n_tables) + " tables #" + std::to_string(rep) + " (" + std::to_string(c.n_bags) +
               " bags, dim " + std::to_string(c.dim) + ", form " + std::to_string(c.form) + ", avg " + std::to_string(c.avg_len) +
               ", " + std::to_string(c.topo.cus) + "/" + std::to_string(c.topo.xcds) + ")";
      run_case(c);
    }
  }
  // hints that are not numbers are harmless (avg_len) or refused (per-table arrays)
  {
    Case c;
    c.name = "avg_len NaN";
    c.n_tables = 4;
    c.n_bags = 1000;
    c.avg_len = std::nan("");
    run_case(c);
    c.avg_len = 1e300;
    c.name = "avg_len huge";
    run_case(c);
    c.avg_len = -5.0;
    c.name = "avg_len negative";
    run_case(c);
    c.avg_len = 8.0;
    c.n_bags = 0;
    c.name = "no bags";
    run_case(c);
    c.n_bags = 1000;
    c.len_hint = {1.0f, std::nanf(""), 2.0f, 3.0f};
    c.name = "table_avg_len NaN";
    expect_error(c, "table_avg_len");
    c.len_hint = {1.0f, -1.0f, 2.0f, 3.0f};
    c.name = "table_avg_len negative";
    expect_error(c, "table_avg_len");
    c.len_hint.clear();
    c.affinity = true;
    c.cost = {1.0f, 0.0f, 1.0f, 1.0f};
    c.name = "table_cost zero";
    expect_error(c, "table_cost");
    c.cost = {1.0f, std::nanf(""), 1.0f, 1.0f};
    c.name = "table_cost NaN";
    expect_error(c, "table_cost");
    c.cost.clear();
    c.topo = BagTopology{0, 8};
    c.name = "device without CUs";
    expect_error(c, "CUs");
    c.topo = BagTopology{256, 8};
    c.form = 2;
    c.n_tables = kInlineTables + 1;
    c.name = "too many inline tables";
    expect_error(c, "do not fit");
  }
  // Arguments at the ends of their types, in every combination the generator hits: the plan either
  // refuses them with a reason or is a plan; the sanitizers this file is built with see any signed
  // overflow, out-of-range conversion or read past an array on the way.
  {
    static const int dummy[64] = {};
    alignas(16) static char out[16];
    const int64_t bags[] = {-1, 0, 1, 7, 65536, 2147483647, 2147483648ll, (int64_t)1 << 40, (int64_t)1 << 62, INT64_MAX};
    const int64_t lens[] = {-1, -1, -1, 0, 1, 40, 2147483648ll, (int64_t)1 << 62, INT64_MAX};
    const int dims[] = {-1, 0, 1, 8, 128, 1 << 20, 1 << 30, INT32_MAX};
    const int tables[] = {-1, 0, 1, 2, 26, 64, 65, 1024, 2048, 100000, INT32_MAX};
    const double avgs[] = {std::nan(""), INFINITY, -INFINITY, 0.0, 1.0, 16.0, 1e308, -1e308, 5e-324};
    const int ops[] = {-1, 0, 1, 2, 3, 4, 999, 12345, INT32_MAX};
    const int types[] = {FWDMI_F32, FWDMI_F16, FWDMI_I8, FWDMI_I32, FWDMI_I64, -1, 77};
    const int64_t strides[] = {0, 0, 1, 128, 3328, -5, (int64_t)1 << 40, INT64_MAX};
    const int cus[] = {-1, 0, 1, 32, 256, 304, 1 << 30, INT32_MAX}, xcds[] = {-1, 0, 1, 2, 8, 9, 1 << 30};
    long refused = 0, planned = 0;
    std::vector<float> ones(2048, 1.0f), wild(2048);
    for (size_t i = 0; i < wild.size(); ++i) wild[i] = (i % 5 == 0) ? 3e38f : (float)(i % 300);
#define ANY(a) a[rng() % (sizeof(a) / sizeof(a[0]))]
    // mostly plausible values, so that the extreme ones get past the first checks one or two at a time
    const int64_t sane_bags[] = {1, 7, 1000, 65536, 3000000}, sane_lens[] = {-1, -1, -1, 0, 1, 40}, sane_strides[] = {0, 0, 0, 1 << 20};
    const int sane_dims[] = {1, 8, 64, 128, 1000, 4096}, sane_tables[] = {1, 2, 26, 40, 41, 64, 65, 700};
    const double sane_avgs[] = {0.5, 1.0, 16.3, 300.0};
    const int sane_ops[] = {0, 0, 1, 2, 3}, sane_types[] = {FWDMI_F32, FWDMI_F16}, sane_cus[] = {256, 256, 32, 304}, sane_xcds[] = {8, 8, 1, 4};
#define PICK(a) (uni(0, 5) ? ANY(sane_##a) : ANY(a))
    for (int it = 0; it < 200000; ++it) {
      const int n_tables = PICK(tables), form = uni(0, 2);
      fwdmi_bag_ext x{};
      x.table_dtype = PICK(types);
      x.index_dtype = uni(0, 3) ? (uni(0, 1) ? FWDMI_I32 : FWDMI_I64) : PICK(types);
      x.out_dtype = uni(0, 3) ? (uni(0, 1) ? FWDMI_F32 : FWDMI_F16) : PICK(types);
      x.include_last_offset = uni(0, 2) - 1;
      x.out_row_stride = PICK(strides);
      x.flags = uni(0, 7);
      const bool arrays_fit = n_tables > 0 && n_tables <= 2048;
      if (arrays_fit && uni(0, 1)) x.table_cost = uni(0, 1) ? ones.data() : wild.data();
      if (arrays_fit && (x.flags & FWDMI_BAG_TABLE_AVG_LEN) && uni(0, 1)) x.table_avg_len = uni(0, 1) ? ones.data() : wild.data();
      if (!arrays_fit) x.flags &= ~FWDMI_BAG_TABLE_AVG_LEN, x.table_avg_len = nullptr;
      if (uni(0, 5) == 0) x.per_sample_weights = dummy;
      if (uni(0, 5) == 0) x.max_indices = out;
      if (uni(0, 5) == 0) x.square_sum_out = out;
      fwdmi_bag_table single{uni(0, 9) ? dummy : nullptr, uni(0, 9) ? dummy : nullptr, uni(0, 9) ? dummy : nullptr,
                             PICK(bags), PICK(bags), PICK(lens), PICK(strides), nullptr};
      std::vector<fwdmi_bag_table> inl;
      if (form == 2 && n_tables > 0 && n_tables <= kInlineTables) inl.assign((size_t)n_tables, single);
      const fwdmi_bag_table* dev = form == 1 ? reinterpret_cast<const fwdmi_bag_table*>(dummy) : nullptr;
      const BagTopology tp{PICK(cus), PICK(xcds)};
      BagPlan P;
      const int rc = bag_plan(dev, inl.empty() ? nullptr : inl.data(), form == 0 ? 1 : n_tables, single, uni(0, 9) ? out : nullptr,
                              PICK(bags), PICK(lens), PICK(dims), PICK(ops), PICK(avgs), uni(0, 9) ? &x : nullptr, tp, &P);
      if (rc != FWDMI_OK) {
        ++refused;
        if (fwdmi_last_error()[0] == '\0') {
          std::fprintf(stderr, "FAIL extreme arguments #%d: refused without a reason\n", it);
          ++g_failures;
        }
      } else {
        ++planned;
        if (!P.empty && (P.grid <= 0 || P.block <= 0 || P.lds > (size_t)kBagLdsLimit)) {
          std::fprintf(stderr, "FAIL extreme arguments #%d: grid %d block %d lds %zu\n", it, P.grid, P.block, P.lds);
          ++g_failures;
        }
      }
    }
#undef PICK
#undef ANY
    std::printf("extreme arguments: %ld refused, %ld planned\n", refused, planned);
  }
  std::printf("%ld plans walked, %d failures\n", g_plans, g_failures);
  return g_failures ? 1 : 0;
}
