// Launch plan of the bag-reduction kernel (see bag_plan.h): lane mapping, run sizes, LDS window,
// per-die segments of the table-major work list.  Host arithmetic only.
#include "bag_plan.h"

#include <algorithm>
#include <climits>
#include <cmath>

#include "../status.h"

#ifndef FWDMI_BAG_STREAM_BYTES
#define FWDMI_BAG_STREAM_BYTES (8.0 * 1048576.0)  // results of at least this size are stored with the non-temporal hint
#endif
#ifndef FWDMI_BAG_TAIL_RUNS
#define FWDMI_BAG_TAIL_RUNS(resident) ((resident) / 4)  // measured best on the 26-table configuration (16 .. 384 tried)
#endif

namespace fwdmi {
namespace {

int next_pow2(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

const fwdmi_bag_ext kDefaultExt = {FWDMI_F32, FWDMI_I32, FWDMI_F32, 0, nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, nullptr};

}  // namespace

int bag_plan(const fwdmi_bag_table* tables_dev, const fwdmi_bag_table* tables_inline, int n_tables,
             const fwdmi_bag_table& single, void* output, int64_t n_bags, int64_t fixed_len, int dim, int op,
             double avg_len, const fwdmi_bag_ext* ext, const BagTopology& topo, BagPlan* plan) {
  const bool multi = tables_dev || tables_inline;
  const fwdmi_bag_ext& x = ext ? *ext : kDefaultExt;
  // Per-table mean bag lengths are read only when the flag announces them: a caller built against
  // a header whose struct ends before that member never sets the bit.
  const float* const table_avg_len = (x.flags & FWDMI_BAG_TABLE_AVG_LEN) ? x.table_avg_len : nullptr;

  if (!is_float_dtype(x.table_dtype) || !is_float_dtype(x.out_dtype) || !is_index_dtype(x.index_dtype))
    return set_error(FWDMI_ERR_UNSUPPORTED, "embedding bag: unsupported dtype (table %d, index %d, out %d)",
                     x.table_dtype, x.index_dtype, x.out_dtype);
  if (op != FWDMI_OP_SUM && op != FWDMI_OP_MEAN && op != FWDMI_OP_MAX && op != FWDMI_OP_SQUARE_SUM)
    return set_error(FWDMI_ERR_UNSUPPORTED, "embedding bag: unknown op %d", op);
  // dim: a row's byte size and a run's (bag, slice) count stay far inside 32 bits
  // n_tables: the per-table passes below stay short whatever a caller passes
  FWDMI_REQUIRE(n_bags >= 0 && dim > 0 && dim <= (1 << 24) && n_tables > 0 && n_tables <= (1 << 20),
                "embedding bag: n_bags=%lld dim=%d (1 .. 2^24) n_tables=%d (1 .. 2^20)", (long long)n_bags, dim, n_tables);
  FWDMI_REQUIRE(!(x.per_sample_weights || (multi && (x.flags & FWDMI_BAG_TABLE_WEIGHTS))) || op == FWDMI_OP_SUM,
                "embedding bag: per_sample_weights needs op SUM (got %d)", op);
  FWDMI_REQUIRE(!x.max_indices || (op == FWDMI_OP_MAX && !multi),
                "embedding bag: max_indices needs op MAX on a single table");
  const int64_t out_stride = x.out_row_stride > 0 ? x.out_row_stride : dim;
  FWDMI_REQUIRE(out_stride >= dim, "embedding bag: out_row_stride %lld < dim %d", (long long)out_stride, dim);
  FWDMI_REQUIRE(topo.cus > 0 && topo.xcds > 0, "embedding bag: device of %d CUs on %d dies", topo.cus, topo.xcds);
  plan->empty = n_bags == 0;
  if (n_bags == 0) return FWDMI_OK;
  FWDMI_REQUIRE(output != nullptr, "embedding bag: null output");
  if (!multi) {
    FWDMI_REQUIRE(single.count > 0 && single.data, "embedding bag: empty table");
    FWDMI_REQUIRE(single.input_size >= 0 && (single.input_size == 0 || single.input),
                  "embedding bag: null ids");
    FWDMI_REQUIRE(fixed_len >= 0 || single.input_2, "embedding bag: null offsets");
    FWDMI_REQUIRE(single.out_col >= 0 && single.out_col <= out_stride - dim, "embedding bag: out_col");
  }

  const size_t sw = dtype_size(x.table_dtype), so = dtype_size(x.out_dtype);
  const int vec_w = (int)(16 / sw);
  // 128-bit row loads need 16-byte row pitch and base; a multi-table launch is checked by its caller.
  bool vec = (dim % vec_w) == 0;
  if (!multi) vec = vec && (reinterpret_cast<uintptr_t>(single.data) % 16) == 0;
  const int VEC = vec ? vec_w : 1;

  BagLaunch& L = plan->L;
  L = BagLaunch{};
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
  // a sizing hint only: anything that is not a number of at least one id (NaN included) counts as
  // one, and no hint is worth more than the longest bag a 32-bit id count allows
  if (!(avg_len >= 1.0)) avg_len = 1.0;
  avg_len = std::min(avg_len, 2147483647.0);
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
  FWDMI_REQUIRE(n_bags <= INT64_MAX / n_tables, "embedding bag: %lld bags x %d tables", (long long)n_bags, n_tables);
  const int64_t total_bags = n_bags * n_tables;
  const int64_t target_wgs = (int64_t)topo.cus * 4;
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
    // the 26-table configuration: 0.490 -> 0.440 ms together with the register budget of the weighted kernel.
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
  if (table_avg_len) {
    for (int t = 0; t < n_tables; ++t) {
      const double a = (double)table_avg_len[t];
      FWDMI_REQUIRE(a >= 0.0 && a < 1e30, "embedding bag: table_avg_len must be finite and not negative");
    }
  }
  if (multi && table_avg_len && n_tables > 1 && n_tables <= kMaxVarTables) {
    const int64_t want_all = std::min<int64_t>(std::max<int64_t>(1, total_bags / target_wgs), kMaxBagsPerWG);
    int lo = INT_MAX, hi = 0, cap_max = 0;
    for (int t = 0; t < n_tables; ++t) {
      const double avg_t = std::max(1.0, (double)table_avg_len[t]);
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
  auto runs_of = [&](int per_run) { return n_bags / per_run + (n_bags % per_run != 0); };  // no sum that could overflow
  const int64_t wgs = runs_of(L.bags_per_wg);
  FWDMI_REQUIRE(wgs < (int64_t)1 << 31 && wgs * n_tables < (int64_t)1 << 31, "embedding bag: grid too large");
  L.wgs_per_table = (int)wgs;
  int64_t total_runs = wgs * n_tables;
  L.var_runs = 0;
  if (var_runs) {
    total_runs = 0;
    for (int t = 0; t < n_tables; ++t) {
      L.run_start[t] = (int32_t)total_runs;
      L.run_bags[t] = (uint16_t)run_bags[t];
      const int64_t runs_t = runs_of(run_bags[t]);
      FWDMI_REQUIRE(runs_t < (int64_t)1 << 31, "embedding bag: grid too large");
      total_runs += runs_t;
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

  // A result of several MiB does not survive in the 4 MiB L2 of the die that wrote it until somebody
  // reads it (and a reader on another die would not find it there anyway); written with the
  // non-temporal hint it does not displace table rows on its way out.  Measured: 2.8 % off the
  // 26-table launch (19 % when every row hits in cache), 3.8 % off 26 single-table launches of
  // 16 MiB results each; a reader of a 16 MiB result right behind the launch costs 2 % more.
  if (L.vec_store && (double)n_bags * n_tables * dim * so >= FWDMI_BAG_STREAM_BYTES) L.vec_store = 2;
  // Eight fp32 results per lane (fp16 table, fp32 output) leave in two 16-byte stores; with every
  // column slice full the lanes of a slot trade halves first, so that each store instruction writes
  // contiguous bytes instead of every other 16 (measured on the 26-table launch: 0.595 -> 0.535 ms).
  if (L.vec_store == 2 && VEC * so == 32 && lanes >= 2 && dim % (lanes * VEC) == 0) L.vec_store = 3;

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
  // The per-die mapping rests on the hardware dealing workgroup b to die b % xcds: it is used where the
  // device says how many dies it has and the plan can tell them apart; a device of one die (a compute
  // partition) or of more dies than the plan knows keeps the plain table-major order.
  const int xcds = topo.xcds;
  if (multi && n_tables > 1 && (x.flags & FWDMI_BAG_XCD_TABLE_AFFINITY) && xcds >= 2 && xcds <= kMaxXcds &&
      topo.cus >= xcds) {
    // Cut the table-major work list into one contiguous segment per die, of equal estimated cost
    // (equal length when the caller gives no per-table cost).
    L.xcd_affinity = xcds;
    // A bag costs its rows plus a constant (result store, bookkeeping) worth kBagRows rows: fixed-length
    // launches of 1 .. 64 rows per bag fit rows / 36.6 TB/s + result bytes / 3.7 TB/s, and one-hot
    // tables beside tables of 33 ids per bag measure 1 : 4.1 per bag.  With every table's mean bag
    // length known the caller's per-bag cost is scaled by it; without, all tables count as equally long.
    constexpr double kBagRows = 9.6;
    auto cost_of = [&](int u) {
      double c = x.table_cost ? (double)x.table_cost[u] : 1.0;
      if (table_avg_len) c *= (std::max(0.0, (double)table_avg_len[u]) + kBagRows) / (avg_len + kBagRows);
      return c;
    };
    double total = 0.0;
    for (int t = 0; t < n_tables; ++t) {
      const double c = cost_of(t);
      FWDMI_REQUIRE(c > 0.0 && c < 1e30, "embedding bag: table_cost must be positive and finite");
      total += c * (double)wgs;
    }
    int t = 0;
    double before = 0.0;  // cost of the tables before t
    int longest = 0;
    L.xcd_start[0] = 0;
    if (var_runs) {
      // the same cut with runs whose size differs from table to table: a table's cost is its bags' cost
      double all = 0.0;
      for (int u = 0; u < n_tables; ++u) all += cost_of(u) * (double)n_bags;
      for (int k = 1; k <= xcds; ++k) {
        int cut = grid;
        if (k < xcds) {
          const double target = all * k / xcds;
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
      for (int k = 1; k <= xcds; ++k) {
        int cut = grid;
        if (k < xcds) {
          const double target = total * k / xcds;
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
    // Runs cut in four at the end of every segment (see bag_decode): as many as a quarter of what a die holds
    // at once, and only in launches that fill the chip several times over.
    const int resident = topo.cus / xcds * 6;  // workgroups of 256 lanes a die holds at the 6-per-CU occupancy
    L.tail_runs = 0;
    bool can_cut = block == kWG && L.bags_per_wg % 4 == 0 && L.bags_per_wg / 4 >= slots;
    for (int u = 0; var_runs && u < n_tables; ++u) can_cut = can_cut && run_bags[u] % 4 == 0 && run_bags[u] / 4 >= slots;
    if (can_cut && longest >= 4 * resident) L.tail_runs = FWDMI_BAG_TAIL_RUNS(resident);
    int most = 0;  // workgroups of the die with the most
    for (int k = 0; k < xcds; ++k) {
      const int len = L.xcd_start[k + 1] - L.xcd_start[k];
      most = std::max(most, len + 3 * std::min(len, L.tail_runs));
    }
    FWDMI_REQUIRE((int64_t)most * xcds < (int64_t)1 << 31, "embedding bag: grid too large");
    grid = most * xcds;
  }
  plan->grid = grid;
  plan->block = block;
  plan->lds = bag_lds_bytes(L, kind == kWeighted);
  FWDMI_REQUIRE(plan->lds <= (size_t)kBagLdsLimit, "embedding bag: a run needs %zu bytes of LDS", plan->lds);
  plan->kind = kind;
  plan->f16 = x.table_dtype == FWDMI_F16;
  plan->i64 = i64_ids;
  plan->vec = vec;
  plan->ext = L.var_runs || (L.multi && !L.tables);  // per-table run sizes, or descriptors among the arguments
  return FWDMI_OK;
}

}  // namespace fwdmi
