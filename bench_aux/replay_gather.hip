// Measurement aid of bench.py, not part of the plugin path: replays the row-id stream of a multi-table bag
// workload as the simplest possible gather, to tell what the memory system charges for fetching
// those rows in that order from what the bag structure (lengths, ordering, per-bag results) adds.
//
// Same shape as the product kernel where it matters for memory behaviour: a 256-lane workgroup
// owns a contiguous chunk of one table's ids, copies them into LDS (16-byte loads), and sixteen 16-lane slots read
// 256-byte fp16 rows with 128-bit loads, eight in flight per lane, fp32 accumulation; workgroups
// are dealt to the eight XCDs in contiguous segments of the table-major work list.  There are no
// bags: a slot sums a contiguous part of the chunk and (optionally) stores a 256-byte result row
// every `store_every` rows, so the stored bytes can be made equal to the product's output.
#include <hip/hip_runtime.h>
#include <stdint.h>

#define FWDMI_MB_GLOBAL __attribute__((address_space(1)))

extern "C" {
struct fwdmi_mb_table {
  const void* data;  // [rows, 128] fp16
  const int32_t* ids;
};
struct fwdmi_mb_args {
  const fwdmi_mb_table* tables;  // device
  const int32_t* item_table;     // device [n_items]
  const int32_t* item_start;     // device [n_items]: first id of the chunk
  const int32_t* item_count;     // device [n_items]: ids in the chunk (at most 4096)
  void* out;                     // device: n_items * 16 slots * 64 rows * 256 bytes (4 MiB in all with store_mode 3)
  int32_t xcd_start[9];          // segment of the work list each XCD works through
  int32_t store_every;           // rows per stored result row; 0 = one result per slot at the end
  int32_t store_mode;            // 1 plain stores, 2 non-temporal stores, 3 plain stores into a 4 MiB region
  float one;                     // 1.0f
};
}

namespace {
typedef _Float16 Half8 __attribute__((ext_vector_type(8)));
typedef uint32_t U4 __attribute__((ext_vector_type(4)));
constexpr int kInFlight = 8;

__device__ __forceinline__ void store_row(Half8 FWDMI_MB_GLOBAL* p, Half8 r, int mode) {
  if (mode == 2) {
    U4 x;
    __builtin_memcpy(&x, &r, 16);
    // s_nop 1: the wait states a vector write to the data registers of a 128-bit store needs, which the
    // compiler does not insert behind an asm statement
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(p), "v"(x) : "memory");
  } else {
    *p = r;
  }
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(6))) void replay_gather_kernel(const fwdmi_mb_args A) {
  __shared__ uint32_t s_row[4096];
  const int x = blockIdx.x % 8;
  const int item = A.xcd_start[x] + blockIdx.x / 8;
  if (item >= A.xcd_start[x + 1]) return;
  const int t = A.item_table[item], s0 = A.item_start[item], n = min(A.item_count[item], 4096);
  const fwdmi_mb_table FWDMI_MB_GLOBAL* tp = (const fwdmi_mb_table FWDMI_MB_GLOBAL*)A.tables + t;
  const int32_t FWDMI_MB_GLOBAL* ids = (const int32_t FWDMI_MB_GLOBAL*)tp->ids;
  const char FWDMI_MB_GLOBAL* tab = (const char FWDMI_MB_GLOBAL*)tp->data;
  const int tid = threadIdx.x;
  {
    // 16-byte loads like the product kernel's staging pass; the ends of the chunk go id by id
    const int32_t FWDMI_MB_GLOBAL* first = ids + s0;
    const int head = min(n, (int)((4 - ((reinterpret_cast<uintptr_t>(first) >> 2) & 3)) & 3));
    const int n_vec = (n - head) / 4;
    for (int v = tid; v < n_vec; v += 256) {
      const U4 q = *(const U4 FWDMI_MB_GLOBAL*)(first + head + 4 * v);
#pragma unroll
      for (int e = 0; e < 4; ++e) s_row[head + 4 * v + e] = q[e];
    }
    if (tid < head) s_row[tid] = (uint32_t)first[tid];
    const int done = head + 4 * n_vec;
    if (done + tid < n) s_row[done + tid] = (uint32_t)first[done + tid];
  }
  __syncthreads();
  const int slot = tid >> 4, gl = tid & 15;
  const int per = (n + 15) / 16;
  int i = slot * per;
  const int end = min(n, i + per);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  const size_t region = A.store_mode == 3 ? (size_t)(item & 15) : (size_t)item;
  Half8 FWDMI_MB_GLOBAL* outp = (Half8 FWDMI_MB_GLOBAL*)A.out + (region * 16 + slot) * 16 * 64 + gl;
  int since = 0, nout = 0;
  for (; i + kInFlight <= end; i += kInFlight) {
    Half8 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) v[u] = *(const Half8 FWDMI_MB_GLOBAL*)(tab + (size_t)s_row[i + u] * 256 + gl * 16);
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf((float)v[u][e], A.one, acc[e]);
    if (A.store_every > 0) {
      since += kInFlight;
      if (since >= A.store_every) {
        Half8 r;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          r[e] = (_Float16)acc[e];
          acc[e] = 0.f;
        }
        store_row(&outp[(nout++ & 63) * 16], r, A.store_mode);
        since = 0;
      }
    }
  }
  for (; i < end; ++i) {
    const Half8 v = *(const Half8 FWDMI_MB_GLOBAL*)(tab + (size_t)s_row[i] * 256 + gl * 16);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf((float)v[e], A.one, acc[e]);
  }
  Half8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (_Float16)acc[e];
  store_row(&outp[(nout & 63) * 16], r, A.store_mode);
}
}  // namespace

// Launches one replay on `stream`; `grid_per_xcd` = items of the longest XCD segment.  Returns the
// hipError_t of the launch (0 = ok).
extern "C" int fwdmi_mb_replay_gather(const fwdmi_mb_args* args, int grid_per_xcd, void* stream) {
  if (!args || grid_per_xcd <= 0) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(replay_gather_kernel, dim3(grid_per_xcd * 8), dim3(256), 0, static_cast<hipStream_t>(stream), *args);
  return (int)hipGetLastError();
}
