// Measurement aid of bench.py, not part of the plugin path: the bag-free replay of a multi-table id
// stream (see replay_gather.hip) with the hottest rows of every table served from LDS instead of
// through the vector L1.  The host names each table's K hottest rows and rearranges every
// workgroup's chunk into the ids of its other rows followed by one LDS slot number per fetch of a
// hot row; the kernel copies the K rows into LDS once per workgroup, gathers the first part from
// the table with 128-bit loads (eight in flight per lane) and reads the second part from LDS
// (`ds_read_b128`, eight in flight per lane).  What it measures is an upper bound for such a cache
// in a bag reduction: the split is free here and no bag boundary constrains either loop.
#include <hip/hip_runtime.h>
#include <stdint.h>

#define FWDMI_MB_GLOBAL __attribute__((address_space(1)))

extern "C" {
struct fwdmi_mb_hot_table {
  const void* data;    // [rows, 128] fp16
  const int32_t* ids;  // the rearranged stream: per chunk, table row numbers, then LDS slot numbers
  const int32_t* hot;  // [n_hot] row numbers of the table's hottest rows (slot k holds row hot[k])
};
struct fwdmi_mb_hot_args {
  const fwdmi_mb_hot_table* tables;  // device
  const int32_t* item_table;         // device [n_items]
  const int32_t* item_start;         // device [n_items]: first entry of the chunk
  const int32_t* item_count;         // device [n_items]: entries in the chunk (at most 2048)
  const int32_t* item_hot;           // device [n_items]: how many of them, at the end, are LDS slot numbers
  void* out;                         // device: n_items * 16 slots * 64 rows * 256 bytes
  int32_t xcd_start[9];
  int32_t store_every;               // rows per stored result row; 0 = one result per slot at the end
  int32_t store_mode;                // 1 plain stores, 2 non-temporal stores
  int32_t n_hot;                     // rows kept in LDS (at most 64)
  float one;                         // 1.0f
};
}

namespace {
typedef _Float16 Half8 __attribute__((ext_vector_type(8)));
typedef uint32_t U4 __attribute__((ext_vector_type(4)));
constexpr int kInFlight = 8;
constexpr int kMaxHot = 64;
constexpr int kMaxChunk = 2048;

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

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(6))) void replay_hot_kernel(const fwdmi_mb_hot_args A) {
  __shared__ uint32_t s_row[kMaxChunk];
  __shared__ Half8 s_hot[kMaxHot * 16];
  const int x = blockIdx.x % 8;
  const int item = A.xcd_start[x] + blockIdx.x / 8;
  if (item >= A.xcd_start[x + 1]) return;
  const int t = A.item_table[item], s0 = A.item_start[item], n = min(A.item_count[item], kMaxChunk);
  const int n_hot = min(A.item_hot[item], n), n_cold = n - n_hot;
  const fwdmi_mb_hot_table FWDMI_MB_GLOBAL* tp = (const fwdmi_mb_hot_table FWDMI_MB_GLOBAL*)A.tables + t;
  const int32_t FWDMI_MB_GLOBAL* ids = (const int32_t FWDMI_MB_GLOBAL*)tp->ids;
  const int32_t FWDMI_MB_GLOBAL* hot = (const int32_t FWDMI_MB_GLOBAL*)tp->hot;
  const char FWDMI_MB_GLOBAL* tab = (const char FWDMI_MB_GLOBAL*)tp->data;
  const int tid = threadIdx.x;
  const int slot = tid >> 4, gl = tid & 15;
  {
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
    // the table's hot rows into LDS: sixteen lanes per row, sixteen rows per round
    const int k_hot = min(A.n_hot, kMaxHot);
    for (int r = slot; r < k_hot; r += 16)
      s_hot[r * 16 + gl] = *(const Half8 FWDMI_MB_GLOBAL*)(tab + (size_t)(uint32_t)hot[r] * 256 + gl * 16);
  }
  __syncthreads();
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  Half8 FWDMI_MB_GLOBAL* outp = (Half8 FWDMI_MB_GLOBAL*)A.out + ((size_t)item * 16 + slot) * 16 * 64 + gl;
  int since = 0, nout = 0;
  auto fold = [&](const Half8* v) {
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
  };
  {  // rows that come from the table
    const int per = (n_cold + 15) / 16;
    int i = slot * per;
    const int end = min(n_cold, i + per);
    for (; i + kInFlight <= end; i += kInFlight) {
      Half8 v[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) v[u] = *(const Half8 FWDMI_MB_GLOBAL*)(tab + (size_t)s_row[i + u] * 256 + gl * 16);
      fold(v);
    }
    for (; i < end; ++i) {
      const Half8 v = *(const Half8 FWDMI_MB_GLOBAL*)(tab + (size_t)s_row[i] * 256 + gl * 16);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf((float)v[e], A.one, acc[e]);
    }
  }
  {  // rows that come from LDS
    const int per = (n_hot + 15) / 16;
    int i = n_cold + slot * per;
    const int end = min(n, i + per);
    for (; i + kInFlight <= end; i += kInFlight) {
      Half8 v[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) v[u] = s_hot[(s_row[i + u] & (kMaxHot - 1)) * 16 + gl];
      fold(v);
    }
    for (; i < end; ++i) {
      const Half8 v = s_hot[(s_row[i] & (kMaxHot - 1)) * 16 + gl];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf((float)v[e], A.one, acc[e]);
    }
  }
  Half8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (_Float16)acc[e];
  store_row(&outp[(nout & 63) * 16], r, A.store_mode);
}
}  // namespace

// Launches one replay on `stream`; `grid_per_xcd` = items of the longest XCD segment.  Returns the
// hipError_t of the launch (0 = ok).
extern "C" int fwdmi_mb_replay_hot(const fwdmi_mb_hot_args* args, int grid_per_xcd, void* stream) {
  if (!args || grid_per_xcd <= 0 || args->n_hot < 0 || args->n_hot > kMaxHot) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(replay_hot_kernel, dim3(grid_per_xcd * 8), dim3(256), 0, static_cast<hipStream_t>(stream), *args);
  return (int)hipGetLastError();
}
