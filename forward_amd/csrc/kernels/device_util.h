// Device-side helpers shared by the kernels: 16-byte register packs and global-memory accessors.
#pragma once

#include <hip/hip_runtime.h>

namespace fwdmi {

template <typename T, int N>
struct alignas((sizeof(T) * N) < 16 ? (sizeof(T) * N) : 16) Pack {
  T v[N];
};

// Pointers that reach the kernel inside a struct (or are loaded from the table array) are
// generic to the compiler, which then emits flat_* accesses; these casts pin them to global
// memory so rows are fetched with global_load_dwordx4.
#define FWDMI_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ const T FWDMI_GLOBAL* gconst(const void* p) {
  return (const T FWDMI_GLOBAL*)(p);
}
template <typename T>
__device__ __forceinline__ T FWDMI_GLOBAL* gmut(void* p) {
  return (T FWDMI_GLOBAL*)(p);
}

// N-element (at most 16-byte aligned) vector load / store in global memory.
template <typename T, int N>
__device__ __forceinline__ Pack<T, N> gload(const T FWDMI_GLOBAL* p) {
  Pack<T, N> r;
  if constexpr (N == 1) {
    r.v[0] = *p;
  } else {
    typedef T V __attribute__((ext_vector_type(N), aligned(alignof(Pack<T, N>))));
    const V x = *(const V FWDMI_GLOBAL*)p;
    __builtin_memcpy(&r, &x, sizeof(r));
  }
  return r;
}
// The same load with the non-temporal hint, for data that is read once (a run's ids and weights):
// the lines pass through L2 without taking the place of table rows.
template <typename T, int N>
__device__ __forceinline__ Pack<T, N> gload_stream(const T FWDMI_GLOBAL* p) {
  static_assert(N > 1, "vector loads only");
  typedef T V __attribute__((ext_vector_type(N), aligned(alignof(Pack<T, N>))));
  const V x = __builtin_nontemporal_load((const V FWDMI_GLOBAL*)p);
  Pack<T, N> r;
  __builtin_memcpy(&r, &x, sizeof(r));
  return r;
}
template <typename T, int N>
__device__ __forceinline__ void gstore(T FWDMI_GLOBAL* p, const Pack<T, N>& r) {
  if constexpr (N == 1) {
    *p = r.v[0];
  } else {
    typedef T V __attribute__((ext_vector_type(N), aligned(alignof(Pack<T, N>))));
    V x;
    __builtin_memcpy(&x, &r, sizeof(r));
    *(V FWDMI_GLOBAL*)p = x;
  }
}
// The same store (8, 16 or 32 bytes) with the non-temporal hint: the line is streamed through L2 instead of
// staying there as a dirty line that displaces table rows.  For results far larger than the L2s.
// Written as the instruction itself: a builtin store next to a plain store of the same value (one
// per branch of a run-time choice) is merged with it by the optimiser and loses the hint.
// Each store is followed by `s_nop 1`: on this architecture a vector instruction that overwrites the
// data registers of a store wider than 64 bits needs two wait states behind it, and the compiler, which
// inserts them for stores it emits itself, does not look inside an asm statement (the registers are
// dead to it as soon as the statement ends).
template <typename T, int N>
__device__ __forceinline__ void gstore_stream(T FWDMI_GLOBAL* p, const Pack<T, N>& r) {
  constexpr int kBytes = (int)sizeof(Pack<T, N>);
  static_assert(kBytes == 8 || kBytes == 16 || kBytes == 32, "packs of 8, 16 or 32 bytes");
  typedef uint32_t U4 __attribute__((ext_vector_type(4)));
  typedef uint32_t U2 __attribute__((ext_vector_type(2)));
  if constexpr (kBytes == 8) {
    U2 x;
    __builtin_memcpy(&x, &r, 8);
    asm volatile("global_store_dwordx2 %0, %1, off nt\n\ts_nop 1" ::"v"(p), "v"(x) : "memory");
  } else {
    U4 x;
    __builtin_memcpy(&x, &r, 16);
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(p), "v"(x) : "memory");
    if constexpr (kBytes == 32) {
      __builtin_memcpy(&x, reinterpret_cast<const char*>(&r) + 16, 16);
      asm volatile("global_store_dwordx4 %0, %1, off offset:16 nt\n\ts_nop 1" ::"v"(p), "v"(x) : "memory");
    }
  }
}

}  // namespace fwdmi
