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

}  // namespace fwdmi
