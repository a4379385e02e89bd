// Internal helpers shared by the gfx950 kernels of libaptserve_hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "aptserve_hip.h"

namespace aps {

// N-byte plain-old-data vector moved by one global load/store instruction.
template <int BYTES> struct VecOf;
template <> struct VecOf<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct VecOf<8>  { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct VecOf<4>  { typedef uint32_t type; };
template <> struct VecOf<2>  { typedef uint16_t type; };
template <> struct VecOf<1>  { typedef uint8_t type; };

template <int BYTES>
__device__ __forceinline__ typename VecOf<BYTES>::type load_vec(const char* p) {
  return *reinterpret_cast<const typename VecOf<BYTES>::type*>(p);
}
template <int BYTES>
__device__ __forceinline__ void store_vec(char* p, typename VecOf<BYTES>::type v) {
  *reinterpret_cast<typename VecOf<BYTES>::type*>(p) = v;
}
// Streaming variants: data that is touched once should not displace the L2
// working set of the kernels running next to the copy.
template <int BYTES>
__device__ __forceinline__ typename VecOf<BYTES>::type load_vec_stream(const char* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const typename VecOf<BYTES>::type*>(p));
}
template <int BYTES>
__device__ __forceinline__ void store_vec_stream(char* p, typename VecOf<BYTES>::type v) {
  __builtin_nontemporal_store(v, reinterpret_cast<typename VecOf<BYTES>::type*>(p));
}

// Largest power-of-two vector width (<=16 bytes) dividing every value given.
inline int common_vec_bytes(std::initializer_list<uint64_t> vals) {
  uint64_t acc = 0;
  for (uint64_t v : vals) acc |= v;
  for (int b = 16; b > 1; b >>= 1)
    if ((acc & (uint64_t)(b - 1)) == 0) return b;
  return 1;
}

inline uint64_t addr(const void* p) { return (uint64_t)(uintptr_t)p; }

// Every kernel launch goes through APS_LAUNCH, which first drops whatever error an earlier, unrelated call
// left in the runtime's per-thread slot: launch_status() then reports this launch and nothing older.
#define APS_LAUNCH(...)             \
  do {                              \
    (void)hipGetLastError();        \
    hipLaunchKernelGGL(__VA_ARGS__); \
  } while (0)

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? APS_OK : (int)e;
}

inline int elem_bytes_of(int dtype) {
  switch (dtype) {
    case APS_F16: case APS_BF16: return 2;
    case APS_F32: return 4;
    case APS_F64: return 8;
    case APS_FP8_E4M3: return 1;
    default: return 0;
  }
}

}  // namespace aps
