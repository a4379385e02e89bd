// Shared pieces of the matrix-core kernels (gfx950): operand vector types, MFMA wrappers,
// buffer descriptors, rounding to the 16-bit output types, hand-placed wait points.
#pragma once
#include <atomic>

#include "aps_common.h"

namespace aps {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef float float4v __attribute__((ext_vector_type(4)));

// Buffer descriptor over [p, p + bytes): loads past the end return zeros and touch no memory.  For an operand of
// `rows` rows `stride` bytes apart of which `row_bytes` are valid, bytes is (rows - 1) * stride + row_bytes, not
// rows * stride: the last row of a strided view (a column slice of a wider tensor) ends where its storage ends.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes <= 0 ? 0u : (bytes > 0xffffffffll ? 0xffffffffu : (uint32_t)bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}

template <bool BF16>
__device__ __forceinline__ float16v mfma32(const u32x4& a, const u32x4& b, const float16v& c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0,
                                                  0);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }
// The same for code that is inlined into more than one kernel whose results are compared bit for bit: x is rounded
// to fp32 first, whatever produced it.  The conversion of a product can otherwise be fused with the multiply into
// one instruction that rounds once (v_fma_mixlo_f16) in one of those kernels and not in another.  (Not the default:
// the empty asm is a scheduling obstacle, and the streaming weighted sum, at its register limit, runs 60 % longer
// with it.)
__device__ __forceinline__ uint16_t f32_to_f16_bits_rounded(float x) {
  asm volatile("" : "+v"(x));
  return __builtin_bit_cast(uint16_t, (_Float16)x);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// Hand-placed wait points: a __syncthreads() would add fences that wait for every outstanding DMA load.
#define APS_WAIT_VM(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")
#define APS_WAIT_LGKM0() asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory")
#define APS_BARRIER() asm volatile("s_barrier" ::: "memory")

template <bool BF16>
__device__ __forceinline__ float4v mfma16(const u32x4& a, const u32x4& b, const float4v& c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0,
                                                  0);
}

// ---- results handed from workgroup to workgroup inside one launch
// The partial results of a split reduction cross between workgroups through device-coherent stores and loads
// (they go past the L2 of the compute die, which is not coherent with the other dies' inside a launch) and one
// counter per output tile: a workgroup waits until its own stores are acknowledged, counts itself in, and the
// one that finds every other workgroup of the tile counted does the sum.  No workgroup waits for another;
// whichever arrives last adds the parts in part order, so the result does not depend on which.  No device-scope
// fence is used: a release writes the whole L2 back (measured: 8-10 us per launch of 240 workgroups, more than a
// second launch for the sum costs).
__device__ __forceinline__ void coherent_store(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// True in every thread of the workgroup that arrives last of `count` at `counter` (zero before the first arrival;
// the last arrival puts it back to zero).  Called by all threads of the workgroup after their coherent_store()s;
// `flag` is a word of LDS that no wavefront still uses.
__device__ __forceinline__ bool last_arrival(int* counter, int count, int* flag) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);   // every store of this wavefront acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = before == count - 1;
    // nobody else touches the counter any more in this launch: zero for the next one
    if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last;
  }
  __syncthreads();
  return *flag != 0;
}

template <bool BF16>
__device__ __forceinline__ float load_16bit_as_f32(const void* p, int64_t i) {
  const uint16_t v = ((const uint16_t*)p)[i];
  return BF16 ? __uint_as_float((uint32_t)v << 16) : (float)__builtin_bit_cast(_Float16, v);
}

// More than 64 KiB of dynamic LDS has to be allowed per function and device: done once per (kernel, device)
// instead of on every launch.  `slot` numbers the kernel instantiations of one source file that need it.
inline hipError_t allow_dynamic_lds(const void* fn, int bytes, int slot) {
  static std::atomic<uint64_t> done[40];
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  const uint64_t bit = device >= 0 && device < 64 ? (uint64_t)1 << device : 0;
  if (bit && (done[slot].load(std::memory_order_relaxed) & bit)) return hipSuccess;
  e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && bit) done[slot].fetch_or(bit, std::memory_order_relaxed);
  return e;
}

}  // namespace
}  // namespace aps
