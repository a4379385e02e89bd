// Measurement kernels of the hybrid-cache library for gfx950, built into a library of their own
// (libaptserve_probes.so): plain copy / read / fill streams and matrix-core instruction streams that show what
// the part sustains, so that the product kernels can be held against a measured ceiling as well as against the
// published peak.  Nothing of the product path calls into this file.
#include "aps_common.h"
#include "mfma_common.h"
#include "aptserve_probes.h"

namespace aps {
namespace {

constexpr int kMaxThreads = 256;

// Plain streams in the shape of the row movers: a workgroup owns 256 * U consecutive 16-byte chunks and every
// thread moves U of them (all loads, then all stores); no loop, workgroups are dispatched in address order.
template <int U>
__global__ __launch_bounds__(kMaxThreads) void copy_bytes_kernel(VecOf<16>::type* __restrict__ dst,
                                                                  const VecOf<16>::type* __restrict__ src,
                                                                  int64_t n_vec) {
  const int64_t base = (int64_t)blockIdx.x * (kMaxThreads * U) + threadIdx.x;
  VecOf<16>::type v[U];
#pragma unroll
  for (int j = 0; j < U; ++j)
    if (base + j * kMaxThreads < n_vec) v[j] = __builtin_nontemporal_load(src + base + j * kMaxThreads);
#pragma unroll
  for (int j = 0; j < U; ++j)
    if (base + j * kMaxThreads < n_vec) __builtin_nontemporal_store(v[j], dst + base + j * kMaxThreads);
}

template <int U>
__global__ __launch_bounds__(kMaxThreads) void read_bytes_kernel(uint32_t* __restrict__ sink,
                                                                  const VecOf<16>::type* __restrict__ src,
                                                                  int64_t n_vec) {
  const int64_t base = (int64_t)blockIdx.x * (kMaxThreads * U) + threadIdx.x;
  uint32_t x = 0;
  VecOf<16>::type v[U];
#pragma unroll
  for (int j = 0; j < U; ++j) {
    v[j] = VecOf<16>::type{0u, 0u, 0u, 0u};
    if (base + j * kMaxThreads < n_vec) v[j] = __builtin_nontemporal_load(src + base + j * kMaxThreads);
  }
#pragma unroll
  for (int j = 0; j < U; ++j) x ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  if (x == 0x9e3779b9u && sink) *sink = x;  // keeps the loads alive; practically never taken
}

template <int U>
__global__ __launch_bounds__(kMaxThreads) void fill_bytes_kernel(VecOf<16>::type* __restrict__ dst, int64_t n_vec,
                                                                  uint32_t seed) {
  const int64_t base = (int64_t)blockIdx.x * (kMaxThreads * U) + threadIdx.x;
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const int64_t i = base + j * kMaxThreads;
    // not a constant pattern: what the memory sustains depends on the data
    const uint32_t h = ((uint32_t)i * 2654435761u) ^ seed;
    const VecOf<16>::type v = {h, h * 0x85ebca6bu, h ^ 0xc2b2ae35u, h * 0x27d4eb2fu};
    if (i < n_vec) __builtin_nontemporal_store(v, dst + i);
  }
}


// ---------------------------------------------------------------- what the matrix cores sustain
// Nothing but MFMA instructions on operands that stay in registers: 4 wavefronts per workgroup (one per SIMD),
// one workgroup per CU, `iters` rounds of 16 independent 32x32x16 (shape 0) or 32 independent 16x16x32
// (shape 1) products each, i.e. 2 * 16 * 32*32*16 flops per wavefront and round in both shapes.  The operands
// are whatever 16-bit values the caller put into `operands` (one 128-byte line per lane): with random values
// the part throttles its clock under the power the matrix cores draw, which is what this probe is for.
template <int SHAPE, bool BF16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mfma_probe_kernel(
    const u32x4* __restrict__ operands, float* __restrict__ sink, int iters) {
  u32x4 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[threadIdx.x * 8 + i];
    b[i] = operands[threadIdx.x * 8 + 4 + i];
  }
  // One asm statement per instruction, accumulators in the accumulation registers: the loop body is exactly the
  // MFMA stream written here, back to back, every accumulator 16 (32) instructions away from its next use.
  float s = 0.f;
  if constexpr (SHAPE == 0) {
    float16v acc[16];
#pragma unroll
    for (int q = 0; q < 16; ++q)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[q][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        if constexpr (BF16)
          asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[q]) : "v"(a[q >> 2]), "v"(b[q & 3]));
        else
          asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[q]) : "v"(a[q >> 2]), "v"(b[q & 3]));
      }
    }
    asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc[12]), "+a"(acc[13]), "+a"(acc[14]), "+a"(acc[15]));
#pragma unroll
    for (int q = 0; q < 16; ++q)
#pragma unroll
      for (int e = 0; e < 16; ++e) s += acc[q][e];
  } else {
    float4v acc[32];
#pragma unroll
    for (int q = 0; q < 32; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[q][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int q = 0; q < 32; ++q) {
        if constexpr (BF16)
          asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[q]) : "v"(a[(q >> 3) & 3]), "v"(b[q & 3]));
        else
          asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[q]) : "v"(a[(q >> 3) & 3]), "v"(b[q & 3]));
      }
    }
    asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc[28]), "+a"(acc[29]), "+a"(acc[30]), "+a"(acc[31]));
#pragma unroll
    for (int q = 0; q < 32; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) s += acc[q][e];
  }
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}


// How one SIMD issues matrix and vector instructions side by side (shapes 2..6 of the probe).  A round is 16
// v_mfma_f32_32x32x16 on four accumulators and / or 16 vector units of one v_exp_f32 and three v_fma_f32 on
// values that stay in registers, one asm statement per instruction so the order below is the order issued:
// MODE 0 the two kinds alternate instruction by instruction, 1 all MFMAs then all vector units, 2 vector units
// only.  WAVES = wavefronts per workgroup (4: one per SIMD, 8: two).
template <int MODE, bool BF16, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void issue_mix_probe_kernel(const u32x4* __restrict__ operands,
                                                                     float* __restrict__ sink, int iters) {
  u32x4 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[(threadIdx.x & 255) * 8 + i];
    b[i] = operands[(threadIdx.x & 255) * 8 + 4 + i];
  }
  float x[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = __uint_as_float(a[i & 3][i >> 2]) * 1e-3f;
  float c0 = 1e-3f, c1 = 0.5f;
  asm volatile("" : "+v"(c0), "+v"(c1));
  float16v acc[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[q][e] = 0.f;
  auto mfma = [&](int q) __attribute__((always_inline)) {
    if constexpr (BF16)
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[q & 3]) : "v"(a[q & 3]), "v"(b[(q >> 2) & 3]));
    else
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[q & 3]) : "v"(a[q & 3]), "v"(b[(q >> 2) & 3]));
  };
  auto vec = [&](int q) __attribute__((always_inline)) {
    asm volatile("v_exp_f32 %0, %0\n\tv_fma_f32 %0, %0, %1, %2\n\tv_fma_f32 %0, %0, %1, %2\n\tv_fma_f32 %0, %0, %1, %2"
                 : "+v"(x[q & 7])
                 : "v"(c0), "v"(c1));
  };
  for (int it = 0; it < iters; ++it) {
    if constexpr (MODE == 0) {
#pragma unroll
      for (int q = 0; q < 16; ++q) { mfma(q); vec(q); }
    } else {
      if constexpr (MODE == 1) {
#pragma unroll
        for (int q = 0; q < 16; ++q) mfma(q);
      }
#pragma unroll
      for (int q = 0; q < 16; ++q) vec(q);
    }
  }
  asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc[0]), "+a"(acc[1]), "+a"(acc[2]), "+a"(acc[3]));
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[q][e];
#pragma unroll
  for (int i = 0; i < 8; ++i) s += x[i];
  sink[blockIdx.x * (WAVES * 64) + threadIdx.x] = s;
}

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

int aps_copy_bytes(void* dst, const void* src, int64_t nbytes, aps_stream_t stream) {
  return aps_stream_probe(0, 1, dst, src, nbytes, stream);
}

int aps_stream_probe(int mode, int chunks_per_thread, void* dst, const void* src, int64_t nbytes,
                     aps_stream_t stream) {
  if (nbytes < 0 || mode < 0 || mode > 2) return APS_ERR_INVALID_ARG;
  if (chunks_per_thread != 1 && chunks_per_thread != 4) return APS_ERR_INVALID_ARG;
  if (nbytes == 0) return APS_OK;
  if ((mode != 2 && !src) || !dst) return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({mode == 1 ? 0 : addr(dst), addr(src), (uint64_t)nbytes}) != 16) return APS_ERR_UNSUPPORTED;
  const int64_t n_vec = nbytes / 16;
  const int64_t per_block = (int64_t)kMaxThreads * chunks_per_thread;
  const int64_t grid = (n_vec + per_block - 1) / per_block;
  if (grid >= (int64_t)1 << 31) return APS_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  const dim3 g((unsigned)grid), b(kMaxThreads);
  VecOf<16>::type* d = (VecOf<16>::type*)dst;
  const VecOf<16>::type* sp = (const VecOf<16>::type*)src;
  if (chunks_per_thread == 1) {
    if (mode == 0) APS_LAUNCH(copy_bytes_kernel<1>, g, b, 0, s, d, sp, n_vec);
    else if (mode == 1) APS_LAUNCH(read_bytes_kernel<1>, g, b, 0, s, (uint32_t*)dst, sp, n_vec);
    else APS_LAUNCH(fill_bytes_kernel<1>, g, b, 0, s, d, n_vec, 0x3c003c00u);
  } else {
    if (mode == 0) APS_LAUNCH(copy_bytes_kernel<4>, g, b, 0, s, d, sp, n_vec);
    else if (mode == 1) APS_LAUNCH(read_bytes_kernel<4>, g, b, 0, s, (uint32_t*)dst, sp, n_vec);
    else APS_LAUNCH(fill_bytes_kernel<4>, g, b, 0, s, d, n_vec, 0x3c003c00u);
  }
  return launch_status();
}

}  // extern "C"

extern "C" int aps_mfma_probe(int shape, int dtype, const void* operands, void* sink, int workgroups, int iters,
                              aps_stream_t stream) {
  if (shape < 0 || shape > 6 || (dtype != APS_F16 && dtype != APS_BF16) || !operands || !sink) return APS_ERR_INVALID_ARG;
  if (workgroups <= 0 || iters <= 0) return APS_OK;
  if ((addr(operands) & 15) || (addr(sink) & 3)) return APS_ERR_INVALID_ARG;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)workgroups), block(256);
  const u32x4* op = (const u32x4*)operands;
  if (shape >= 2) {
    const bool bf = dtype == APS_BF16;
    float* out = (float*)sink;
#define APS_MIX(MODE, WAVES)                                                                                   \
  do {                                                                                                         \
    if (bf) APS_LAUNCH((issue_mix_probe_kernel<MODE, true, WAVES>), grid, dim3(WAVES * 64), 0, s, op, out, iters); \
    else APS_LAUNCH((issue_mix_probe_kernel<MODE, false, WAVES>), grid, dim3(WAVES * 64), 0, s, op, out, iters);   \
  } while (0)
    switch (shape) {
      case 2: APS_MIX(0, 4); break;
      case 3: APS_MIX(1, 4); break;
      case 4: APS_MIX(2, 4); break;
      case 5: APS_MIX(0, 8); break;
      default: APS_MIX(1, 8); break;
    }
#undef APS_MIX
    return launch_status();
  }
  if (shape == 0) {
    if (dtype == APS_BF16) APS_LAUNCH((mfma_probe_kernel<0, true>), grid, block, 0, s, op, (float*)sink, iters);
    else APS_LAUNCH((mfma_probe_kernel<0, false>), grid, block, 0, s, op, (float*)sink, iters);
  } else {
    if (dtype == APS_BF16) APS_LAUNCH((mfma_probe_kernel<1, true>), grid, block, 0, s, op, (float*)sink, iters);
    else APS_LAUNCH((mfma_probe_kernel<1, false>), grid, block, 0, s, op, (float*)sink, iters);
  }
  return launch_status();
}
