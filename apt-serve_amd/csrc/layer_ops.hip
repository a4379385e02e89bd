// Residual add + LayerNorm of the OPT decoder layer for gfx950, one launch per (add, norm) pair.
//
// A decode step of OPT-13B runs two LayerNorms and two residual adds per layer on a handful of rows: as four
// element-wise launches of a tensor library they cost more in launch and memory round trips than in work.  Here
// one workgroup owns one row: it adds the residual in fp32, rounds the sum once to the 16-bit activation type
// (that rounded sum is the next residual), and normalises the rounded values — mean and variance in two passes
// over registers, fp32 — so the results are those of "add, then LayerNorm" on 16-bit tensors.
#include "aps_common.h"
#include "mfma_common.h"

namespace aps {
namespace {

constexpr int kLnThreads = 256, kLnVecs = 8;  // a row of up to 256 * 8 * 8 = 16384 elements lives in registers

struct AddLnArgs {
  char* normed; char* sum;                       // sum nullable
  const char* x; const char* residual;           // residual nullable
  const char* gamma; const char* beta;           // beta nullable
  int64_t x_stride_b, res_stride_b, normed_stride_b, sum_stride_b;
  int width;
  float eps;
};

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  __syncthreads();  // red may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <bool BF16>
__device__ __forceinline__ float from16(uint32_t bits) {
  if constexpr (BF16) return __uint_as_float(bits << 16);
  else return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}
template <bool BF16>
__device__ __forceinline__ uint32_t to16(float v) {
  return BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
}

template <bool BF16, int VECS>
__global__ __launch_bounds__(kLnThreads) void add_layer_norm_kernel(const AddLnArgs g) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int nvec = g.width >> 3;  // 8 elements (16 bytes) per vector
  const char* x = g.x + row * g.x_stride_b;
  const char* r = g.residual ? g.residual + row * g.res_stride_b : nullptr;
  float v[VECS][8];
  float total = 0.f;
  // scale and shift of the norm are requested with the row itself: on a handful of rows the launch lasts as long
  // as its chain of memory round trips, and these two would otherwise form a third one after the statistics
  u32x4 gw[VECS], gb[VECS];
#pragma unroll
  for (int j = 0; j < VECS; ++j) {
    const int i = min((int)threadIdx.x + j * kLnThreads, nvec - 1);
    gw[j] = *(const u32x4*)(g.gamma + (int64_t)i * 16);
    gb[j] = g.beta ? *(const u32x4*)(g.beta + (int64_t)i * 16) : u32x4{0u, 0u, 0u, 0u};
  }
#pragma unroll
  for (int j = 0; j < VECS; ++j) {
    const int i = threadIdx.x + j * kLnThreads;
    if (i < nvec) {
      const u32x4 a = *(const u32x4*)(x + (int64_t)i * 16);
      u32x4 b = {0u, 0u, 0u, 0u};
      if (r) b = *(const u32x4*)(r + (int64_t)i * 16);
      u32x4 s16;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float lo = from16<BF16>(a[e] & 0xffffu), hi = from16<BF16>(a[e] >> 16);
        if (r) {  // the sum is rounded once to the activation type; the norm sees the rounded sum
          lo = from16<BF16>(to16<BF16>(lo + from16<BF16>(b[e] & 0xffffu)));
          hi = from16<BF16>(to16<BF16>(hi + from16<BF16>(b[e] >> 16)));
        }
        v[j][2 * e] = lo;
        v[j][2 * e + 1] = hi;
        s16[e] = to16<BF16>(lo) | (to16<BF16>(hi) << 16);
        total += lo + hi;
      }
      if (g.sum) *(u32x4*)(g.sum + row * g.sum_stride_b + (int64_t)i * 16) = s16;
    }
  }
  const float mean = block_sum(total, red) / (float)g.width;
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < VECS; ++j) {
    if (threadIdx.x + j * kLnThreads < nvec) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = v[j][e] - mean;
        sq += d * d;
      }
    }
  }
  const float rstd = rsqrtf(block_sum(sq, red) / (float)g.width + g.eps);
#pragma unroll
  for (int j = 0; j < VECS; ++j) {
    const int i = threadIdx.x + j * kLnThreads;
    if (i < nvec) {
      const u32x4 w = gw[j], bb = gb[j];
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = (v[j][2 * e] - mean) * rstd * from16<BF16>(w[e] & 0xffffu) + from16<BF16>(bb[e] & 0xffffu);
        const float hi = (v[j][2 * e + 1] - mean) * rstd * from16<BF16>(w[e] >> 16) + from16<BF16>(bb[e] >> 16);
        o[e] = to16<BF16>(lo) | (to16<BF16>(hi) << 16);
      }
      *(u32x4*)(g.normed + row * g.normed_stride_b + (int64_t)i * 16) = o;
    }
  }
}

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" int aps_add_layer_norm(void* normed, void* sum, const void* x, const void* residual, const void* gamma,
                                  const void* beta, int64_t rows, int64_t width, int64_t x_stride,
                                  int64_t residual_stride, int64_t normed_stride, int64_t sum_stride, float eps,
                                  int dtype, aps_stream_t stream) {
  if (rows < 0 || width <= 0 || !(eps >= 0.f)) return APS_ERR_INVALID_ARG;
  if (rows == 0) return APS_OK;
  if (!normed || !x || !gamma) return APS_ERR_INVALID_ARG;
  if (dtype != APS_F16 && dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  if (width % 8 != 0 || width > kLnThreads * kLnVecs * 8 || rows > 0x7fffffff) return APS_ERR_UNSUPPORTED;
  if (x_stride < width || normed_stride < width || (residual && residual_stride < width) ||
      (sum && sum_stride < width))
    return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(normed), addr(sum), addr(x), addr(residual), addr(gamma), addr(beta),
                        (uint64_t)x_stride * 2, (uint64_t)residual_stride * 2, (uint64_t)normed_stride * 2,
                        (uint64_t)sum_stride * 2}) != 16)
    return APS_ERR_UNSUPPORTED;
  AddLnArgs g{(char*)normed, (char*)sum, (const char*)x, (const char*)residual, (const char*)gamma,
              (const char*)beta, x_stride * 2, residual_stride * 2, normed_stride * 2, sum_stride * 2, (int)width, eps};
  const dim3 grid((unsigned)rows);
  // rows of up to 3 * 256 * 8 = 6144 elements (every OPT up to 13B) keep 3 vectors per thread, wider ones 8
  const bool narrow = width <= 3 * kLnThreads * 8;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == APS_BF16) {
    if (narrow) APS_LAUNCH((add_layer_norm_kernel<true, 3>), grid, dim3(kLnThreads), 0, s, g);
    else APS_LAUNCH((add_layer_norm_kernel<true, kLnVecs>), grid, dim3(kLnThreads), 0, s, g);
  } else {
    if (narrow) APS_LAUNCH((add_layer_norm_kernel<false, 3>), grid, dim3(kLnThreads), 0, s, g);
    else APS_LAUNCH((add_layer_norm_kernel<false, kLnVecs>), grid, dim3(kLnThreads), 0, s, g);
  }
  return launch_status();
}
