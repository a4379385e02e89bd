// K/V re-projection GEMM for gfx950:  C[M,N] = A[M,K] * W[N,K]^T + bias[N]
// fp16 or bf16 operands, fp32 accumulation on the matrix cores, result in the
// operand dtype.  Both operands are K-contiguous ("NT"), which is how the
// fused QKV weight [3*Hd, Hd] and the holder of gathered hidden rows [T, Hd]
// are laid out.
//
// Tiling: one 256-thread workgroup (4 wavefronts, 2 x 2) owns a 256 x 256 tile
// of C; each wavefront owns 128 x 128 = 4 x 4 MFMA 32x32x16 tiles (256 fp32
// accumulator registers per lane).  The K loop moves BK = 64 at a time through
// a two-stage LDS ring (2 x (32 + 32) KiB of the 160 KiB per CU): tile t+1 is
// copied global -> LDS by buffer_load ... lds (no VGPR round trip) while the
// matrix cores consume tile t.
//
// LDS layout: a tile is [256 rows][8 chunks of 16 B]; chunk c of row r lives at
// position c ^ (r % 8), so that the 128-bit fragment reads of 8 consecutive rows
// touch 8 different 16-byte bank groups.  The DMA writes 1 KiB per wavefront in
// lane order, so the swizzle is applied on the global side: lane l of a
// wave-wide load fetches chunk (l%8) ^ (l/8) of row l/8.
//
// Workgroups are renumbered so that the 32 workgroups an XCD runs together
// form an 8 x 4 block of tiles and share their A and W panels in that XCD's L2.
#include "aps_common.h"

namespace aps {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK * 2;          // 32 KiB, same for A and W tiles
constexpr int kStageBytes = 2 * kTileBytes;      // A + W
constexpr int kStages = 2;
constexpr int kLdsBytes = kStages * kStageBytes;  // 128 KiB
constexpr int kNumXcd = 8;
constexpr int kGroupM = 8;

struct GemmArgs {
  const char* a; const char* w; const void* bias; char* c;
  int64_t lda_b, ldw_b, ldc;  // lda/ldw in bytes, ldc in elements
  int64_t m, n, k;
  int tiles_m, tiles_n;
  // optional row scatter of the epilogue: row t of C goes to row_map[t] (rows of ldc elements), <0 skipped
  const int64_t* row_map;
  int64_t row_map_limit;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes > 0xffffffffll ? 0xffffffffu : (uint32_t)bytes;
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
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <bool BF16>
__global__ __launch_bounds__(kThreads, 1) void gemm_nt_kernel(const GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- tile assignment: XCD-contiguous, grouped 8 tiles along M
  int pid_m, pid_n;
  {
    const int total = g.tiles_m * g.tiles_n;
    const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
    const int w = blockIdx.x;
    const int logical = (w % kNumXcd) * per_xcd + w / kNumXcd;
    if (logical >= total) return;
    const int in_group = kGroupM * g.tiles_n;
    const int group = logical / in_group;
    const int first_m = group * kGroupM;
    const int gsz = min(g.tiles_m - first_m, kGroupM);
    const int r = logical - group * in_group;
    pid_m = first_m + r % gsz;
    pid_n = r / gsz;
  }

  // ---- global -> LDS DMA addressing
  const int64_t row0 = (int64_t)pid_m * BM, col0 = (int64_t)pid_n * BN;
  const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(g.a + row0 * g.lda_b, (g.m - row0) * g.lda_b);
  const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(g.w + col0 * g.ldw_b, (g.n - col0) * g.ldw_b);
  const int lrow = lane >> 3;                       // row within the 8-row group of a wave-wide load
  const int lchunk = (lane & 7) ^ lrow;             // swizzled 16-byte chunk this lane fetches
  const uint32_t voff_a = (uint32_t)(lrow * g.lda_b + lchunk * 16);
  const uint32_t voff_w = (uint32_t)(lrow * g.ldw_b + lchunk * 16);
  const uint32_t grp_a = (uint32_t)(8 * g.lda_b), grp_w = (uint32_t)(8 * g.ldw_b);

  auto issue_loads = [&](int kt, int stage) {
    char* sa = lds + stage * kStageBytes;
    char* sw = sa + kTileBytes;
    const uint32_t koff = (uint32_t)kt * (BK * 2);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = wave * 8 + j;  // 8-row group of the tile handled by this wave-wide load
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(sa + i * 1024), 16,
                                               voff_a, koff + i * grp_a, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void*)(sw + i * 1024), 16,
                                               voff_w, koff + i * grp_w, 0, 0);
    }
  };

  // ---- LDS -> register fragment addressing (row = base + lane%32, chunk = 2*ks + lane/32, swizzled)
  const int frow = lane & 31, fhalf = lane >> 5;
  const uint32_t a_row_off = (uint32_t)((wm * 128 + frow) * (BK * 2));
  const uint32_t w_row_off = (uint32_t)((wn * 128 + frow) * (BK * 2));
  uint32_t chunk_off[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) chunk_off[ks] = (uint32_t)(((2 * ks + fhalf) ^ (frow & 7)) * 16);

  float16v acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int nk = (int)(g.k / BK);
  issue_loads(0, 0);
  for (int kt = 0; kt < nk; ++kt) {
    const int stage = kt & 1;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of tile kt has landed in LDS
    __syncthreads();                      // everyone's part has landed; everyone is done with the other stage
    if (kt + 1 < nk) issue_loads(kt + 1, stage ^ 1);
    const char* sa = lds + stage * kStageBytes;
    const char* sw = sa + kTileBytes;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4 af[4], wf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = *(const u32x4*)(sa + a_row_off + i * (32 * BK * 2) + chunk_off[ks]);
        wf[i] = *(const u32x4*)(sw + w_row_off + i * (32 * BK * 2) + chunk_off[ks]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma32<BF16>(af[i], wf[j], acc[i][j]);
    }
  }

  // ---- epilogue: bias, convert, store.  Lane l of a 32x32 result tile holds column l%32 and
  // rows 8*(e/4) + 4*(l/32) + e%4, e = 0..15.
  uint16_t* c = (uint16_t*)g.c;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t col = col0 + wn * 128 + j * 32 + frow;
    float bv = 0.f;
    if (g.bias) {
      const uint16_t bb = ((const uint16_t*)g.bias)[col];
      bv = BF16 ? __uint_as_float((uint32_t)bb << 16) : (float)__builtin_bit_cast(_Float16, bb);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        int64_t row = row0 + wm * 128 + i * 32 + 8 * (e >> 2) + 4 * fhalf + (e & 3);
        if (row >= g.m) continue;
        if (g.row_map) {
          row = g.row_map[row];
          if (row < 0 || row >= g.row_map_limit) continue;
        }
        const float v = acc[i][j][e] + bv;
        c[row * g.ldc + col] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
      }
    }
  }
}

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

int aps_linear_nt(const void* x, const void* weight, const void* bias, void* out, int64_t m, int64_t n, int64_t k,
                  int64_t x_stride, int64_t w_stride, int64_t out_stride, const int64_t* out_row_map,
                  int64_t out_rows, int dtype, aps_stream_t stream) {
  if (m < 0 || n <= 0 || k <= 0) return APS_ERR_INVALID_ARG;
  if (m == 0) return APS_OK;
  if (!x || !weight || !out) return APS_ERR_INVALID_ARG;
  if (dtype != APS_F16 && dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  if (n % BN != 0 || k % BK != 0) return APS_ERR_UNSUPPORTED;
  if (x_stride < k || w_stride < k || out_stride < n) return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(x), addr(weight), (uint64_t)x_stride * 2, (uint64_t)w_stride * 2}) != 16)
    return APS_ERR_UNSUPPORTED;
  // one tile's rows must be addressable with 32-bit byte offsets
  if ((int64_t)BM * x_stride * 2 >= ((int64_t)1 << 31) || (int64_t)BN * w_stride * 2 >= ((int64_t)1 << 31))
    return APS_ERR_UNSUPPORTED;
  GemmArgs g{};
  g.a = (const char*)x; g.w = (const char*)weight; g.bias = bias; g.c = (char*)out;
  g.lda_b = x_stride * 2; g.ldw_b = w_stride * 2; g.ldc = out_stride;
  g.m = m; g.n = n; g.k = k;
  g.tiles_m = (int)((m + BM - 1) / BM); g.tiles_n = (int)(n / BN);
  g.row_map = out_row_map; g.row_map_limit = out_rows;
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  if (total >= ((int64_t)1 << 30)) return APS_ERR_UNSUPPORTED;
  const int64_t per_xcd = (total + kNumXcd - 1) / kNumXcd;
  const dim3 grid((unsigned)(per_xcd * kNumXcd));
  hipStream_t s = (hipStream_t)stream;
  // more than 64 KiB of dynamic LDS has to be allowed per function (and per device)
  const void* fn = dtype == APS_BF16 ? (const void*)gemm_nt_kernel<true> : (const void*)gemm_nt_kernel<false>;
  const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e != hipSuccess) return (int)e;
  if (dtype == APS_BF16)
    hipLaunchKernelGGL(gemm_nt_kernel<true>, grid, dim3(kThreads), kLdsBytes, s, g);
  else
    hipLaunchKernelGGL(gemm_nt_kernel<false>, grid, dim3(kThreads), kLdsBytes, s, g);
  return launch_status();
}

}  // extern "C"
