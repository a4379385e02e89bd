// Device side of the paged decode attention: argument block, the walk of one wavefront over one partition of a
// sequence, and the group path's workgroup body.  A header because two translation units use it: the attention
// launcher, and the launch that attends K/V-cached and hidden-cached sequences of a decode step together.
#pragma once
#include <hip/hip_fp16.h>

#include <math.h>

#include "aps_common.h"
#include "mfma_common.h"

namespace aps {
namespace {

// No implicit fused multiply-adds in this header (the ones wanted are spelled fmaf): which products the compiler
// fuses with a following add depends on the code around them, and these functions are inlined into more than one
// kernel whose results are compared bit for bit.
#pragma clang fp contract(off)


typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

constexpr int kTile = 16;  // tokens per tile
constexpr float kLog2e = 1.4426950408889634f;

enum KvKind { KV_F16 = 0, KV_BF16 = 1, KV_FP8 = 2 };

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

// Sum over groups of LPT consecutive lanes; every lane of the group gets the sum.
template <int LPT>
__device__ __forceinline__ float group_sum(float x) {
  if constexpr (LPT >= 2) x += dpp_f32<0xB1>(x);   // quad_perm [1,0,3,2]
  if constexpr (LPT >= 4) x += dpp_f32<0x4E>(x);   // quad_perm [2,3,0,1]
  if constexpr (LPT >= 8) x += dpp_f32<0x141>(x);  // row_half_mirror
  if constexpr (LPT >= 16) x += dpp_f32<0x140>(x); // row_mirror
  if constexpr (LPT >= 32) x += __shfl_xor(x, 16);
  return x;
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// 16 bytes of K or V as EPL floats.
template <int KV>
struct Unpack;
template <>
struct Unpack<KV_F16> {
  static constexpr int EPL = 8;
  __device__ static __forceinline__ void run(const u32x4& r, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // copy the lane out first: __builtin_bit_cast applied directly to a vector
      // element reads element 0 whatever the index
      const uint32_t w = r[i];
      const half2_t h = __builtin_bit_cast(half2_t, w);
      f[2 * i] = (float)h.x;
      f[2 * i + 1] = (float)h.y;
    }
  }
};
template <>
struct Unpack<KV_BF16> {
  static constexpr int EPL = 8;
  __device__ static __forceinline__ void run(const u32x4& r, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = bf16_lo(r[i]);
      f[2 * i + 1] = bf16_hi(r[i]);
    }
  }
};
template <>
struct Unpack<KV_FP8> {
  static constexpr int EPL = 16;
  __device__ static __forceinline__ void run(const u32x4& r, float (&f)[16]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)r[i], false);
      const float2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)r[i], true);
      f[4 * i] = lo.x; f[4 * i + 1] = lo.y; f[4 * i + 2] = hi.x; f[4 * i + 3] = hi.y;
    }
  }
};

template <int QT>
__device__ __forceinline__ float q_to_f32(uint16_t bits) {
  if constexpr (QT == APS_F16) return (float)__builtin_bit_cast(_Float16, bits);
  else return __uint_as_float((uint32_t)bits << 16);
}
template <int QT>
__device__ __forceinline__ uint16_t f32_to_q(float x) {
  if constexpr (QT == APS_F16) {
    // x is rounded to fp32 first, whatever produced it: the conversion of a product can otherwise be fused with the
    // multiply into one instruction that rounds once (v_fma_mixlo_f16), in some of the kernels this is inlined into
    // and not in others
    asm volatile("" : "+v"(x));
    return __builtin_bit_cast(uint16_t, (_Float16)x);
  } else {  // bf16, round to nearest even
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
}

struct AttnArgs {
  void* out;                 // [B, H, D] (q dtype)
  float* part_out;           // [B, H, P, D] fp32   (flat path only)
  float* part_lse;           // [B, H, P]   fp32 (log2 domain)
  const void* q;
  const char* k_cache; const char* v_cache;
  const char* ws_k_cache; const char* ws_v_cache;
  const int32_t* block_tables; const uint8_t* block_types; const int32_t* seq_lens;
  const int32_t* seq_order;  // group path: sequence handled by workgroup row y (nullptr: rank in the kernel, or y itself)
  int64_t q_stride, out_stride, table_stride, types_stride;
  int64_t cache_block_stride_b, ws_block_stride_b;  // bytes
  int64_t num_cache_blocks, num_ws_blocks;
  int num_heads, block_size, partition_size, num_partitions, table_width;
  int batch, rank_in_kernel;
  float scale_log2;  // softmax_scale * k_scale * log2(e)
  float v_scale;
};

// State of one wavefront after it has walked its partition: the LPR lanes of token row 0 hold, for their
// (head, 16-byte chunk of the head vector), the running maximum m (log2 domain), the sum l of 2^(s - m) and the
// unnormalised weighted sum acc of V.
template <int EPL>
struct WaveResult {
  float m, l;
  float acc[EPL];
};

// One wavefront walks tokens [start, end) of sequence `seq` for HPW adjacent heads starting at head0.
// HPW adjacent heads share the wavefront: the LPT lanes of head h+1 sit next to those of head h, so one token
// contributes HPW*D contiguous elements to a wave-wide load (longer DRAM bursts per token row).
// DEPTH tiles of 16 tokens are in flight: the ring is filled with unconditional buffer loads (a tile past the
// end of the partition, or one whose block id is unusable, gets a zero-length descriptor: its loads touch no
// memory and return zeros), so no load sits under a branch and the compiler's wait counts stay exact.
template <int QT, int KV, int D, int HPW, int DEPTH>
__device__ __forceinline__ void decode_wave(const AttnArgs& a, int seq, int head0, int start, int end, int lane,
                                            WaveResult<Unpack<KV>::EPL>& res) {
  constexpr int EPL = Unpack<KV>::EPL;        // elements per lane
  constexpr int LPT = D / EPL;                // lanes per (token, head)
  constexpr int LPR = LPT * HPW;              // lanes per token row of the wave
  constexpr int TPL = 64 / LPR;               // tokens per wave-wide load
  constexpr int NG = kTile / TPL;             // loads per tile and per K/V
  static_assert(LPT >= 2 && LPR <= 32 && NG >= 1, "unsupported head size");
  constexpr int KV_ELEM_B = (KV == KV_FP8) ? 1 : 2;

  const int tl = lane / LPR;                            // token row of this lane
  const int head = head0 + (lane % LPR) / LPT;
  const int dl = lane % LPT;                            // 16-byte chunk of the head vector
  const int n_tiles = (end > start) ? (end - start + kTile - 1) / kTile : 0;

  // query fragment of this lane: fp32, or, when the cache holds the query's 16-bit type, the packed pairs as
  // they are (v_dot2 multiplies the 16-bit pairs exactly and accumulates in fp32: 4 instructions per 8 elements
  // instead of 8 conversions and 8 FMAs, and half the registers)
  // An fp8 cache under an fp16 query takes the same route: e4m3 values are exact in fp16, and one conversion
  // yields a packed pair.
  constexpr bool kDot2 = (KV == KV_F16 && QT == APS_F16) || (KV == KV_BF16 && QT == APS_BF16) ||
                         (KV == KV_FP8 && QT == APS_F16);
  float qf[kDot2 ? 1 : EPL];
  uint32_t qpk[kDot2 ? EPL / 2 : 1];
  {
    const uint16_t* qp = (const uint16_t*)a.q + (int64_t)seq * a.q_stride + (int64_t)head * D + dl * EPL;
#pragma unroll
    for (int i = 0; i < EPL; i += 8) {
      const u32x4 r = *(const u32x4*)(qp + i);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (kDot2) {
          qpk[i / 2 + j] = r[j];
        } else {
          qf[i + 2 * j] = q_to_f32<QT>((uint16_t)(r[j] & 0xffffu));
          qf[i + 2 * j + 1] = q_to_f32<QT>((uint16_t)(r[j] >> 16));
        }
      }
    }
  }

  // block ids (and types) of this partition: lane j holds logical block first_blk + j
  const int first_blk = start / a.block_size;
  const int n_blk = (end > start) ? (end - 1) / a.block_size - first_blk + 1 : 0;
  int my_blk = -1;
  int my_type = 0;
  if (lane < n_blk && first_blk + lane < a.table_width) {
    my_blk = a.block_tables[(int64_t)seq * a.table_stride + first_blk + lane];
    if (a.block_types) my_type = a.block_types[(int64_t)seq * a.types_stride + first_blk + lane];
  }

  const int64_t row_b = (int64_t)a.num_heads * D * KV_ELEM_B;       // one token, all heads
  const uint32_t tile_b = (uint32_t)(kTile * row_b);                // the 16 token rows of a tile
  const uint32_t lane_voff = (uint32_t)(tl * row_b + (int64_t)head * D * KV_ELEM_B + dl * 16);
  const uint32_t group_b = (uint32_t)(TPL * row_b);
  const int tiles_per_block = a.block_size / kTile;                 // start is a multiple of the block size

  float m = -INFINITY, l = 0.f;
  float acc[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) acc[i] = 0.f;

  u32x4 kr[DEPTH][NG], vr[DEPTH][NG];
  bool ok[DEPTH];

  // Issue the loads of tile t; returns false if the tile does not exist or its block is unusable.
  auto load_tile = [&](int t, u32x4(&kq)[NG], u32x4(&vq)[NG]) -> bool {
    const bool in = t < n_tiles;
    const int tt = in ? t : 0;
    const int bi = tiles_per_block == 1 ? tt : tt / tiles_per_block;
    const int in_blk = tiles_per_block == 1 ? 0 : tt - bi * tiles_per_block;
    const int blk = __builtin_amdgcn_readlane(my_blk, bi);
    const int type = __builtin_amdgcn_readlane(my_type, bi);
    const bool ws = type != 0;
    const int64_t nblk = ws ? a.num_ws_blocks : a.num_cache_blocks;
    const bool valid = in && blk >= 0 && blk < nblk;
    const int64_t base = valid ? (int64_t)blk * (ws ? a.ws_block_stride_b : a.cache_block_stride_b) +
                                     (int64_t)in_blk * tile_b
                               : 0;
    const __amdgpu_buffer_rsrc_t rk = make_rsrc((ws ? a.ws_k_cache : a.k_cache) + base, valid ? tile_b : 0);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc((ws ? a.ws_v_cache : a.v_cache) + base, valid ? tile_b : 0);
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      kq[g] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rk, lane_voff + g * group_b, 0, 2));
      vq[g] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rv, lane_voff + g * group_b, 0, 2));
    }
    return valid;
  };

  auto consume_tile = [&](int t, const u32x4(&kq)[NG], const u32x4(&vq)[NG]) {
    const int tok0 = start + t * kTile;
    const bool partial = tok0 + kTile > end;
    float s[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      float d = 0.f;
      if constexpr (kDot2 && KV == KV_FP8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int kw = (int)kq[g][i];
          d = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(kw, 1.0f, false),
                                     __builtin_bit_cast(half2_t, qpk[2 * i]), d, false);
          d = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(kw, 1.0f, true),
                                     __builtin_bit_cast(half2_t, qpk[2 * i + 1]), d, false);
        }
      } else if constexpr (kDot2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t kw = kq[g][i], qw = qpk[i];
          if constexpr (KV == KV_F16)
            d = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, kw), __builtin_bit_cast(half2_t, qw), d, false);
          else
            d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, kw), __builtin_bit_cast(bf16x2_t, qw), d,
                                                false);
        }
      } else {
        float kf[EPL];
        Unpack<KV>::run(kq[g], kf);
#pragma unroll
        for (int i = 0; i < EPL; ++i) d = fmaf(qf[i], kf[i], d);
      }
      d = group_sum<LPT>(d) * a.scale_log2;
      s[g] = (tok0 + g * TPL + tl < end) ? d : -INFINITY;
    }
    float m_new = m;
#pragma unroll
    for (int g = 0; g < NG; ++g) m_new = fmaxf(m_new, s[g]);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    float p[NG];
    float psum = 0.f;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      p[g] = __builtin_amdgcn_exp2f(s[g] - m_use);
      psum += p[g];
    }
    l = fmaf(l, alpha, psum);   // (every multiply-add is spelled out: the same bits whichever kernel the code is inlined into)
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] *= alpha;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      float vf[EPL];
      Unpack<KV>::run(vq[g], vf);
      if (partial) {  // slots past the end of the sequence may hold anything, NaN included
        const bool live = tok0 + g * TPL + tl < end;
#pragma unroll
        for (int i = 0; i < EPL; ++i) vf[i] = live ? vf[i] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < EPL; ++i) acc[i] = fmaf(p[g], vf[i], acc[i]);
    }
    m = m_new;
  };

#pragma unroll
  for (int i = 0; i < DEPTH - 1; ++i) ok[i] = load_tile(i, kr[i], vr[i]);
  for (int t0 = 0; t0 < n_tiles; t0 += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      constexpr int kAhead = DEPTH - 1;
      const int fill = (j + kAhead) % DEPTH;
      ok[fill] = load_tile(t0 + j + kAhead, kr[fill], vr[fill]);
      if (ok[j]) consume_tile(t0 + j, kr[j], vr[j]);  // uniform; a tile that does not exist is never ok
    }
  }

  // merge the TPL token rows (lanes that share dl)
#pragma unroll
  for (int off = LPR; off < 64; off <<= 1) {
    const float m_o = __shfl_xor(m, off);
    const float l_o = __shfl_xor(l, off);
    const float m_n = fmaxf(m, m_o);
    const float m_u = (m_n == -INFINITY) ? 0.f : m_n;
    const float wa = __builtin_amdgcn_exp2f(m - m_u), wb = __builtin_amdgcn_exp2f(m_o - m_u);
    l = fmaf(l_o, wb, l * wa);
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] = fmaf(__shfl_xor(acc[i], off), wb, acc[i] * wa);
    m = m_n;
  }
  res.m = m;
  res.l = l;
#pragma unroll
  for (int i = 0; i < EPL; ++i) res.acc[i] = acc[i];
}

// Rounded result of lane (head, dl): acc * inv -> out[seq, head, dl*EPL ...]
template <int QT, int EPL, int D>
__device__ __forceinline__ void store_out(const AttnArgs& a, int seq, int head, int dl, const float (&acc)[EPL],
                                          float inv) {
  uint16_t* op = (uint16_t*)a.out + (int64_t)seq * a.out_stride + (int64_t)head * D + dl * EPL;
#pragma unroll
  for (int i = 0; i < EPL; i += 8) {
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      r[j] = (uint32_t)f32_to_q<QT>(acc[i + 2 * j] * inv) | ((uint32_t)f32_to_q<QT>(acc[i + 2 * j + 1] * inv) << 16);
    *(u32x4*)(op + i) = r;
  }
}

// Flat path: one wavefront (one 64-thread workgroup) per (head group, partition, sequence); partitions of one
// (sequence, head) are combined by combine_partitions_kernel.  Used when a sequence has more partitions than a
// workgroup has wavefronts.
template <int QT, int KV, int D, int HPW, int DEPTH>
__global__ __launch_bounds__(64) void paged_decode_kernel(const AttnArgs a) {
  constexpr int EPL = Unpack<KV>::EPL, LPT = D / EPL, LPR = LPT * HPW;
  const int part = blockIdx.y, seq = blockIdx.z, lane = threadIdx.x;
  const int seq_len = a.seq_lens[seq];
  const int start = part * a.partition_size;
  if (start >= seq_len && !(part == 0 && seq_len <= 0)) return;
  const int end = min(seq_len, start + a.partition_size);
  WaveResult<EPL> r;
  decode_wave<QT, KV, D, HPW, DEPTH>(a, seq, blockIdx.x * HPW, start, end, lane, r);
  if (lane >= LPR) return;
  const int head = blockIdx.x * HPW + lane / LPT, dl = lane % LPT;
  const float inv = (r.l > 0.f) ? a.v_scale / r.l : 0.f;
  if (a.num_partitions == 1) {
    store_out<QT, EPL, D>(a, seq, head, dl, r.acc, inv);
  } else {
    const int64_t ph = ((int64_t)seq * a.num_heads + head) * a.num_partitions + part;
    float* po = a.part_out + ph * D + dl * EPL;
#pragma unroll
    for (int i = 0; i < EPL; i += 4) {
      float4 v = make_float4(r.acc[i] * inv, r.acc[i + 1] * inv, r.acc[i + 2] * inv, r.acc[i + 3] * inv);
      *(float4*)(po + i) = v;
    }
    if (dl == 0) a.part_lse[ph] = (r.l > 0.f) ? r.m + log2f(r.l) : -INFINITY;
  }
}

constexpr int kRankInKernelMax = 512;  // up to this many sequences a workgroup ranks the lengths itself

// Group path: one workgroup per (head group, sequence); wavefront w walks partition w of the sequence and the
// wavefront that finishes last merges the partial results through LDS: no partials in HBM, no second launch.
// Wavefronts whose partition is empty leave at once (their registers and wave slot are free from then on).
// Workgroup rows are dealt out longest sequence first (list scheduling): the order comes from seq_order, or,
// for batches up to kRankInKernelMax, from ranking the lengths in LDS at the start of every workgroup.
// (the body takes its place in the grid as arguments: head group bx, workgroup row by)
template <int QT, int KV, int D, int HPW, int DEPTH, int WAVES>
__device__ __forceinline__ void paged_decode_group_body(const AttnArgs& a, const int bx, const int by) {
  constexpr int EPL = Unpack<KV>::EPL, LPT = D / EPL, LPR = LPT * HPW;
  __shared__ int s_arrived, s_seq;
  __shared__ int s_len[kRankInKernelMax];
  __shared__ float s_part[WAVES][LPR][EPL + 2];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;

  if (tid == 0) {
    s_arrived = 0;
    s_seq = a.seq_order ? a.seq_order[by] : by;
  }
  if (a.rank_in_kernel) {
    for (int j = tid; j < a.batch; j += 64 * WAVES) s_len[j] = a.seq_lens[j];
    __syncthreads();
    for (int j = tid; j < a.batch; j += 64 * WAVES) {
      const int mine = s_len[j];
      int rank = 0;
      for (int k = 0; k < a.batch; ++k) {
        const int other = s_len[k];
        rank += (other > mine || (other == mine && k < j)) ? 1 : 0;
      }
      if (rank == by) s_seq = j;
    }
  }
  __syncthreads();
  const int seq = s_seq;
  const int seq_len = a.rank_in_kernel ? s_len[seq] : a.seq_lens[seq];
  int np = (seq_len + a.partition_size - 1) / a.partition_size;
  np = np < 1 ? 1 : (np > WAVES ? WAVES : np);
  if (wave >= np) return;
  const int start = wave * a.partition_size;
  const int end = min(seq_len, start + a.partition_size);
  WaveResult<EPL> r;
  decode_wave<QT, KV, D, HPW, DEPTH>(a, seq, bx * HPW, start, end, lane, r);
  const int head = bx * HPW + lane / LPT, dl = lane % LPT;
  if (np == 1) {
    if (lane < LPR) store_out<QT, EPL, D>(a, seq, head, dl, r.acc, (r.l > 0.f) ? a.v_scale / r.l : 0.f);
    return;
  }
  if (lane < LPR) {
    float* sp = s_part[wave][lane];
    sp[0] = r.m;
    sp[1] = r.l;
#pragma unroll
    for (int i = 0; i < EPL; ++i) sp[2 + i] = r.acc[i];
  }
  // LDS operations of a wavefront execute in order, and the counter is an LDS atomic: whoever reads np - 1 has
  // every other wavefront's partial result in LDS already
  int arrived = 0;
  if (lane == 0) arrived = __hip_atomic_fetch_add(&s_arrived, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
  arrived = __builtin_amdgcn_readfirstlane(arrived);
  if (arrived != np - 1 || lane >= LPR) return;
  // fixed order of the merge (partition 0, 1, ...), whoever is last: the result does not depend on timing
  float m = -INFINITY;
  for (int p = 0; p < np; ++p) m = fmaxf(m, s_part[p][lane][0]);
  const float m_u = (m == -INFINITY) ? 0.f : m;
  float l = 0.f, acc[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) acc[i] = 0.f;
  for (int p = 0; p < np; ++p) {
    const float* sp = s_part[p][lane];
    const float w = __builtin_amdgcn_exp2f(sp[0] - m_u);
    l = fmaf(sp[1], w, l);
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] = fmaf(sp[2 + i], w, acc[i]);
  }
  store_out<QT, EPL, D>(a, seq, head, dl, acc, (l > 0.f) ? a.v_scale / l : 0.f);
}

template <int QT, int KV, int D, int HPW, int DEPTH, int WAVES>
__global__ __launch_bounds__(64 * WAVES)
void paged_decode_group_kernel(const AttnArgs a) {
  paged_decode_group_body<QT, KV, D, HPW, DEPTH, WAVES>(a, (int)blockIdx.x, (int)blockIdx.y);
}

#ifndef APS_HPW_F16
#define APS_HPW_F16 1
#endif
#ifndef APS_HPW_FP8
#define APS_HPW_FP8 2
#endif
// Tiles of 16 tokens a wavefront keeps in flight.  Measured at 128 sequences x 40 heads x 128, lognormal
// lengths: 2, 3 and 4 run within 2 % of each other (the kernel is not short of bytes in flight), and 2 keeps
// the register count low enough for four wavefronts per SIMD.
#ifndef APS_DEPTH_F16
#define APS_DEPTH_F16 2
#endif
#ifndef APS_DEPTH_FP8
#define APS_DEPTH_FP8 2
#endif

// wavefronts (= partitions of a sequence) of a group-path workgroup; 16 would cap the kernel at 128 registers
constexpr int kMaxGroupWaves = 8;

// Path and scratch of a problem, shared by the launcher and the workspace query.
struct DecodePlan {
  int64_t np;          // partitions of the longest sequence
  bool group;          // one workgroup per (head group, sequence), merge in LDS
  int waves;           // group path: wavefronts per workgroup
  bool sorted;         // group path: workgroup rows dealt out longest sequence first
  bool order_scratch;  // the order comes from rank_sequences_kernel (int32 per sequence in the scratch)
};


// A call of the decode attention that has been checked and planned but not launched (host side): what the
// launcher needs, and what a launch of another translation unit needs to take the group path's workgroups in.
constexpr uint32_t kPagedJobMagic = 0x4a445041u;
struct PagedJob {
  uint32_t magic;
  int head_size, q_dtype, kv_dtype;
  int64_t batch;       // 0: nothing to do
  DecodePlan plan;
  AttnArgs a;
};

#pragma clang fp contract(fast)   // (the compiler's default for device code, for what follows the include)

}  // namespace
}  // namespace aps
