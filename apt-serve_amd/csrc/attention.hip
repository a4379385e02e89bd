// Paged decode attention over a hybrid cache for gfx950.
//
// A wavefront owns (sequence, group of HPW adjacent heads, partition): a partition is a run of `partition_size`
// consecutive tokens of one sequence.  Lane layout for a head vector of D elements: LPT = D*elem_bytes/16 lanes
// hold one (token, head) (16 bytes each), the HPW heads of a token sit side by side, so one wave-wide 128-bit
// load covers TPL = 64/(LPT*HPW) tokens; a tile of 16 tokens (never crossing a block because the block size is a
// multiple of 16) takes NG = 16/TPL loads for K and NG for V.  Each of the TPL token rows of the wave runs its
// own online softmax over the tokens it sees (no cross-row traffic in the loop); rows are merged once at the end.
// DEPTH tiles are in flight per wavefront, requested through buffer descriptors so that no load sits under a
// branch.
//
// Per tile the K or V source is chosen per block: block_types[b][i] != 0 reads logical block i from the
// re-projection workspace, otherwise from the persistent K/V cache.
//
// Two ways to put the partitions of a (sequence, head group) together:
//   group path (a sequence has at most 8 partitions): one workgroup per (head group, sequence), wavefront w walks
//     partition w, and the wavefront that finishes last merges the partial results through LDS - one launch, no
//     partial results in HBM.  Workgroups are dealt out longest sequence first.
//   flat path (more partitions than a workgroup has wavefronts): one 64-thread workgroup per (head group,
//     partition, sequence) leaves fp32 partial results and their log-sum-exp; combine_partitions_kernel merges them.
#include <hip/hip_fp16.h>

#include <math.h>

#include <mutex>

#include "aps_common.h"
#include "mfma_common.h"

namespace aps {
namespace {

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
    l = l * alpha + psum;
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
    l = l * wa + l_o * wb;
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] = acc[i] * wa + __shfl_xor(acc[i], off) * wb;
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
template <int QT, int KV, int D, int HPW, int DEPTH, int WAVES>
__global__ __launch_bounds__(64 * WAVES)
void paged_decode_group_kernel(const AttnArgs a) {
  constexpr int EPL = Unpack<KV>::EPL, LPT = D / EPL, LPR = LPT * HPW;
  __shared__ int s_arrived, s_seq;
  __shared__ int s_len[kRankInKernelMax];
  __shared__ float s_part[WAVES][LPR][EPL + 2];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;

  if (tid == 0) {
    s_arrived = 0;
    s_seq = a.seq_order ? a.seq_order[blockIdx.y] : (int)blockIdx.y;
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
      if (rank == (int)blockIdx.y) s_seq = j;
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
  decode_wave<QT, KV, D, HPW, DEPTH>(a, seq, blockIdx.x * HPW, start, end, lane, r);
  const int head = blockIdx.x * HPW + lane / LPT, dl = lane % LPT;
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

// seq_order[r] = the sequence with the r-th longest length (ties by index): one thread per sequence.
__global__ __launch_bounds__(256) void rank_sequences_kernel(const int32_t* __restrict__ seq_lens, int batch,
                                                             int32_t* __restrict__ seq_order) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= batch) return;
  const int mine = seq_lens[j];
  int rank = 0;
  for (int k = 0; k < batch; ++k) {
    const int other = seq_lens[k];
    rank += (other > mine || (other == mine && k < j)) ? 1 : 0;
  }
  seq_order[rank] = j;
}

// out[b,h,:] = sum_p w_p * part_out[b,h,p,:] / sum_p w_p,  w_p = 2^(lse_p - max lse)
template <int QT>
__global__ __launch_bounds__(256) void combine_partitions_kernel(void* out, const float* part_out,
                                                                const float* part_lse, const int32_t* seq_lens,
                                                                int64_t out_stride, int num_heads, int head_size,
                                                                int num_partitions, int partition_size) {
  const int head = blockIdx.x, seq = blockIdx.y;
  const int seq_len = seq_lens[seq];
  int np = (seq_len + partition_size - 1) / partition_size;
  if (np < 1) np = 1;
  if (np > num_partitions) np = num_partitions;
  const int64_t ph = ((int64_t)seq * num_heads + head) * num_partitions;
  float mx = -INFINITY;
  for (int p = 0; p < np; ++p) mx = fmaxf(mx, part_lse[ph + p]);
  uint16_t* op = (uint16_t*)out + (int64_t)seq * out_stride + (int64_t)head * head_size;
  for (int d = threadIdx.x; d < head_size; d += blockDim.x) {
    float num = 0.f, den = 0.f;
    if (mx != -INFINITY) {
      for (int p = 0; p < np; ++p) {
        const float w = __builtin_amdgcn_exp2f(part_lse[ph + p] - mx);
        num = fmaf(w, part_out[(ph + p) * head_size + d], num);
        den += w;
      }
    }
    op[d] = f32_to_q<QT>(den > 0.f ? num / den : 0.f);
  }
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

inline DecodePlan plan_decode(int64_t batch, int num_heads, int64_t max_seq_len, int partition_size) {
  DecodePlan p{};
  p.np = (max_seq_len + partition_size - 1) / partition_size;
  if (p.np < 1) p.np = 1;
  p.group = p.np <= kMaxGroupWaves;
  p.waves = 1;
  while (p.waves < p.np) p.waves <<= 1;
  // more than one round of resident wavefronts (256 compute units x 16): the order of the workgroups decides
  // how long the last ones run alone
  p.sorted = p.group && batch > 1 && batch * num_heads * p.np > 4096;
  p.order_scratch = p.sorted && batch > kRankInKernelMax;
  return p;
}

template <int QT, int KV, int D, int HPW, int DEPTH>
void launch_group(const AttnArgs& a, int64_t batch, int waves, hipStream_t s) {
  const dim3 grid((unsigned)(a.num_heads / HPW), (unsigned)batch);
  switch (waves) {
    case 1: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 1>), grid, dim3(64), 0, s, a); break;
    case 2: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 2>), grid, dim3(128), 0, s, a); break;
    case 4: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 4>), grid, dim3(256), 0, s, a); break;
    default: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 8>), grid, dim3(512), 0, s, a); break;
  }
}

// Heads per wavefront: adjacent heads of one token are contiguous in memory, so HPW heads per wave make
// the contiguous piece a wave-wide load takes from one token row HPW times longer.
template <int QT, int KV, int D>
void launch_head_size(const AttnArgs& a, int64_t batch, const DecodePlan& plan, hipStream_t s) {
  constexpr int kWant = (KV == KV_FP8) ? APS_HPW_FP8 : APS_HPW_F16;
  constexpr int DEPTH = (KV == KV_FP8) ? APS_DEPTH_FP8 : APS_DEPTH_F16;
  constexpr int LPT = D / Unpack<KV>::EPL;
  constexpr int HPW = (LPT * kWant <= 32) ? kWant : 1;
  if constexpr (HPW > 1) {
    if (a.num_heads % HPW == 0) {
      if (plan.group) {
        launch_group<QT, KV, D, HPW, DEPTH>(a, batch, plan.waves, s);
      } else {
        const dim3 grid((unsigned)(a.num_heads / HPW), (unsigned)a.num_partitions, (unsigned)batch);
        APS_LAUNCH((paged_decode_kernel<QT, KV, D, HPW, DEPTH>), grid, dim3(64), 0, s, a);
      }
      return;
    }
  }
  if (plan.group) {
    launch_group<QT, KV, D, 1, DEPTH>(a, batch, plan.waves, s);
  } else {
    const dim3 grid((unsigned)a.num_heads, (unsigned)a.num_partitions, (unsigned)batch);
    APS_LAUNCH((paged_decode_kernel<QT, KV, D, 1, DEPTH>), grid, dim3(64), 0, s, a);
  }
}

template <int QT, int KV>
int launch_decode(const AttnArgs& a, int head_size, int64_t batch, const DecodePlan& plan, hipStream_t s) {
  if (plan.order_scratch) {
    APS_LAUNCH(rank_sequences_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, a.seq_lens,
                       (int)batch, const_cast<int32_t*>(a.seq_order));
    const int st = launch_status();
    if (st != APS_OK) return st;
  }
  switch (head_size) {
    case 64: launch_head_size<QT, KV, 64>(a, batch, plan, s); break;
    case 128: launch_head_size<QT, KV, 128>(a, batch, plan, s); break;
    case 256: launch_head_size<QT, KV, 256>(a, batch, plan, s); break;
    case 32:
      if constexpr (KV == KV_FP8) return APS_ERR_UNSUPPORTED;
      else launch_head_size<QT, KV, 32>(a, batch, plan, s);
      break;
    default: return APS_ERR_UNSUPPORTED;
  }
  int st = launch_status();
  if (st != APS_OK || plan.group || a.num_partitions == 1) return st;
  const int threads = head_size >= 256 ? 256 : (head_size + 63) / 64 * 64;
  APS_LAUNCH((combine_partitions_kernel<QT>), dim3((unsigned)a.num_heads, (unsigned)batch), dim3(threads), 0,
                     s, a.out, a.part_out, a.part_lse, a.seq_lens, a.out_stride, a.num_heads, head_size,
                     a.num_partitions, a.partition_size);
  return launch_status();
}

inline int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

int aps_decode_attention_partition_size(int64_t batch, int num_heads, int64_t max_seq_len, int block_size) {
  if (batch <= 0 || num_heads <= 0 || max_seq_len <= 0 || block_size <= 0) return 256;
  // Aim for a few thousand wavefronts (256 compute units x 8-16 resident waves);
  // shorten the partitions of small batches, never below two tiles.  512 tokens = at most four wavefronts per
  // workgroup for sequences up to 2048: workgroups of four pack the 12 or 16 wave slots of a compute unit
  // without a remainder (8-wavefront workgroups left a third of the slots empty with the fp8 kernel).
  int64_t part = 512;
  while (part > 32 && batch * num_heads * ((max_seq_len + part - 1) / part) < 4096) part >>= 1;
  if (part % block_size != 0) part = (part + block_size - 1) / block_size * block_size;
  // few sequences whose longest still fits the eight wavefronts of one workgroup at partitions of at most 128
  // tokens: take those instead, one launch whose partial results merge in LDS (5 sequences of up to 1000 tokens:
  // 19 against 23-25 us per call; with longer partitions a wavefront walks too many tiles one after the other:
  // one sequence of 2048 tokens, 32 against 23 us)
  if ((max_seq_len + part - 1) / part > kMaxGroupWaves) {
    const int64_t eighth = (max_seq_len + kMaxGroupWaves - 1) / kMaxGroupWaves;
    const int64_t gp = (eighth + block_size - 1) / block_size * block_size;
    if (gp <= 128) part = gp;
  }
  // plenty of sequences: lengthen the partitions until a sequence fits the wavefronts of one workgroup (the
  // partial results then merge in LDS), as far as the 64 block ids a wavefront holds allow
  if (batch * num_heads >= 1024)
    while ((max_seq_len + part - 1) / part > kMaxGroupWaves && 2 * part / block_size <= 64) part *= 2;
  return (int)part;
}

int64_t aps_decode_attention_workspace_bytes(int64_t batch, int num_heads, int head_size, int64_t max_seq_len,
                                             int partition_size) {
  if (batch <= 0 || num_heads <= 0 || head_size <= 0 || max_seq_len <= 0 || partition_size <= 0) return 0;
  const DecodePlan plan = plan_decode(batch, num_heads, max_seq_len, partition_size);
  if (plan.group) return plan.order_scratch ? align_up(batch * 4, 256) : 0;
  const int64_t n = batch * num_heads * plan.np;
  return align_up(n * head_size * 4, 256) + align_up(n * 4, 256);
}

// Both entry points: the scratch for the partial results is the caller's workspace or the library's static array.
static int decode_attention_impl(void* out, const void* q, const void* k_cache, const void* v_cache,
                                 const void* ws_k_cache, const void* ws_v_cache, const int32_t* block_tables,
                                 const uint8_t* block_types, const int32_t* seq_lens, int64_t batch, int num_heads,
                                 int head_size, int block_size, int64_t table_width, int64_t table_stride,
                                 int64_t types_stride, int64_t q_stride, int64_t out_stride,
                                 int64_t cache_block_stride, int64_t num_cache_blocks, int64_t ws_block_stride,
                                 int64_t num_ws_blocks, int64_t max_seq_len, int partition_size, float softmax_scale,
                                 int q_dtype, int kv_dtype, float k_scale, float v_scale, void* workspace,
                                 int64_t workspace_bytes, int too_small_status, aps_stream_t stream) {
  if (batch < 0 || num_heads <= 0 || head_size <= 0 || block_size <= 0 || table_width < 0) return APS_ERR_INVALID_ARG;
  if (batch == 0) return APS_OK;
  if (!out || !q || !seq_lens) return APS_ERR_INVALID_ARG;
  if (max_seq_len > 0 && (!k_cache || !v_cache || !block_tables)) return APS_ERR_INVALID_ARG;
  if (block_types && (!ws_k_cache || !ws_v_cache)) return APS_ERR_INVALID_ARG;
  if (block_size % kTile != 0) return APS_ERR_UNSUPPORTED;
  if (q_dtype != APS_F16 && q_dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  if (kv_dtype != q_dtype && kv_dtype != APS_FP8_E4M3) return APS_ERR_UNSUPPORTED;
  if (q_stride < (int64_t)num_heads * head_size || out_stride < (int64_t)num_heads * head_size)
    return APS_ERR_INVALID_ARG;
  const int kv_b = kv_dtype == APS_FP8_E4M3 ? 1 : 2;
  const int64_t row = (int64_t)num_heads * head_size;
  if (cache_block_stride < row * block_size || (block_types && ws_block_stride < row * block_size))
    return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(q), addr(out), (uint64_t)q_stride * 2, (uint64_t)out_stride * 2, addr(k_cache),
                        addr(v_cache), addr(ws_k_cache), addr(ws_v_cache), (uint64_t)cache_block_stride * kv_b,
                        (uint64_t)ws_block_stride * kv_b, (uint64_t)head_size * kv_b}) != 16)
    return APS_ERR_UNSUPPORTED;
  if (max_seq_len < 1) max_seq_len = 1;
  if (partition_size <= 0)
    partition_size = aps_decode_attention_partition_size(batch, num_heads, max_seq_len, block_size);
  if (partition_size % block_size != 0 || partition_size / block_size > 64) return APS_ERR_INVALID_ARG;
  const DecodePlan plan = plan_decode(batch, num_heads, max_seq_len, partition_size);
  const int64_t np = plan.np;
  if (np > 65535 || batch > 65535) return APS_ERR_UNSUPPORTED;

  AttnArgs a;
  a.out = out;
  a.q = q;
  a.k_cache = (const char*)k_cache; a.v_cache = (const char*)v_cache;
  a.ws_k_cache = (const char*)ws_k_cache; a.ws_v_cache = (const char*)ws_v_cache;
  a.block_tables = block_tables; a.block_types = block_types; a.seq_lens = seq_lens;
  a.q_stride = q_stride; a.out_stride = out_stride; a.table_stride = table_stride; a.types_stride = types_stride;
  a.cache_block_stride_b = cache_block_stride * kv_b; a.ws_block_stride_b = ws_block_stride * kv_b;
  a.num_cache_blocks = num_cache_blocks; a.num_ws_blocks = num_ws_blocks;
  a.num_heads = num_heads; a.block_size = block_size; a.partition_size = partition_size;
  a.num_partitions = (int)np; a.table_width = (int)table_width;
  const float ks = kv_dtype == APS_FP8_E4M3 ? k_scale : 1.f;
  a.scale_log2 = softmax_scale * ks * kLog2e;
  a.v_scale = kv_dtype == APS_FP8_E4M3 ? v_scale : 1.f;
  a.part_out = nullptr; a.part_lse = nullptr; a.seq_order = nullptr;
  a.batch = (int)batch;
  a.rank_in_kernel = plan.sorted && !plan.order_scratch;
  const int64_t need = aps_decode_attention_workspace_bytes(batch, num_heads, head_size, max_seq_len, partition_size);
  if (need > 0) {
    if (workspace && workspace_bytes < need) return too_small_status;
    if (!workspace || (addr(workspace) & 15)) return APS_ERR_WORKSPACE;
    if (plan.group) {
      a.seq_order = (const int32_t*)workspace;
    } else {
      const int64_t n = batch * num_heads * np;
      a.part_out = (float*)workspace;
      a.part_lse = (float*)((char*)workspace + align_up(n * head_size * 4, 256));
    }
  }
  hipStream_t s = (hipStream_t)stream;
  if (q_dtype == APS_F16) {
    return kv_dtype == APS_FP8_E4M3 ? launch_decode<APS_F16, KV_FP8>(a, head_size, batch, plan, s)
                                    : launch_decode<APS_F16, KV_F16>(a, head_size, batch, plan, s);
  }
  return kv_dtype == APS_FP8_E4M3 ? launch_decode<APS_BF16, KV_FP8>(a, head_size, batch, plan, s)
                                  : launch_decode<APS_BF16, KV_BF16>(a, head_size, batch, plan, s);
}

int aps_paged_decode_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                               const void* ws_k_cache, const void* ws_v_cache, const int32_t* block_tables,
                               const uint8_t* block_types, const int32_t* seq_lens, int64_t batch, int num_heads,
                               int head_size, int block_size, int64_t table_width, int64_t table_stride,
                               int64_t types_stride, int64_t q_stride, int64_t out_stride,
                               int64_t cache_block_stride, int64_t num_cache_blocks, int64_t ws_block_stride,
                               int64_t num_ws_blocks, int64_t max_seq_len, int partition_size, float softmax_scale,
                               int q_dtype, int kv_dtype, float k_scale, float v_scale, void* workspace,
                               int64_t workspace_bytes, aps_stream_t stream) {
  return decode_attention_impl(out, q, k_cache, v_cache, ws_k_cache, ws_v_cache, block_tables, block_types, seq_lens,
                               batch, num_heads, head_size, block_size, table_width, table_stride, types_stride,
                               q_stride, out_stride, cache_block_stride, num_cache_blocks, ws_block_stride,
                               num_ws_blocks, max_seq_len, partition_size, softmax_scale, q_dtype, kv_dtype, k_scale,
                               v_scale, workspace, workspace_bytes, APS_ERR_WORKSPACE, stream);
}

}  // extern "C"

// ---------------------------------------------------------------- the entry point that allocates nothing
// The partial results of split sequences live in a device array that is part of the library image: every GPU
// the library runs on holds its own copy until the process ends.  In host code the array's name is only a
// handle; the device address is looked up once per device and that pointer is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[APS_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices];  // device address of `scratch` on every device seen so far

// Device address of the scratch array on the current device (status != 0: the runtime's error code).
void* scratch_on_current_device(int* status) {
  *status = APS_OK;
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) { *status = (int)e; return nullptr; }
  if (device < 0 || device >= kMaxDevices) { *status = APS_ERR_UNSUPPORTED; return nullptr; }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[device]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) { *status = e != hipSuccess ? (int)e : APS_ERR_UNSUPPORTED; return nullptr; }
    scratch_ptr[device] = p;
  }
  return scratch_ptr[device];
}
}  // namespace

extern "C" int aps_paged_decode_attention_static(
    void* out, const void* q, const void* k_cache, const void* v_cache, const void* ws_k_cache,
    const void* ws_v_cache, const int32_t* block_tables, const uint8_t* block_types, const int32_t* seq_lens,
    int64_t batch, int num_heads, int head_size, int block_size, int64_t table_width, int64_t table_stride,
    int64_t types_stride, int64_t q_stride, int64_t out_stride, int64_t cache_block_stride, int64_t num_cache_blocks,
    int64_t ws_block_stride, int64_t num_ws_blocks, int64_t max_seq_len, int partition_size, float softmax_scale,
    int q_dtype, int kv_dtype, float k_scale, float v_scale, aps_stream_t stream) {
  int st = APS_OK;
  void* ws = scratch_on_current_device(&st);
  if (st != APS_OK) return st;
  return decode_attention_impl(out, q, k_cache, v_cache, ws_k_cache, ws_v_cache, block_tables, block_types, seq_lens,
                               batch, num_heads, head_size, block_size, table_width, table_stride, types_stride,
                               q_stride, out_stride, cache_block_stride, num_cache_blocks, ws_block_stride,
                               num_ws_blocks, max_seq_len, partition_size, softmax_scale, q_dtype, kv_dtype, k_scale,
                               v_scale, ws, APS_STATIC_SCRATCH_BYTES, APS_ERR_SCRATCH_LIMIT, stream);
}
