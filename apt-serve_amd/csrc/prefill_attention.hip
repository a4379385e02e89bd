// Causal attention over freshly projected, packed (varlen) q/k/v for gfx950 — the prompt step.
//
// One 256-thread workgroup owns 128 consecutive queries of one (sequence, head); each of its four
// wavefronts owns 32 of them.  Keys/values are consumed 64 at a time through LDS.
//
// The score tile is computed transposed, S^T = K Q^T, with v_mfma_f32_32x32x16: in the result layout
// a lane owns ONE query (column lane%32) and 16 of the 32 keys of a tile, so the running max / sum of
// the online softmax are per-lane scalars plus one exchange with lane^32.  The same registers, rounded
// to the operand dtype, are directly the B operand (k = keys) of O^T = V^T P^T, provided V^T is laid
// out in LDS in the key order the result layout produces:
//     position (key/16)*16 + ((key%8)/4)*8 + (key%16/8)*4 + key%4   holds   key.
// V is transposed on its way into LDS: a thread loads an 8x8 block (the 8 keys of one 16-byte run of stored
// positions, 8 consecutive d), transposes it in registers and stores 8 rows of V^T; K is staged row-major
// with its 16-byte chunks XOR-swizzled by key%16 so the fragment reads do not collide in the 64 banks.
// The next tile's pieces travel global -> registers while the current tile is multiplied.
//
// PAGED variant (a prompt step that continues a cached prefix: chunked prompts, prefix caching): the queries are
// the step's new tokens, the keys and values the whole sequence so far — prefix and new tokens alike — read from
// the paged K/V cache through the sequence's block table; query i of a sequence with qlen new tokens and klen
// tokens in all attends to keys 0 .. i + (klen - qlen).  Everything after the address of a key row is shared.
#include "aps_common.h"

#include <math.h>

namespace aps {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int BQ = 128;   // queries per workgroup
constexpr int BKV = 64;   // keys per iteration
constexpr int kThreads = 256;
constexpr float kLog2e = 1.4426950408889634f;

struct PrefillArgs {
  const char* q; const char* k; const char* v; char* out;
  const int32_t* cu_seqlens;
  int64_t q_stride_b, k_stride_b, v_stride_b, out_stride_b;  // token row strides in bytes
  int num_heads;
  int64_t num_tokens;  // rows of q / k / v / out: sequence boundaries outside [0, num_tokens] are not followed
  float scale_log2;
  // PAGED: k / v are [blocks, block_size, heads, D] caches, k_stride_b / v_stride_b their token row strides
  const int32_t* cu_seqlens_k; const int32_t* block_tables;
  int64_t table_stride, table_width, block_stride_b, num_blocks;
  int block_size;
};

template <bool BF16>
__device__ __forceinline__ float16v mfma32(const u32x4& a, const u32x4& b, const float16v& c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0,
                                                  0);
}

template <bool BF16>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  if constexpr (BF16) {
    auto cv = [](float x) -> uint32_t {
      uint32_t u = __float_as_uint(x);
      if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40;
      u += 0x7fffu + ((u >> 16) & 1u);
      return u >> 16;
    };
    return cv(a) | (cv(b) << 16);
  } else {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)a) |
           ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)b) << 16);
  }
}

template <bool BF16, int D, bool PAGED>
// Two wavefronts per SIMD: the kernel needs ~244 registers, and left to itself the compiler splits them into
// 244 + 64 accumulation registers, which leaves room for one.
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void prefill_attention_kernel(
    const PrefillArgs a) {
  constexpr int KS = D / 16;          // k-steps of the score product
  constexpr int DT = D / 32;          // 32-row tiles of O^T
  constexpr int KROW = D * 2;         // bytes per key row in LDS
  constexpr int KCH = KROW / 16;      // 16-byte chunks per key row
  // V^T in LDS: row d = 64 keys in stored order (8 chunks of 8 keys, 16 bytes each); chunk o of row d sits at
  // slot o ^ ((d/8 ^ d/2) % 8), and rows 64.. start 128 bytes (32 banks) later.  With that both the fragment
  // reads (16 lanes = 16 consecutive d, one chunk) and the transposed stores (16 lanes = rows 8 apart, one
  // chunk) touch 16 different 16-byte bank groups.
  constexpr int VROW = BKV * 2;
  __shared__ __attribute__((aligned(16))) char k_lds[BKV * KROW];
  __shared__ __attribute__((aligned(16))) char vt_lds[D * VROW + 128];
  auto vt_addr = [&](int d, int chunk) {
    return vt_lds + d * VROW + ((d >> 6) << 7) + ((chunk ^ (((d >> 3) ^ (d >> 1)) & 7)) << 4);
  };

  // Grid (head, sequence, query tile), the last query tiles first: under the causal mask a workgroup's work grows
  // with its tile's position, and workgroups start in grid order, so the long ones go first and the short ones
  // fill the end (list scheduling).
  const int seq = blockIdx.y, head = blockIdx.x;
  const int s0 = a.cu_seqlens[seq], s1 = a.cu_seqlens[seq + 1];
  if (s0 < 0 || s1 < s0 || s1 > a.num_tokens) return;  // boundaries come from device memory: never follow bad ones
  const int qlen = s1 - s0;          // queries of this sequence in this step
  int len = qlen;                    // keys: the same tokens, or (PAGED) everything cached so far
  if constexpr (PAGED) {
    len = a.cu_seqlens_k[seq + 1] - a.cu_seqlens_k[seq];
    if (len < qlen || (int64_t)(len + a.block_size - 1) / a.block_size > a.table_width) return;
  }
  const int off = len - qlen;        // query i sees keys 0 .. i + off
  const int q0 = (int)(gridDim.z - 1 - blockIdx.z) * BQ;
  if (q0 >= qlen) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int qcol = lane & 31, half = lane >> 5;
  const int my_q = q0 + wave * 32 + qcol;      // query index inside the sequence's new tokens (may be >= qlen)
  const bool q_live = my_q < qlen;

  // Q^T fragments: B operand, lane = (query, 8 consecutive d of each 16-wide k-step)
  u32x4 qf[KS];
  {
    const char* qp = a.q + (int64_t)(s0 + (q_live ? my_q : qlen - 1)) * a.q_stride_b + (int64_t)head * D * 2;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *(const u32x4*)(qp + (16 * s + 8 * half) * 2);
  }

  float16v o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // Staging.  K: thread tid moves the 16-byte pieces tid + 256*j of the tile (row-major, swizzled).  V: thread
  // (octet o, d-chunk ch), o = tid / KCH < 8, loads the 8 keys whose stored positions are 8o .. 8o+7 (16 bytes = 8 d
  // each: 16 lanes read 256 contiguous bytes of a key row), transposes the 8x8 block in registers with v_perm and
  // stores 8 rows d of 16 bytes (8 keys).  The pieces of the next tile are loaded into registers before the
  // current tile is multiplied and written to LDS after it.
  constexpr int PER_K = BKV * KCH / kThreads;
  const bool v_thread = tid < 8 * KCH;           // whole wavefronts
  const int vo = tid / KCH, vch = tid % KCH;
  const char* k_base = a.k + (PAGED ? 0 : (int64_t)s0 * a.k_stride_b) + (int64_t)head * D * 2;
  const char* v_base = a.v + (PAGED ? 0 : (int64_t)s0 * a.v_stride_b) + (int64_t)head * D * 2 + vch * 16;
  // byte offset of key gk of the sequence from k_base / v_base (`stride_b`: the operand's token row stride)
  auto key_off = [&](int gk, int64_t stride_b) -> int64_t {
    if constexpr (PAGED) {
      const int bi = gk / a.block_size;
      int64_t blk = a.block_tables[(int64_t)seq * a.table_stride + bi];
      blk = blk < 0 ? 0 : (blk >= a.num_blocks ? a.num_blocks - 1 : blk);  // a bad table: wrong numbers, no fault
      return blk * a.block_stride_b + (int64_t)(gk - bi * a.block_size) * stride_b;
    } else {
      return (int64_t)gk * stride_b;
    }
  };
  u32x4 kreg[PER_K], vreg[8];
  auto fetch_tile = [&](int kv0) {
#pragma unroll
    for (int j = 0; j < PER_K; ++j) {
      const int c = tid + j * kThreads;
      const int key = c / KCH, ch = c % KCH;
      const int gk = min(kv0 + key, len - 1);
      kreg[j] = *(const u32x4*)(k_base + key_off(gk, a.k_stride_b) + ch * 16);
    }
    if (v_thread) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {  // stored position 8*vo + j holds this key (see the file comment)
        const int key = (vo >> 1) * 16 + (vo & 1) * 4 + (j & 3) + (j >> 2) * 8;
        const int gk = min(kv0 + key, len - 1);
        vreg[j] = *(const u32x4*)(v_base + key_off(gk, a.v_stride_b));
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < PER_K; ++j) {
      const int c = tid + j * kThreads;
      const int key = c / KCH, ch = c % KCH;
      *(u32x4*)(k_lds + key * KROW + ((ch ^ (key & (KCH - 1) & 15)) * 16)) = kreg[j];
    }
    if (v_thread) {
#pragma unroll
      for (int dd = 0; dd < 8; ++dd) {  // row d = 8*vch + dd: dword p = (key position 2p, 2p+1)
        const uint32_t sel = (dd & 1) ? 0x07060302u : 0x05040100u;
        u32x4 col;
#pragma unroll
        for (int p4 = 0; p4 < 4; ++p4)
          col[p4] = __builtin_amdgcn_perm(vreg[2 * p4 + 1][dd >> 1], vreg[2 * p4][dd >> 1], sel);
        *(u32x4*)vt_addr(vch * 8 + dd, vo) = col;
      }
    }
  };

  const int kv_end = min(len, q0 + BQ + off);  // causal: keys beyond the tile's last query are never needed
  const int wave_q0 = q0 + wave * 32 + off;    // last key the first query of this wavefront sees
  fetch_tile(0);
  for (int kv0 = 0; kv0 < kv_end; kv0 += BKV) {
    __syncthreads();  // previous tile fully consumed
    store_tile();
    __syncthreads();
    if (kv0 + BKV < kv_end) fetch_tile(kv0 + BKV);  // in flight while this tile is multiplied
    if (kv0 > wave_q0 + 31) continue;               // every key of the tile lies after this wavefront's queries

    // ---- S^T = K Q^T for the two 32-key tiles
    float16v st[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int e = 0; e < 16; ++e) st[t][e] = 0.f;
      const int key = t * 32 + qcol;  // A operand row of this lane
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int ch = 2 * s + half;
        const u32x4 kf = *(const u32x4*)(k_lds + key * KROW + ((ch ^ (key & (KCH - 1) & 15)) * 16));
        st[t] = mfma32<BF16>(kf, qf[s], st[t]);
      }
    }
    // ---- online softmax for this lane's query (its 32 keys here, the other 32 in lane^32)
    // Only a tile that reaches past the wavefront's first query or past the sequence needs the mask.
    // The maximum is taken on the raw scores (the scale is positive) and the scale goes into the exponent's
    // fused multiply-add: max, fma, exp2 and add per score, nothing else.
    const bool masked = kv0 + BKV - 1 > wave_q0 || kv0 + BKV > len;
    float mx = m_run;   // raw-score domain
    if (masked) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = kv0 + t * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
          if (!(key <= my_q + off && key < len)) st[t][e] = -INFINITY;
        }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) mx = fmaxf(mx, st[t][e]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_use = (mx == -INFINITY) ? 0.f : mx;
    const float neg_m = -m_use * a.scale_log2;
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float p = __builtin_amdgcn_exp2f(fmaf(st[t][e], a.scale_log2, neg_m));
        st[t][e] = p;
        psum += p;
      }
    psum += __shfl_xor(psum, 32);
    // the running maximum rarely moves after the first tiles: rescale O only when some query of the wavefront
    // needs it (a wave-uniform branch)
    const bool moved = mx != m_run;
    if (__builtin_amdgcn_ballot_w64(moved) != 0) {
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * a.scale_log2);
      l_run *= alpha;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
    }
    l_run += psum;
    m_run = mx;
    // ---- O^T += V^T P^T : four k-steps of 16 keys; P^T fragment = 8 consecutive result registers
#pragma unroll
    for (int t32 = 0; t32 < 2; ++t32)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        u32x4 pf;
#pragma unroll
        for (int i = 0; i < 4; ++i) pf[i] = pack2<BF16>(st[t32][8 * ks + 2 * i], st[t32][8 * ks + 2 * i + 1]);
        const int chunk = (t32 * 2 + ks) * 2 + half;  // this lane's 8 keys of the step, in stored order
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          const u32x4 vf = *(const u32x4*)vt_addr(t * 32 + qcol, chunk);
          o[t] = mfma32<BF16>(vf, pf, o[t]);
        }
      }
  }

  // ---- normalise and store: lane owns query my_q, rows d = 32 t + 8 (e/4) + 4 half + e%4
  if (!q_live) return;
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  char* op = a.out + (int64_t)(s0 + my_q) * a.out_stride_b + (int64_t)head * D * 2;
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = 32 * t + 8 * g + 4 * half;
      uint2 w;
      w.x = pack2<BF16>(o[t][4 * g] * inv, o[t][4 * g + 1] * inv);
      w.y = pack2<BF16>(o[t][4 * g + 2] * inv, o[t][4 * g + 3] * inv);
      *(uint2*)(op + d * 2) = w;
    }
}

}  // namespace
}  // namespace aps

using namespace aps;

namespace {
int launch_prefill(PrefillArgs& a, bool paged, int64_t num_seqs, int64_t max_seqlen_q, int num_heads, int head_size,
                   int dtype, aps_stream_t stream) {
  const int64_t q_tiles = (max_seqlen_q + BQ - 1) / BQ;
  if (q_tiles > 65535 || num_seqs > 65535 || num_heads > 65535) return APS_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)num_heads, (unsigned)num_seqs, (unsigned)q_tiles);
  hipStream_t s = (hipStream_t)stream;
#define APS_LAUNCH_PF(B, D_, P) APS_LAUNCH((prefill_attention_kernel<B, D_, P>), grid, dim3(kThreads), 0, s, a)
#define APS_LAUNCH_PF_D(B, P)                                        \
  do {                                                               \
    if (head_size == 64) APS_LAUNCH_PF(B, 64, P); else APS_LAUNCH_PF(B, 128, P); \
  } while (0)
  if (paged) {
    if (dtype == APS_F16) APS_LAUNCH_PF_D(false, true); else APS_LAUNCH_PF_D(true, true);
  } else {
    if (dtype == APS_F16) APS_LAUNCH_PF_D(false, false); else APS_LAUNCH_PF_D(true, false);
  }
#undef APS_LAUNCH_PF_D
#undef APS_LAUNCH_PF
  return launch_status();
}
}  // namespace

extern "C" {

int aps_varlen_prefill_attention(void* out, const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                                 int64_t num_seqs, int64_t num_tokens, int64_t max_seqlen, int num_heads,
                                 int head_size, int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t out_stride,
                                 float softmax_scale, int dtype, aps_stream_t stream) {
  if (num_seqs < 0 || num_tokens < 0 || max_seqlen < 0 || num_heads <= 0 || head_size <= 0) return APS_ERR_INVALID_ARG;
  // the running maximum is taken on raw scores and the scale folded into the exponent: a positive, finite scale only
  if (!(softmax_scale > 0.f) || softmax_scale > 3.0e38f) return APS_ERR_INVALID_ARG;
  if (num_seqs == 0 || num_tokens == 0 || max_seqlen == 0) return APS_OK;
  if (!out || !q || !k || !v || !cu_seqlens) return APS_ERR_INVALID_ARG;
  if (dtype != APS_F16 && dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  if (head_size != 64 && head_size != 128) return APS_ERR_UNSUPPORTED;
  const int64_t row = (int64_t)num_heads * head_size;
  if (q_stride < row || k_stride < row || v_stride < row || out_stride < row) return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(q), addr(k), addr(v), (uint64_t)q_stride * 2, (uint64_t)k_stride * 2,
                        (uint64_t)v_stride * 2}) != 16 ||
      common_vec_bytes({addr(out), (uint64_t)out_stride * 2}) < 8)
    return APS_ERR_UNSUPPORTED;
  PrefillArgs a{};
  a.q = (const char*)q; a.k = (const char*)k; a.v = (const char*)v; a.out = (char*)out;
  a.cu_seqlens = cu_seqlens;
  a.q_stride_b = q_stride * 2; a.k_stride_b = k_stride * 2; a.v_stride_b = v_stride * 2; a.out_stride_b = out_stride * 2;
  a.num_heads = num_heads;
  a.num_tokens = num_tokens;
  a.scale_log2 = softmax_scale * kLog2e;
  return launch_prefill(a, false, num_seqs, max_seqlen, num_heads, head_size, dtype, stream);
}

int aps_paged_prefill_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                const int32_t* block_tables, const int32_t* cu_seqlens_q,
                                const int32_t* cu_seqlens_k, int64_t num_seqs, int64_t num_q_tokens,
                                int64_t max_seqlen_q, int num_heads, int head_size, int block_size,
                                int64_t table_stride, int64_t table_width, int64_t q_stride, int64_t out_stride,
                                int64_t cache_block_stride, int64_t num_cache_blocks, float softmax_scale, int dtype,
                                aps_stream_t stream) {
  if (num_seqs < 0 || num_q_tokens < 0 || max_seqlen_q < 0 || num_heads <= 0 || head_size <= 0 || block_size <= 0 ||
      table_width < 0 || num_cache_blocks < 0)
    return APS_ERR_INVALID_ARG;
  if (!(softmax_scale > 0.f) || softmax_scale > 3.0e38f) return APS_ERR_INVALID_ARG;
  if (num_seqs == 0 || num_q_tokens == 0 || max_seqlen_q == 0) return APS_OK;
  if (!out || !q || !k_cache || !v_cache || !block_tables || !cu_seqlens_q || !cu_seqlens_k || num_cache_blocks == 0)
    return APS_ERR_INVALID_ARG;
  if (dtype != APS_F16 && dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  if (head_size != 64 && head_size != 128) return APS_ERR_UNSUPPORTED;
  const int64_t row = (int64_t)num_heads * head_size;
  if (q_stride < row || out_stride < row || cache_block_stride < row * block_size || table_stride < table_width)
    return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(q), addr(k_cache), addr(v_cache), (uint64_t)q_stride * 2,
                        (uint64_t)cache_block_stride * 2}) != 16 ||
      common_vec_bytes({addr(out), (uint64_t)out_stride * 2}) < 8)
    return APS_ERR_UNSUPPORTED;
  PrefillArgs a{};
  a.q = (const char*)q; a.k = (const char*)k_cache; a.v = (const char*)v_cache; a.out = (char*)out;
  a.cu_seqlens = cu_seqlens_q; a.cu_seqlens_k = cu_seqlens_k; a.block_tables = block_tables;
  a.q_stride_b = q_stride * 2; a.k_stride_b = row * 2; a.v_stride_b = row * 2; a.out_stride_b = out_stride * 2;
  a.table_stride = table_stride; a.table_width = table_width;
  a.block_stride_b = cache_block_stride * 2; a.num_blocks = num_cache_blocks; a.block_size = block_size;
  a.num_heads = num_heads;
  a.num_tokens = num_q_tokens;
  a.scale_log2 = softmax_scale * kLog2e;
  return launch_prefill(a, true, num_seqs, max_seqlen_q, num_heads, head_size, dtype, stream);
}

}  // extern "C"
