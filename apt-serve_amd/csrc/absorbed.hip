// Decode attention of hidden-cached sequences computed on the cached hidden rows themselves
// ("absorbed" projection weights), for gfx950.
//
// For a hidden-cached sequence the K and V of a context token are W_k h_t + b_k and W_v h_t + b_v.
// Instead of re-projecting every cached row in every layer,
//     s[h][t] = scale * <W_k[h]^T q[h], h_t>      (the b_k term is the same for all t: softmax drops it)
//     out[h]  = W_v[h] (sum_t p[h][t] h_t) + b_v[h]
// so the hidden rows are read twice (scores, then the weighted sum) and the projections shrink to
// products with one row per sequence and head:
//   1. qt[s][h][:]  = scale*log2(e) * W_k[h]^T q[s][h]     query_image_kernel (a head's slab of W_k in registers; one
//                                                            extra workgroup plans the ragged batch for the kernels
//                                                            below); heads wider than 128: nn_few_rows_kernel and
//                                                            seq_plan_kernel
//   2. S[s][h][t]   = <qt[s][h], h_t>  (fp32)               hidden_scores_kernel: tiles of 128 cached rows through
//                                                            the row-streaming MFMA core, K in parts for small
//                                                            batches (score_parts_sum_kernel adds them)
//   3. ctx[s][h][:] = sum_t softmax_t(S[s][h])[t] h_t        hidden_wsum_kernel: one pass over the rows with the
//                                                            online softmax inside (long sequences in partitions);
//                                                            few cached rows in all: hidden_wsum_chunk_kernel, one
//                                                            96-token chunk per workgroup; wsum_combine_kernel
//                                                            merges partitions / chunks
//   4. out[s][h*D+d] = <W_v[h*D+d], ctx[s][h]> + b_v         head_proj_kernel; up to 16 sequences: the
//                                                            weight-streaming kernels of the projection file, x
//                                                            chosen per head
// A decode step's other work can share these launches (aps_hybrid_decode_attention): the step's cache writes
// ride beside the absorbed queries, the paged attention of the K/V-cached sequences beside the chunked sum.
// Per cached token and layer that is 2 x Hd x 2 bytes of HBM reads and ~4*H*Hd flops, against a
// gather, a 4*Hd*Hd-flop GEMM, a cache write and an attention read for the re-projection flow.
#include <type_traits>

#include "aps_common.h"
#include "mfma_common.h"
#include "paged_decode_core.h"
#include "row_mover_core.h"
#include "row_stream_core.h"

// the per-head value projection lives with the other weight-streaming kernels
__attribute__((visibility("hidden"))) int aps_internal_headwise_linear(
    const void* x, const void* weight, const void* bias, void* out, int64_t m, int64_t n, int64_t k, int64_t x_stride,
    int64_t x_head_stride, int head_rows, int64_t w_stride, int64_t out_stride, const int64_t* out_row_map,
    int64_t out_rows, int dtype, void* workspace, int64_t workspace_bytes, int32_t* tile_counters, hipStream_t stream);
// bytes of fp32 partial products that call uses for m rows (0: it runs a kernel that needs none)
__attribute__((visibility("hidden"))) int64_t aps_internal_headwise_workspace_bytes(int64_t m, int64_t n, int64_t k,
                                                                                   int head_rows);
// a planned paged decode attention, launched by itself (the attention launcher's translation unit)
extern "C" int aps_attention_job_launch(const void* job, aps_stream_t stream);
// a decode step's planned cache writes, launched by themselves (the cache operators' translation unit)
extern "C" int aps_cache_job_launch(const void* job, aps_stream_t stream);

namespace aps {
namespace {

// ------------------------------------------------------------------ NN product with few rows (wide heads)
// out[z][m][n] = alpha * sum_k A[z][m][k] * B[z*k_fixed + k][n],  m < m_rows (tiles of 16*MT rows), k < k_fixed:
// the absorbed queries of heads wider than 128 (query_image_kernel keeps a head's whole slab of W_k in registers
// and stops there).  B rows are n-contiguous; A is K-contiguous, row m of A is row a_row_ids[m].
//
// The matrix core wants, per lane, 8 consecutive k of one column.  A lane therefore loads an 8x8
// block (8 rows k, 16 bytes = 8 columns each; the 16 lanes of a quarter-wave read 256 contiguous
// bytes of a row), transposes it in registers with v_perm_b32 and feeds 8 MFMAs, MFMA j taking
// column 8c+j from lane (g, c).  No LDS for the data; a workgroup of 4 wavefronts covers 512 columns.
struct NnArgs {
  const char* a; int64_t a_batch_stride_b, lda_b; int m_rows;
  const int64_t* a_row_ids; int64_t num_a_rows;
  const char* b; int64_t b_row_stride_b, num_b_rows;
  int k_fixed;
  int64_t n;
  char* out; int64_t out_batch_stride, out_row_stride;  // elements
  int batches, m_tiles;
  float alpha;
};

constexpr int kNnWaves = 4;
constexpr int kNnRing = 3;

template <bool BF16, int MT>
__global__ __launch_bounds__(kNnWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void nn_few_rows_kernel(
    const NnArgs g) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int z = blockIdx.y / g.m_tiles;
  const int m0 = (blockIdx.y % g.m_tiles) * (16 * MT);
  const int kend = g.k_fixed;
  const int64_t col0 = (int64_t)blockIdx.x * (kNnWaves * 128) + wave * 128 + 8 * c;
  const bool col_ok = col0 < g.n;
  const char* a_base = g.a + (int64_t)z * g.a_batch_stride_b;  // uniform; rows of a batch lie within 4 GiB of it
  uint32_t a_off[MT];
  bool a_ok[MT];
#pragma unroll
  for (int ht = 0; ht < MT; ++ht) {
    const int m = m0 + 16 * ht + c;
    a_ok[ht] = m < g.m_rows;
    int64_t arow = 0;
    if (a_ok[ht]) {
      arow = g.a_row_ids[m];
      a_ok[ht] = arow >= 0 && arow < g.num_a_rows;
    }
    if (!a_ok[ht]) arow = 0;  // a row that exists; its product is discarded
    a_off[ht] = (uint32_t)(arow * g.lda_b + g4 * 16);
  }
  float4v acc[MT][8];
#pragma unroll
  for (int ht = 0; ht < MT; ++ht)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[ht][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // Loads are unconditional (a row or column that does not exist reads row 0 / column 0 and is replaced by
  // zeros afterwards): with per-lane branches around them the wait counts before the MFMAs degrade to
  // "everything outstanding", which serialises the register sets.
  const char* b_col = g.b + (col_ok ? col0 : 0) * 2;
  auto load_step = [&](int t0, u32x4(&r)[8], u32x4(&pf)[MT], uint32_t& bad) {
    bad = 0;  // bit i: row i of this lane does not exist; applied when the block is consumed
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t row = (int64_t)z * g.k_fixed + t0 + 8 * g4 + i;
      const bool ok = col_ok && (t0 + 8 * g4 + i < kend) && row < g.num_b_rows;
      if (!ok) bad |= 1u << i;
      r[i] = __builtin_nontemporal_load((const u32x4*)(b_col + (ok ? row : 0) * g.b_row_stride_b));
    }
#pragma unroll
    for (int ht = 0; ht < MT; ++ht) pf[ht] = *(const u32x4*)(a_base + (a_off[ht] + (uint32_t)t0 * 2));
  };
  auto mac_step = [&](u32x4(&r)[8], u32x4(&pf)[MT], uint32_t bad) {
    if (__builtin_amdgcn_ballot_w64(bad != 0) != 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (bad & (1u << i)) r[i] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int ht = 0; ht < MT; ++ht)
      if (!a_ok[ht]) pf[ht] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // column j of the 8x8 block: dword p = (row 2p, row 2p+1)
      u32x4 tcol;
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const uint32_t lo = r[2 * p][j >> 1], hi = r[2 * p + 1][j >> 1];
        tcol[p] = __builtin_amdgcn_perm(hi, lo, sel);
      }
#pragma unroll
      for (int ht = 0; ht < MT; ++ht) acc[ht][j] = mfma16<BF16>(pf[ht], tcol, acc[ht][j]);
    }
  };

  // ring of kNnRing row blocks: two steps (16 KiB per wavefront) are in flight while one is multiplied
  u32x4 r[kNnRing][8], pf[kNnRing][MT];
  uint32_t bad[kNnRing];
  int t0 = 0;
#pragma unroll
  for (int d = 0; d < kNnRing - 1; ++d)
    if (t0 + 32 * d < kend) load_step(t0 + 32 * d, r[d], pf[d], bad[d]);
  while (t0 < kend) {
#pragma unroll
    for (int u = 0; u < kNnRing; ++u) {
      if (t0 < kend) {
        const int ahead = t0 + 32 * (kNnRing - 1);
        if (ahead < kend) load_step(ahead, r[(u + kNnRing - 1) % kNnRing], pf[(u + kNnRing - 1) % kNnRing],
                                    bad[(u + kNnRing - 1) % kNnRing]);
        mac_step(r[u], pf[u], bad[u]);
        t0 += 32;
      }
    }
  }

  // lane (g4, c) holds rows 16*ht + 4*g4 + i and columns col0 .. col0+7 (MFMA j = column j)
  if (!col_ok) return;
#pragma unroll
  for (int ht = 0; ht < MT; ++ht)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 16 * ht + 4 * g4 + i;
      if (m >= g.m_rows) continue;
      uint16_t h[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float v = acc[ht][j][i] * g.alpha;
        h[j] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
      }
      u32x4 o;
#pragma unroll
      for (int p = 0; p < 4; ++p) o[p] = (uint32_t)h[2 * p] | ((uint32_t)h[2 * p + 1] << 16);
      *(u32x4*)(g.out + ((int64_t)z * g.out_batch_stride + (int64_t)m * g.out_row_stride + col0) * 2) = o;
    }
}

// ------------------------------------------------------------------ scores over paged hidden rows
// S[z][h][t] = sum_k hidden[row_ids[row_start[z] + t]][k] * qt[z][h][k]  (fp32), t < L(z).
// One workgroup = 128 tokens (8 wavefronts x 16) of one sequence x all heads x a part of K (all of it unless the
// batch has few tiles), on the row-streaming core: the hidden rows are the streamed operand, the absorbed
// queries qt[z] the LDS image.
struct ScoreArgs {
  const char* cache; int64_t slot_stride_b, num_slots;
  const int64_t* row_ids; const int64_t* row_start;
  const char* qt; int64_t qt_batch_stride_b, qt_row_stride_b; int heads;
  float* s; int64_t s_batch_stride, s_row_stride;  // elements
  int64_t k;
  const int32_t* tile_start; int n_seqs;  // tile_start[z] = tiles of the sequences before z (n_seqs + 1 entries)
  int64_t k_per_part, s_part_stride;      // blockIdx.y = part of K (whole image chunks); partial scores per part
};


// One workgroup plans the ragged batch:
//   tile_start[z] = sum over y < z of ceil(L(y) / tile_tokens)   (n_seqs + 1 entries; the scores kernel's work list)
//   order[r]      = the sequence with the r-th most rows, ties by index (nullable).  A workgroup of the weighted
//                   sum works through all rows of its sequence and workgroups start in grid order: longest first
//                   keeps the last ones short (list scheduling: within a few % of ideal instead of 20-35 % over).
constexpr int kMaxOrderedSeqs = 4096;  // lengths are ranked out of LDS, quadratic work; larger batches balance anyway
__device__ __forceinline__ void plan_ragged_batch(const int64_t* __restrict__ row_start, int n_seqs, int tile_tokens,
                                                  int32_t* __restrict__ tile_start, int32_t* __restrict__ order,
                                                  u32x4* __restrict__ zero_row, int zero_vecs) {
  // the row of zeros that tokens without a cached row read in the weighted sum; behind it (same region of the
  // workspace, counted in zero_vecs) the arrival counters of the value projection's K split
  for (int i = threadIdx.x; i < zero_vecs; i += 256) zero_row[i] = u32x4{0u, 0u, 0u, 0u};
  __shared__ int32_t part[256];
  __shared__ int32_t carry;
  __shared__ int32_t lens[kMaxOrderedSeqs];
  if (threadIdx.x == 0) { carry = 0; tile_start[0] = 0; }
  __syncthreads();
  for (int base = 0; base < n_seqs; base += 256) {
    const int y = base + threadIdx.x;
    int v = 0;
    if (y < n_seqs) {
      const int64_t len = row_start[y + 1] - row_start[y];
      v = (int)((len + tile_tokens - 1) / tile_tokens);
      if (order) lens[y] = (int32_t)len;
    }
    part[threadIdx.x] = v;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {  // inclusive scan
      const int add = (int)threadIdx.x >= d ? part[threadIdx.x - d] : 0;
      __syncthreads();
      part[threadIdx.x] += add;
      __syncthreads();
    }
    if (y < n_seqs) tile_start[y + 1] = carry + part[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) carry += part[255];
    __syncthreads();
  }
  if (!order) return;
  for (int z = threadIdx.x; z < n_seqs; z += 256) {
    const int len = lens[z];
    int rank = 0;
    for (int y = 0; y < n_seqs; ++y) rank += (lens[y] > len || (lens[y] == len && y < z)) ? 1 : 0;
    order[rank] = z;
  }
}

__global__ __launch_bounds__(256) void seq_plan_kernel(const int64_t* __restrict__ row_start, int n_seqs,
                                                       int tile_tokens, int32_t* __restrict__ tile_start,
                                                       int32_t* __restrict__ order, u32x4* __restrict__ zero_row,
                                                       int zero_vecs) {
  plan_ragged_batch(row_start, n_seqs, tile_tokens, tile_start, order, zero_row, zero_vecs);
}

// ------------------------------------------------------------------ absorbed queries
// qt[s][h][n] = alpha * sum_d q[seq_rows[s]][h*D + d] * W_k[h*D + d][n]:  per head a product of few rows (the
// sequences) with the head's D rows of W_k.  A wavefront owns (head, 128 columns): it loads its D x 128 slab of W_k
// once — all loads in flight together, 32 KiB per wavefront — keeps it in registers in MFMA operand order (8x8
// blocks transposed with v_perm_b32) and then walks the sequences 16 at a time.  W_k crosses HBM once whatever the
// number of sequences (the generic kernel re-read it for every 48 sequences and kept 4 of its D rows per lane in
// flight).  KS = D / 32 <= 4.  One extra workgroup (blockIdx.y == heads) plans the ragged batch for the kernels
// that follow (the scores kernel's tile list, the weighted sum's longest-first order) instead of a launch of its own.
struct QImageArgs {
  const char* q; int64_t q_stride_b; const int64_t* seq_rows; int64_t num_q_rows; int n_seqs;
  const char* w; int64_t w_stride_b;
  int heads; int64_t hidden;
  char* qt;
  float alpha;
  const int64_t* row_start; int tile_tokens; int32_t* tile_start; int32_t* order;
  u32x4* zero_row; int zero_vecs;
};

// The rows of the grid in front of the heads' rows hold the launch's other work, one workgroup each in the
// grid's linear order: first the plan, then (a launch that has a decode step's cache writes on board) the row
// mover's workgroups.  Those writes touch no operand of this kernel; they only have to be complete before the
// next launch reads the caches, and their short index chains run under the weight stream instead of in a launch
// of their own.
struct StoreRider {
  DecodeStepOp op;
  int64_t n_items;
  uint32_t segs_per_row, row_bytes, items_per_y, blocks;
};

template <bool BF16, int KS, bool STORES>
__device__ __forceinline__ void query_image_body(const QImageArgs& g, const StoreRider* rider) {
  const int aux_rows = (int)gridDim.y - g.heads;
  if ((int)blockIdx.y < aux_rows) {
    const uint32_t id = blockIdx.y * gridDim.x + blockIdx.x;
    if (id == 0) {
      plan_ragged_batch(g.row_start, g.n_seqs, g.tile_tokens, g.tile_start, g.order, g.zero_row, g.zero_vecs);
    } else if constexpr (STORES) {
      if (id - 1 < rider->blocks)
        row_mover_body<16, DecodeStepOp::kChunks, DecodeStepOp>(rider->op, rider->n_items, rider->segs_per_row,
                                                                rider->row_bytes, rider->items_per_y, id - 1, 0);
    }
    return;
  }
  constexpr int D = KS * 32;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int h = (int)blockIdx.y - aux_rows;
  const int64_t col0 = (int64_t)blockIdx.x * 512 + wave * 128 + 8 * c;
  const bool col_ok = col0 < g.hidden;
  const char* b_col = g.w + (col_ok ? col0 : 0) * 2 + (int64_t)h * D * g.w_stride_b;
  u32x4 tcol[KS][8];
  {
    u32x4 r[KS][8];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        r[ks][i] = __builtin_nontemporal_load((const u32x4*)(b_col + (int64_t)(32 * ks + 8 * g4 + i) * g.w_stride_b));
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
        for (int p = 0; p < 4; ++p)
          tcol[ks][j][p] = __builtin_amdgcn_perm(r[ks][2 * p + 1][j >> 1], r[ks][2 * p][j >> 1], sel);
      }
  }
  // A operand of a tile of 16 sequences: lane (g4, c) = sequence m0 + c, d = 32 ks + 8 g4 .. + 7
  auto load_a = [&](int m0, u32x4(&pf)[KS], bool& ok) {
    const int m = m0 + c;
    int64_t row = 0;
    ok = m < g.n_seqs;
    if (ok) {
      row = g.seq_rows[m];
      ok = row >= 0 && row < g.num_q_rows;
    }
    const char* a = g.q + (ok ? row : 0) * g.q_stride_b + ((int64_t)h * D + 8 * g4) * 2;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) pf[ks] = *(const u32x4*)(a + ks * 64);
  };
  u32x4 pf[2][KS];
  bool ok[2];
  load_a(0, pf[0], ok[0]);
  for (int m0 = 0; m0 < g.n_seqs; m0 += 32) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int mm = m0 + 16 * u;
      if (mm < g.n_seqs) {
        if (mm + 16 < g.n_seqs) load_a(mm + 16, pf[u ^ 1], ok[u ^ 1]);
        float4v acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const u32x4 a = ok[u] ? pf[u][ks] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j] = mfma16<BF16>(a, tcol[ks][j], acc[j]);
        }
        if (col_ok) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int m = mm + 4 * g4 + i;
            if (m >= g.n_seqs) continue;
            uint16_t hh[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float v = acc[j][i] * g.alpha;
              hh[j] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits_rounded(v);
            }
            u32x4 o;
#pragma unroll
            for (int p = 0; p < 4; ++p) o[p] = (uint32_t)hh[2 * p] | ((uint32_t)hh[2 * p + 1] << 16);
            *(u32x4*)(g.qt + (((int64_t)m * g.heads + h) * g.hidden + col0) * 2) = o;
          }
        }
      }
    }
  }
}

template <bool BF16, int KS>
__global__ __launch_bounds__(256) void query_image_kernel(const QImageArgs g) {
  query_image_body<BF16, KS, false>(g, nullptr);
}
static_assert(kMaxThreads == 256, "the row mover's workgroups have the size of this kernel's");
template <bool BF16, int KS>
__global__ __launch_bounds__(256) void query_image_and_stores_kernel(const QImageArgs g, const StoreRider rider) {
  query_image_body<BF16, KS, true>(g, &rider);
}

template <bool BF16, int NHT>
__global__ __launch_bounds__(kScThreads) void hidden_scores_kernel(const ScoreArgs g) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];  // [2][NHT*16 heads][1 KiB]
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  // Work items are the tiles in the list of all sequences' tiles; workgroups past the end of the list leave.  (A (tile, sequence) grid would hold mostly absent tiles of short sequences, and since workgroups
  // are dealt to the 8 XCDs round-robin by linear index, the tiles that exist would crowd onto a few XCDs.)
  // Workgroups are dealt to the 8 XCDs round-robin by linear index: XCD x takes the x-th eighth of the list, so
  // that the tiles of a sequence (neighbours in the list) read its query image through one L2 (measured: 0.96
  // instead of 1.17 GB fetched for 0.95 GB of algorithmic reads; the kernel's time does not change).
  const int total = g.tile_start[g.n_seqs];
  const int per_xcd = (total + 7) >> 3;
  const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per_xcd || tile >= total) return;
  int zlo = 0, zhi = g.n_seqs - 1;
  while (zlo < zhi) {  // last z with tile_start[z] <= tile
    const int mid = (zlo + zhi + 1) >> 1;
    if (g.tile_start[mid] <= tile) zlo = mid; else zhi = mid - 1;
  }
  const int z = zlo;
  const int64_t rs = g.row_start[z];
  const int L = (int)(g.row_start[z + 1] - rs);
  const int tile0 = (tile - g.tile_start[zlo]) * kScTokens;

  // rows of this lane's two tokens in the loading layout (past the sequence / padding slots: slot 0, never used)
  auto token_row = [&](int t) {
    int64_t slot = 0;
    if (t < L) {
      slot = g.row_ids[rs + t];
      if (slot < 0 || slot >= g.num_slots) slot = 0;
    }
    return g.cache + slot * g.slot_stride_b + (lane & 7) * 16;
  };
  const char* rowp0 = token_row(tile0 + wave * 16 + (lane >> 3));
  const char* rowp1 = token_row(tile0 + wave * 16 + 8 + (lane >> 3));
  // few tiles (small batches): K is split over blockIdx.y so that the chip still has workgroups; the softmax
  // adds the partial scores
  const int64_t k0 = (int64_t)blockIdx.y * g.k_per_part;
  const int64_t klen = min(g.k - k0, g.k_per_part);
  float4v acc[NHT];
  stream_rows_times_image<BF16, NHT>(rowp0 + k0 * 2, rowp1 + k0 * 2, g.qt + (int64_t)z * g.qt_batch_stride_b + k0 * 2,
                                     g.qt_row_stride_b, g.heads, klen, lds, acc);

  // lane (g4, c) holds heads 16*ht + 4*g4 + i and token c of its wavefront
  const int t = tile0 + wave * 16 + c;
  if (t >= g.s_row_stride) return;
  float* s_base = g.s + (int64_t)blockIdx.y * g.s_part_stride + (int64_t)z * g.s_batch_stride + t;
#pragma unroll
  for (int ht = 0; ht < NHT; ++ht)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int head = 16 * ht + 4 * g4 + i;
      if (head < g.heads) s_base[(int64_t)head * g.s_row_stride] = acc[ht][i];
    }
}

// S[0] += S[1] + ... + S[parts-1]: the partial scores of a K-split scores pass (few tiles: small batches) made
// whole before the softmax reads them, 4 scores per thread, every part's load independent of the others, added in
// part order.
__global__ __launch_bounds__(256) void score_parts_sum_kernel(float* __restrict__ s, int64_t n, int parts,
                                                              int64_t part_stride) {
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (idx >= n) return;
  float4v acc = *(const float4v*)(s + idx);
  int p = 1;
  for (; p + 3 < parts; p += 4) {
    const float4v v0 = *(const float4v*)(s + p * part_stride + idx);
    const float4v v1 = *(const float4v*)(s + (p + 1) * part_stride + idx);
    const float4v v2 = *(const float4v*)(s + (p + 2) * part_stride + idx);
    const float4v v3 = *(const float4v*)(s + (p + 3) * part_stride + idx);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = (((acc[i] + v0[i]) + v1[i]) + v2[i]) + v3[i];
  }
  for (; p < parts; ++p) {
    const float4v v = *(const float4v*)(s + p * part_stride + idx);
    acc[0] += v[0]; acc[1] += v[1]; acc[2] += v[2]; acc[3] += v[3];
  }
  *(float4v*)(s + idx) = acc;
}

// ------------------------------------------------------------------ per-head projection of many rows
// out[map(m)][h*head_rows + d] = <W[h*head_rows + d], x[m][h]> + bias, for m < m_rows: the per-head value
// projection of the context rows of many sequences.  The same streaming core as the scores: the streamed rows
// are the head's weight rows (128 per workgroup), the image is x[m0 .. m0+16*NHT)[h] (16*NHT sequences), so the
// weights are read once per 16*NHT sequences and x once per 128 weight rows.
struct HeadProjArgs {
  const char* w; int64_t w_stride_b; int head_rows, heads;
  const char* x; int64_t x_row_stride_b, x_head_stride_b; int m_rows;
  const char* bias;                                   // nullable, 16-bit
  char* out; int64_t out_stride; const int64_t* out_row_map; int64_t out_rows;  // elements; map nullable
  int64_t k;
  int m_tiles, row_tiles;                             // per head
};

template <bool BF16, int NHT>
__global__ __launch_bounds__(kScThreads) void head_proj_kernel(const HeadProjArgs g) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  // blockIdx.x = (m tile, head, row tile), row tile fastest: neighbours share the image through L2
  const int row_tile = blockIdx.x % g.row_tiles;
  const int h = (blockIdx.x / g.row_tiles) % g.heads;
  const int m0 = (blockIdx.x / g.row_tiles / g.heads) * (16 * NHT);
  const int tile0 = row_tile * kScTokens;
  auto weight_row = [&](int d) {  // rows past the head: its first row, never used
    const int64_t row = (int64_t)h * g.head_rows + (d < g.head_rows ? d : 0);
    return g.w + row * g.w_stride_b + (lane & 7) * 16;
  };
  float4v acc[NHT];
  stream_rows_times_image<BF16, NHT>(weight_row(tile0 + wave * 16 + (lane >> 3)),
                                     weight_row(tile0 + wave * 16 + 8 + (lane >> 3)),
                                     g.x + (int64_t)m0 * g.x_row_stride_b + (int64_t)h * g.x_head_stride_b,
                                     g.x_row_stride_b, min(16 * NHT, g.m_rows - m0), g.k, lds, acc);
  // lane (g4, c) holds x rows m0 + 16*ht + 4*g4 + i and weight row tile0 + 16*wave + c of the head
  const int d = tile0 + wave * 16 + c;
  if (d >= g.head_rows) return;
  const int64_t col = (int64_t)h * g.head_rows + d;
  const float b = g.bias ? load_16bit_as_f32<BF16>(g.bias, col) : 0.f;
#pragma unroll
  for (int ht = 0; ht < NHT; ++ht)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 16 * ht + 4 * g4 + i;
      if (m >= g.m_rows) continue;
      const int64_t r = g.out_row_map ? g.out_row_map[m] : m;
      if (r < 0 || r >= g.out_rows) continue;
      const float v = acc[ht][i] + b;
      *(uint16_t*)(g.out + (r * g.out_stride + col) * 2) = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
    }
}

// ------------------------------------------------------------------ softmax and weighted sum of paged rows
// ctx[z][h][:] = sum_t softmax_t(S[z][h][:])[t] * hidden row t of sequence z, in one pass over the rows.
//
// A workgroup of kWsWaves wavefronts owns one sequence (or one partition of its tokens) and kWsWaves * 128
// columns; a wavefront owns 128 columns and walks the rows 32 tokens at a time: a lane loads an 8x8 block (8
// rows, 16 bytes = 8 columns each; 16 lanes read 256 contiguous bytes of a row), transposes it in registers with
// v_perm_b32 and feeds 8 MFMAs per 16 heads.  The softmax is an online one, 96 tokens (a chunk = 3 steps) at a
// time: the threads of the workgroup read the fp32 scores of the next chunk of all heads once, keep a running
// maximum and sum per head, and leave p = exp2(s - max) as
// 16-bit values in LDS, where every wavefront fetches its MFMA operand — the scores are read once per workgroup
// instead of the probabilities once per 128 columns (those redundant reads were a quarter of the traffic of the
// kernel this replaces), and no softmax pass or probability buffer exists.  When a chunk moves a head's maximum
// the accumulators of that head are rescaled.
// The loop body is straight-line code: three steps, the three slots of the register ring at fixed positions, every
// load unconditional (a row, column or token that does not exist reads a valid address and is replaced by zeros),
// so that the compiler's wait counts before the MFMAs are exact and two steps (16 KiB per wavefront) stay in
// flight while one is multiplied; with loads under branches it waited for all but the newest step.
// Partitions (kparts > 1: few sequences, or sequences beyond kWsMaxPart tokens) leave unnormalised fp32 sums and
// their (max, sum) pairs for wsum_combine_kernel.
#ifndef APS_WS_WAVES
#define APS_WS_WAVES 8
#endif
#ifndef APS_WS_RING
#define APS_WS_RING 3
#endif
#ifndef APS_WS_OCC
#define APS_WS_OCC 2
#endif
constexpr int kWsWaves = APS_WS_WAVES, kWsThreads = kWsWaves * 64, kWsRing = APS_WS_RING, kWsChunk = 32 * kWsRing;
constexpr int kHeadwiseMaxSeqs = 256;             // sequences up to which the value projection may take the weight streams
constexpr int kFusedHeadSize = 128;               // head size of the paged attention that can ride in the chunk launch
constexpr int kWsMaxPart = 4096;                  // tokens of a partition (their slots are staged in LDS)
constexpr int kWsIds = (kWsMaxPart + kWsChunk - 1) / kWsChunk * kWsChunk + 32 * (kWsRing - 1);
constexpr int kWsPStride = kWsChunk * 2 + 16;     // bytes between heads of a probability chunk (13 x 16: odd)
constexpr int kWsHeadsPerPass = kWsThreads / 32;  // heads whose chunk scores the workgroup reads at a time

// max over the 32 lanes of a half wave, in every lane: butterflies inside a row of 16 lanes are DPP moves
// (quad permutes, then the mirrors of 8 and 16 lanes: a maximum does not care which partner a lane meets), the
// last exchange between the two rows one ds_bpermute.
__device__ __forceinline__ float half_wave_max(float x) {
  int v = __float_as_int(x);
#define APS_DPP_MAX(ctrl)                                                                                     \
  v = __float_as_int(fmaxf(__int_as_float(v), __int_as_float(__builtin_amdgcn_update_dpp(v, v, ctrl, 0xf, 0xf, false))))
  APS_DPP_MAX(0xb1);   // quad_perm [1,0,3,2]
  APS_DPP_MAX(0x4e);   // quad_perm [2,3,0,1]
  APS_DPP_MAX(0x141);  // row_half_mirror
  APS_DPP_MAX(0x140);  // row_mirror
#undef APS_DPP_MAX
  const float y = __int_as_float(v);
  return fmaxf(y, __shfl_xor(y, 16));
}

struct WsumArgs {
  const float* s; int64_t s_batch_stride, s_row_stride;  // S[z][h][t], complete scores
  const char* cache; int64_t slot_stride_b, num_slots;
  const int64_t* row_ids; const int64_t* row_start;
  const char* zero_row;                                   // n zeros (what a token without a cached row reads)
  int heads, m_tiles, n_seqs, k_per_part;
  int64_t n;
  char* out; int64_t out_batch_stride, out_row_stride;   // elements: ctx[z][h][n]
  float* partial; float* partial_ml;                      // kparts > 1: [part][z][h][n] and [part][z][h][2]
  const int32_t* order;                                   // nullable: the y-th sequence dispatched (longest first)
};

template <bool BF16, int MT>
__global__ __launch_bounds__(kWsThreads) __attribute__((amdgpu_waves_per_eu(APS_WS_OCC, APS_WS_OCC))) void hidden_wsum_kernel(
    const WsumArgs g) {
  constexpr int NJ = 16 * MT / kWsHeadsPerPass;   // score quads per thread and chunk
  static_assert(16 * MT % kWsHeadsPerPass == 0, "heads are spread evenly over the passes");
  __shared__ __attribute__((aligned(16))) int32_t ids[kWsIds];
  __shared__ __attribute__((aligned(16))) char p_lds[2][16 * MT * kWsPStride];
  __shared__ __attribute__((aligned(16))) float scale_s[2][16 * MT];
  __shared__ __attribute__((aligned(16))) float fin_s[2][16 * MT];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int zi = blockIdx.y / g.m_tiles;
  const int z = g.order ? g.order[zi] : zi;
  const int m0 = (blockIdx.y % g.m_tiles) * (16 * MT);
  const int64_t rs = g.row_start[z];
  const int K = (int)min(g.row_start[z + 1] - rs, g.s_row_stride);  // a sequence beyond the stated maximum: its head
  const int kbeg = blockIdx.z * g.k_per_part;
  const int kend = min(K, kbeg + g.k_per_part);
  const int n_tok = max(kend - kbeg, 0);
  const int nchunks = (n_tok + kWsChunk - 1) / kWsChunk;
  {  // slots of the partition, -1 for everything a step may touch past its end
    const int staged = nchunks * kWsChunk + 32 * (kWsRing - 1);
    for (int i = tid; i < staged; i += kWsThreads) {
      int64_t slot = -1;
      if (i < n_tok) slot = g.row_ids[rs + kbeg + i];
      ids[i] = (slot >= 0 && slot < g.num_slots) ? (int32_t)slot : -1;
    }
  }
  const int64_t col0 = (int64_t)blockIdx.x * (kWsWaves * 128) + wave * 128 + 8 * c;
  const bool col_ok = col0 < g.n;
  const char* b_col = g.cache + (col_ok ? col0 : 0) * 2;
  const char* z_col = g.zero_row + (col_ok ? col0 : 0) * 2;

  // ---- softmax side: thread (hl, tq) owns the token quads tq + 32 qq of a chunk for the heads hl + HP * j
  constexpr int QJ = (kWsChunk / 4 + 31) / 32;
  const int hl = tid >> 5, tq = tid & 31;
  const float kNegInf = -INFINITY;
  // running maximum and sum of every (thread, head) live in LDS between chunks: the streaming steps need the
  // registers (a spilled value costs a scratch load, whose wait drains the ring of row loads)
  __shared__ float ml_s[2][NJ][kWsThreads];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    ml_s[0][j][tid] = kNegInf;
    ml_s[1][j][tid] = 0.f;
  }
  // the scores of one sequence span less than 4 GiB: a uniform base and 32-bit offsets
  const char* s_base = (const char*)(g.s + (int64_t)z * g.s_batch_stride);
  auto s_off = [&](int j, int ts) {
    const int head = m0 + hl + kWsHeadsPerPass * j;
    return (uint32_t)(((int64_t)(head < g.heads ? head : 0) * g.s_row_stride + ts) * 4);
  };
  // first token of quad qq of this thread in `chunk`, and where to read it: a quad past the chunk or the
  // partition reads the row's first quad (valid memory, never used)
  auto quad_t = [&](int chunk, int qq) { return kbeg + chunk * kWsChunk + 4 * (tq + 32 * qq); };
  auto quad_ok = [&](int qq) { return tq + 32 * qq < kWsChunk / 4; };
  auto fetch_s = [&](int chunk, float4v(&sv)[NJ][QJ]) {
#pragma unroll
    for (int qq = 0; qq < QJ; ++qq) {
      const int t = quad_t(chunk, qq);
      const int ts = (quad_ok(qq) && t < kend) ? t : 0;
#pragma unroll
      for (int j = 0; j < NJ; ++j) sv[j][qq] = *(const float4v*)(s_base + s_off(j, ts));
    }
  };
  auto store_p = [&](int chunk, int buf, float4v(&sv)[NJ][QJ], int j) {
    {
      const bool head_ok = m0 + hl + kWsHeadsPerPass * j < g.heads;
      bool ok[QJ][4];
      float cmax = kNegInf;
#pragma unroll
      for (int qq = 0; qq < QJ; ++qq) {
        const int t = quad_t(chunk, qq);
        const int ts = (quad_ok(qq) && t < kend) ? t : 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          ok[qq][i] = head_ok && quad_ok(qq) && t + i < kend;
          cmax = fmaxf(cmax, ok[qq][i] ? sv[j][qq][i] : kNegInf);
        }
      }
      cmax = half_wave_max(cmax);  // the 32 lanes of a head
      const float m_old = ml_s[0][j][tid];
      const float m_new = fmaxf(m_old, cmax);
      const float scale = m_new == kNegInf ? 1.f : __builtin_amdgcn_exp2f(m_old - m_new);
      float sum = 0.f;
#pragma unroll
      for (int qq = 0; qq < QJ; ++qq) {
        uint16_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // v_exp_f32: arguments are <= 0 here and results below 2^-126 may flush to zero
          const float e = ok[qq][i] ? __builtin_amdgcn_exp2f(sv[j][qq][i] - m_new) : 0.f;
          sum += e;
          o[i] = BF16 ? f32_to_bf16_bits(e) : f32_to_f16_bits(e);
        }
        // no branch in this loop body (the wait counts of the row loads stay exact): a quad past the chunk goes
        // to the spare slot behind the head's row, and all 32 lanes of a head store its (identical) scale
        const int q_dst = quad_ok(qq) ? tq + 32 * qq : kWsChunk / 4;
        *(uint2*)(p_lds[buf] + (hl + kWsHeadsPerPass * j) * kWsPStride + q_dst * 8) =
            uint2{(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
      }
      ml_s[1][j][tid] = ml_s[1][j][tid] * scale + sum;
      ml_s[0][j][tid] = m_new;
      scale_s[buf][hl + kWsHeadsPerPass * j] = scale;
    }
  };

  // ---- streaming side
  float4v acc[MT][8];
#pragma unroll
  for (int ht = 0; ht < MT; ++ht)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[ht][j] = float4v{0.f, 0.f, 0.f, 0.f};
  // rows of the step that starts at token kbeg + i0: unconditional loads; a slot of -1 (a token past the
  // partition, a padding slot) reads the row of zeros the caller keeps for that purpose, a column past the row
  // reads column 0 (its sums are never stored)
  auto load_step = [&](int i0, u32x4(&r)[8]) {
    const u32x4* src = (const u32x4*)(ids + i0 + 8 * g4);  // 8 slots = 32 bytes, 32-byte aligned
    const u32x4 q0 = src[0], q1 = src[1];
    const int32_t slot[8] = {(int32_t)q0[0], (int32_t)q0[1], (int32_t)q0[2], (int32_t)q0[3],
                             (int32_t)q1[0], (int32_t)q1[1], (int32_t)q1[2], (int32_t)q1[3]};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const char* src_row = slot[i] >= 0 ? b_col + (int64_t)slot[i] * g.slot_stride_b : z_col;
      r[i] = __builtin_nontemporal_load((const u32x4*)src_row);
    }
  };
#ifndef APS_WS_ABL
#define APS_WS_ABL 0
#endif
  auto mac_step = [&](u32x4(&r)[8], const char* prow) {
    if constexpr ((APS_WS_ABL & 1) != 0) {  // timing experiment: consume the loads, no products
      uint32_t x = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) x ^= r[i][0] ^ r[i][1] ^ r[i][2] ^ r[i][3];
      acc[0][0][0] += __uint_as_float(x & 0xffu);
      return;
    }
    u32x4 pf[MT];
#pragma unroll
    for (int ht = 0; ht < MT; ++ht) pf[ht] = *(const u32x4*)(prow + ht * 16 * kWsPStride);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      u32x4 tcol;  // column j of the 8x8 block: dword p = (row 2p, row 2p+1)
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int p = 0; p < 4; ++p) tcol[p] = __builtin_amdgcn_perm(r[2 * p + 1][j >> 1], r[2 * p][j >> 1], sel);
#pragma unroll
      for (int ht = 0; ht < MT; ++ht) acc[ht][j] = mfma16<BF16>(pf[ht], tcol, acc[ht][j]);
    }
  };

  float4v sv[NJ][QJ];
  // The loop has no prologue: it starts one chunk early on a ring of zeros and a buffer of zero probabilities
  // (and prepares chunk 0 on that trip), so that the loads in flight at its head are the same on entry and on
  // every later trip.
  for (int i = tid; i < 16 * MT * kWsPStride / 16; i += kWsThreads)
    ((u32x4*)p_lds[1])[i] = u32x4{0u, 0u, 0u, 0u};
  if (tid < 16 * MT) scale_s[1][tid] = 1.f;
  u32x4 r[kWsRing][8];
#pragma unroll
  for (int d = 0; d < kWsRing; ++d)
#pragma unroll
    for (int i = 0; i < 8; ++i) r[d][i] = u32x4{0u, 0u, 0u, 0u};
  __syncthreads();  // slots, running maxima and the zero buffer are in LDS
  // (peeling the last chunk off without its requests was measured: the second copy of the body costs more in
  // spilled registers than the padded requests do)
  for (int chunk = -1; chunk < nchunks; ++chunk) {
    const int buf = chunk & 1;
    {  // heads whose maximum moved with this chunk: bring their sums to the new maximum
      float4v sc[MT];
      bool moved = false;
#pragma unroll
      for (int ht = 0; ht < MT; ++ht) {
        sc[ht] = *(const float4v*)(&scale_s[buf][16 * ht + 4 * g4]);
        moved = moved || sc[ht][0] != 1.f || sc[ht][1] != 1.f || sc[ht][2] != 1.f || sc[ht][3] != 1.f;
      }
      if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
        for (int ht = 0; ht < MT; ++ht)
#pragma unroll
          for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[ht][j][i] *= sc[ht][i];
      }
    }
#pragma unroll
    for (int st = 0; st < kWsRing; ++st) {
      // rows of the step kWsRing - 1 ahead (before token 0 in the first trip: the padded tail of the slot list)
      const int i0 = chunk * kWsChunk + 32 * (st + kWsRing - 1);
      load_step(i0 >= 0 ? i0 : nchunks * kWsChunk, r[(st + kWsRing - 1) % kWsRing]);
      // scores of the next chunk: behind the first rows of this one, so that they are old loads by the time they
      // are used (loads return in order: waiting for a recent one would drain the ring of rows)
      if ((APS_WS_ABL & 2) == 0 && st == 0) fetch_s(chunk + 1, sv);
      mac_step(r[st], p_lds[buf] + c * kWsPStride + (32 * st + 8 * g4) * 2);
      // the softmax of the next chunk, a group of heads per step, between the products of this one: on its own at
      // the end of the chunk it is a stretch of dependent LDS and transcendental latencies in which nothing streams
      if ((APS_WS_ABL & 2) == 0 && st >= 1) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          if (st == 1 + j * (kWsRing - 1) / NJ) store_p(chunk + 1, buf ^ 1, sv, j);
      }
    }
    APS_WAIT_LGKM0();
    if ((APS_WS_ABL & 4) == 0) APS_BARRIER();  // everyone has left this chunk's buffer, the next one is complete
  }

  // ---- totals of the softmax: (max, sum) per head
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    float l = ml_s[1][j][tid];
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) l += __shfl_xor(l, off);
    if (tq == 0) {
      fin_s[0][hl + kWsHeadsPerPass * j] = ml_s[0][j][tid];
      fin_s[1][hl + kWsHeadsPerPass * j] = l;
    }
  }
  __syncthreads();
  if (g.partial_ml && blockIdx.x == 0 && tid < 16 * MT && m0 + tid < g.heads) {
    float* ml = g.partial_ml + (((int64_t)blockIdx.z * g.n_seqs + z) * g.heads + m0 + tid) * 2;
    ml[0] = fin_s[0][tid];
    ml[1] = fin_s[1][tid];
  }
  // lane (g4, c) holds heads m0 + 16*ht + 4*g4 + i and columns col0 .. col0+7 (MFMA j = column j)
  if (!col_ok) return;
#pragma unroll
  for (int ht = 0; ht < MT; ++ht)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 16 * ht + 4 * g4 + i;
      if (m >= g.heads) continue;
      if (g.partial) {
        float* dst = g.partial + (((int64_t)blockIdx.z * g.n_seqs + z) * g.heads + m) * g.n + col0;
        *(float4v*)dst = float4v{acc[ht][0][i], acc[ht][1][i], acc[ht][2][i], acc[ht][3][i]};
        *(float4v*)(dst + 4) = float4v{acc[ht][4][i], acc[ht][5][i], acc[ht][6][i], acc[ht][7][i]};
      } else {
        const float l = fin_s[1][16 * ht + 4 * g4 + i];
        const float inv = l > 0.f ? 1.f / l : 0.f;
        uint16_t h[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float v = acc[ht][j][i] * inv;
          h[j] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
        }
        u32x4 o;
#pragma unroll
        for (int p = 0; p < 4; ++p) o[p] = (uint32_t)h[2 * p] | ((uint32_t)h[2 * p + 1] << 16);
        *(u32x4*)(g.out + ((int64_t)z * g.out_batch_stride + (int64_t)m * g.out_row_stride + col0) * 2) = o;
      }
    }
}

// ------------------------------------------------------------------ few cached rows: one chunk per workgroup
// The same sum for a batch with few cached rows in all (a serving step's handful of sequences).  There the pass
// above is not a stream but a chain of memory latencies - slots, scores, rows, chunk after chunk, with a handful
// of workgroups - and lasts 17-20 us for 6 MB.  Here a workgroup owns ONE chunk of kWsChunk tokens of one sequence
// (and kWsWaves * 128 columns), requests everything it needs at once - its scores and, behind the slots, all rows
// of the chunk - does the chunk's softmax while the rows are on their way, multiplies, and leaves unnormalised
// sums with the chunk's (max, sum) for wsum_combine_kernel: two memory round trips deep whatever the lengths.
// The price is the fp32 sums of every chunk (heads x hidden values: about as many bytes as the chunk's rows),
// which is why only small batches come here.
template <bool BF16, int MT>
__device__ __forceinline__ void hidden_wsum_chunk_body(const WsumArgs& g) {
  constexpr int NJ = 16 * MT / kWsHeadsPerPass;
  __shared__ __attribute__((aligned(16))) char p_lds[16 * MT * kWsPStride];
  __shared__ __attribute__((aligned(16))) float fin_s[2][16 * MT];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int z = blockIdx.y / g.m_tiles;
  const int m0 = (blockIdx.y % g.m_tiles) * (16 * MT);
  const int64_t rs = g.row_start[z];
  const int K = (int)min(g.row_start[z + 1] - rs, g.s_row_stride);
  const int kbeg = blockIdx.z * kWsChunk;
  const int n_tok = min(K - kbeg, kWsChunk);
  const float kNegInf = -INFINITY;
  if (n_tok <= 0 && g.partial) {  // a chunk past the end of its sequence: the combining kernel skips it
    if (blockIdx.x == 0 && tid < 16 * MT && m0 + tid < g.heads) {
      float* ml = g.partial_ml + (((int64_t)blockIdx.z * g.n_seqs + z) * g.heads + m0 + tid) * 2;
      ml[0] = kNegInf;
      ml[1] = 0.f;
    }
    return;
  }
  // ---- requests: the chunk's scores (thread (hl, tq): heads hl + HP*j, tokens 4*tq .. 4*tq+3) ...
  const int hl = tid >> 5, tq = tid & 31;
  const bool quad_ok = tq < kWsChunk / 4 && 4 * tq < n_tok;
  float4v sv[NJ];
  {
    const char* s_base = (const char*)(g.s + (int64_t)z * g.s_batch_stride);
    const int ts = quad_ok ? kbeg + 4 * tq : 0;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int head = m0 + hl + kWsHeadsPerPass * j;
      sv[j] = *(const float4v*)(s_base + ((int64_t)(head < g.heads ? head : 0) * g.s_row_stride + ts) * 4);
    }
  }
  // ... and the rows: lane (g4, c) reads tokens 32*st + 8*g4 + i, columns col0 .. col0+7 (a token past the chunk's
  // end or without a cached row reads the row of zeros, a column past the row column 0)
  const int64_t col0 = (int64_t)blockIdx.x * (kWsWaves * 128) + wave * 128 + 8 * c;
  const bool col_ok = col0 < g.n;
  const char* b_col = g.cache + (col_ok ? col0 : 0) * 2;
  const char* z_col = g.zero_row + (col_ok ? col0 : 0) * 2;
  int64_t slot[kWsRing][8];
#pragma unroll
  for (int st = 0; st < kWsRing; ++st)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = 32 * st + 8 * g4 + i;
      slot[st][i] = g.row_ids[rs + kbeg + (t < n_tok ? t : 0)];
      if (t >= n_tok) slot[st][i] = -1;
    }
  u32x4 r[kWsRing][8];
#pragma unroll
  for (int st = 0; st < kWsRing; ++st)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const bool ok = slot[st][i] >= 0 && slot[st][i] < g.num_slots;
      r[st][i] = __builtin_nontemporal_load((const u32x4*)(ok ? b_col + slot[st][i] * g.slot_stride_b : z_col));
    }
  // ---- softmax of the chunk, 16-bit probabilities into LDS
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const bool head_ok = m0 + hl + kWsHeadsPerPass * j < g.heads;
    bool ok[4];
    float cmax = kNegInf;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ok[i] = head_ok && quad_ok && 4 * tq + i < n_tok;
      cmax = fmaxf(cmax, ok[i] ? sv[j][i] : kNegInf);
    }
    cmax = half_wave_max(cmax);
    float sum = 0.f;
    uint16_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float e = ok[i] ? __builtin_amdgcn_exp2f(sv[j][i] - cmax) : 0.f;
      sum += e;
      o[i] = BF16 ? f32_to_bf16_bits(e) : f32_to_f16_bits_rounded(e);
    }
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    const int q_dst = tq < kWsChunk / 4 ? tq : kWsChunk / 4;  // lanes past the chunk: the spare slot behind the row
    *(uint2*)(p_lds + (hl + kWsHeadsPerPass * j) * kWsPStride + q_dst * 8) =
        uint2{(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
    if (tq == 0) {
      fin_s[0][hl + kWsHeadsPerPass * j] = cmax;
      fin_s[1][hl + kWsHeadsPerPass * j] = sum;
    }
  }
  __syncthreads();
  // ---- products: heads x tokens (LDS) times tokens x columns (registers, 8x8 blocks transposed)
  float4v acc[MT][8];
#pragma unroll
  for (int ht = 0; ht < MT; ++ht)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[ht][j] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < kWsRing; ++st) {
    const char* prow = p_lds + c * kWsPStride + (32 * st + 8 * g4) * 2;
    u32x4 pf[MT];
#pragma unroll
    for (int ht = 0; ht < MT; ++ht) pf[ht] = *(const u32x4*)(prow + ht * 16 * kWsPStride);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      u32x4 tcol;  // column j of the 8x8 block: dword p = (row 2p, row 2p+1)
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int p = 0; p < 4; ++p) tcol[p] = __builtin_amdgcn_perm(r[st][2 * p + 1][j >> 1], r[st][2 * p][j >> 1], sel);
#pragma unroll
      for (int ht = 0; ht < MT; ++ht) acc[ht][j] = mfma16<BF16>(pf[ht], tcol, acc[ht][j]);
    }
  }
  if (g.partial_ml && blockIdx.x == 0 && tid < 16 * MT && m0 + tid < g.heads) {
    float* ml = g.partial_ml + (((int64_t)blockIdx.z * g.n_seqs + z) * g.heads + m0 + tid) * 2;
    ml[0] = fin_s[0][tid];
    ml[1] = fin_s[1][tid];
  }
  if (!col_ok) return;
#pragma unroll
  for (int ht = 0; ht < MT; ++ht)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 16 * ht + 4 * g4 + i;
      if (m >= g.heads) continue;
      if (g.partial) {
        float* dst = g.partial + (((int64_t)blockIdx.z * g.n_seqs + z) * g.heads + m) * g.n + col0;
        *(float4v*)dst = float4v{acc[ht][0][i], acc[ht][1][i], acc[ht][2][i], acc[ht][3][i]};
        *(float4v*)(dst + 4) = float4v{acc[ht][4][i], acc[ht][5][i], acc[ht][6][i], acc[ht][7][i]};
      } else {  // the sequence's only chunk: the context row itself
        const float l = fin_s[1][16 * ht + 4 * g4 + i];
        const float inv = l > 0.f ? 1.f / l : 0.f;
        uint16_t h[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float v = acc[ht][j][i] * inv;
          h[j] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits_rounded(v);
        }
        u32x4 o;
#pragma unroll
        for (int p = 0; p < 4; ++p) o[p] = (uint32_t)h[2 * p] | ((uint32_t)h[2 * p + 1] << 16);
        *(u32x4*)(g.out + ((int64_t)z * g.out_batch_stride + (int64_t)m * g.out_row_stride + col0) * 2) = o;
      }
    }
}

template <bool BF16, int MT>
__global__ __launch_bounds__(kWsThreads) void hidden_wsum_chunk_kernel(const WsumArgs g) {
  hidden_wsum_chunk_body<BF16, MT>(g);
}

// The same launch with the K/V-cached sequences of the step on board: slices z < ws_z of the grid are the chunks
// above; the workgroups of the slices behind them take the (head group, sequence) items of a paged decode
// attention's group path, one each, in the grid's linear order.  The chunk workgroups are few and wait on memory
// most of their time; the attention's workgroups land on compute units that would have been idle, and the step
// has one launch less on its critical path.  Same code as paged_decode_group_kernel, so the same bits.
template <bool BF16, int MT>
__global__ __launch_bounds__(kWsThreads) void hidden_wsum_chunk_and_paged_kernel(const WsumArgs g, const AttnArgs a,
                                                                                 const int ws_z, const int head_groups,
                                                                                 const int items) {
  if ((int)blockIdx.z < ws_z) {
    hidden_wsum_chunk_body<BF16, MT>(g);
    return;
  }
  const int id = (((int)blockIdx.z - ws_z) * (int)gridDim.y + (int)blockIdx.y) * (int)gridDim.x + (int)blockIdx.x;
  if (id >= items) return;
  paged_decode_group_body<BF16 ? APS_BF16 : APS_F16, BF16 ? KV_BF16 : KV_F16, kFusedHeadSize, 1, APS_DEPTH_F16,
                          kWsWaves>(a, id % head_groups, id / head_groups);
}

// ctx[z][h][n] = sum_p w_p * partial[p][z][h][n] / sum_p w_p * l_p with w_p = 2^(m_p - max_p m_p): the partitions
// of a sequence put on one scale, added in the order of the partitions, 4 columns per thread.
template <bool BF16>
__global__ __launch_bounds__(256) void wsum_combine_kernel(const float* __restrict__ partial,
                                                           const float* __restrict__ ml, char* out, int parts,
                                                           int n_seqs, int heads, int64_t n, int64_t out_batch_stride,
                                                           int64_t out_row_stride) {
  const int64_t per_part = (int64_t)n_seqs * heads * n;
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (idx >= per_part) return;
  const int64_t col = idx % n, zh = idx / n;
  float mx = -INFINITY;
  for (int p = 0; p < parts; ++p) mx = fmaxf(mx, ml[((int64_t)p * n_seqs * heads + zh) * 2]);
  float4v num = {0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  for (int p = 0; p < parts; ++p) {
    const float mp = ml[((int64_t)p * n_seqs * heads + zh) * 2], lp = ml[((int64_t)p * n_seqs * heads + zh) * 2 + 1];
    if (mp == -INFINITY) continue;  // a partition past the end of its sequence
    const float w = exp2f(mp - mx);
    const float4v v = *(const float4v*)(partial + p * per_part + idx);
    num[0] += v[0] * w; num[1] += v[1] * w; num[2] += v[2] * w; num[3] += v[3] * w;
    den += lp * w;
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  const int64_t h = zh % heads, z = zh / heads;
  uint16_t* o = (uint16_t*)out + z * out_batch_stride + h * out_row_stride + col;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = BF16 ? f32_to_bf16_bits(num[i] * inv) : f32_to_f16_bits(num[i] * inv);
}

template <bool BF16>
int launch_nn(const NnArgs& g, hipStream_t s) {
  const int mt = g.m_tiles > 1 ? 3 : (g.m_rows <= 16 ? 1 : (g.m_rows <= 32 ? 2 : 3));  // row tiles are 16*mt rows
  const dim3 grid((unsigned)((g.n + kNnWaves * 128 - 1) / (kNnWaves * 128)), (unsigned)(g.batches * g.m_tiles));
  if (mt == 1)
    APS_LAUNCH((nn_few_rows_kernel<BF16, 1>), grid, dim3(kNnWaves * 64), 0, s, g);
  else if (mt == 2)
    APS_LAUNCH((nn_few_rows_kernel<BF16, 2>), grid, dim3(kNnWaves * 64), 0, s, g);
  else
    APS_LAUNCH((nn_few_rows_kernel<BF16, 3>), grid, dim3(kNnWaves * 64), 0, s, g);
  return launch_status();
}

inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

struct Plan {
  int64_t lp;        // padded row length of S
  int kparts;        // token partitions of the weighted sum
  int score_parts;   // parts of K in the scores kernel (partial scores, made whole by score_parts_sum_kernel)
  int64_t score_k_per_part;
  int k_per_part;
  bool chunked;      // few cached rows: one chunk of tokens per workgroup of the weighted sum
  int64_t off_qt, off_s, off_ctx, off_tiles, off_order, off_zero, off_partial, off_ml, off_vp, total;
  int64_t zero_bytes;      // the row of zeros and, behind it, the arrival counters: cleared by the planning workgroup
  int64_t off_vp_counters;
};

Plan make_plan(int64_t n_seqs, int64_t max_len, int heads, int64_t hidden) {
  Plan p{};
  p.lp = align_up(max_len > 0 ? max_len : 1, 32);
  const int64_t col_tiles = (hidden + kWsWaves * 128 - 1) / (kWsWaves * 128) * ((heads + 47) / 48);
  int64_t parts = 1;
  // Fewer workgroups than CUs (few sequences): split the tokens.  A workgroup walks its tokens one after the
  // other, so without a split the longest sequence sets the kernel's time.  The host knows only the longest
  // length; with lengths spread like a serving batch's the rows in all are about a third of n_seqs * longest,
  // and a part should hold about 1/256 of the work of one column tile.
  // Every partition of every sequence leaves fp32 sums of heads x hidden values for the combining kernel: at
  // least two chunks of tokens per partition keep that traffic below what the rows themselves are.
  if (n_seqs * col_tiles < 256) {
    int64_t target = n_seqs * p.lp * col_tiles / 3 / 256;
    if (target < 2 * kWsChunk) target = 2 * kWsChunk;
    parts = (p.lp + target - 1) / target;
    if (parts > 32) parts = 32;
  }
  while ((p.lp + parts - 1) / parts > kWsMaxPart - kWsChunk) parts *= 2;
  p.k_per_part = (int)align_up((p.lp + parts - 1) / parts, kWsChunk);
  p.kparts = (int)((p.lp + p.k_per_part - 1) / p.k_per_part);
  // few cached rows in all (the host knows only an upper bound of the chunks): a chunk per workgroup
#ifndef APS_WS_CHUNKED_MAX
#define APS_WS_CHUNKED_MAX 32
#endif
  p.chunked = n_seqs * ((p.lp + kWsChunk - 1) / kWsChunk) <= APS_WS_CHUNKED_MAX;
  if (p.chunked) {
    p.k_per_part = kWsChunk;
    p.kparts = (int)((p.lp + kWsChunk - 1) / kWsChunk);
  }
  // scores: with few 128-token tiles, K is split by whole 512-element chunks into as many parts as still give
  // at most one workgroup per CU (one round of long-lived workgroups streams fastest)
  {
    const int64_t tiles = n_seqs * ((p.lp + kScTokens - 1) / kScTokens);
    const int64_t chunks = (hidden + kScChunk - 1) / kScChunk;
    int64_t best_per = chunks;
    for (int64_t per = chunks; per >= 1; --per) {
      const int64_t parts = (chunks + per - 1) / per;
      if (tiles * parts > 256) break;
      if ((chunks - (parts - 1) * per) * 2 < per) continue;  // no stub of a last part
      best_per = per;
    }
    p.score_parts = (int)((chunks + best_per - 1) / best_per);
    p.score_k_per_part = best_per * kScChunk;
  }
  int64_t o = 0;
  p.off_qt = o; o += align_up(n_seqs * heads * hidden * 2, 256);
  p.off_s = o; o += align_up(n_seqs * heads * p.lp * 4, 256) * p.score_parts;
  p.off_ctx = o; o += align_up(n_seqs * heads * hidden * 2, 256);
  p.off_tiles = o; o += align_up((n_seqs + 1) * 4, 256);
  p.off_order = o; o += align_up(n_seqs * 4, 256);
  p.off_zero = o; o += align_up(hidden * 2, 256);
  p.off_vp_counters = o; o += APS_LINEAR_TILE_COUNTERS * 4;
  p.zero_bytes = o - p.off_zero;
  p.off_partial = o;
  if (p.kparts > 1) o += align_up((int64_t)p.kparts * n_seqs * heads * hidden * 4, 256);
  p.off_ml = o;
  if (p.kparts > 1) o += align_up((int64_t)p.kparts * n_seqs * heads * 2 * 4, 256);
  p.off_vp = o;   // fp32 partial products of the value projection's K split (few sequences)
  if (n_seqs <= kHeadwiseMaxSeqs)
    o += align_up(aps_internal_headwise_workspace_bytes(n_seqs, hidden, hidden, (int)(hidden / heads)), 256);
  p.total = o;
  return p;
}

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

int64_t aps_absorbed_attention_workspace_bytes(int64_t n_seqs, int64_t max_len, int num_heads, int head_size) {
  if (n_seqs <= 0 || max_len <= 0 || num_heads <= 0 || head_size <= 0) return 0;
  return make_plan(n_seqs, max_len, num_heads, (int64_t)num_heads * head_size).total;
}

// kv_job (nullable): the paged decode attention of the step's K/V-cached sequences, launched here as well
static int hybrid_attention_impl(const StoreJob* store_job, const PagedJob* kv_job, const void* q, int64_t q_stride, const int64_t* seq_rows,
                                 int64_t num_q_rows, const void* paged_cache, int64_t slot_stride, int64_t num_slots,
                                 const int64_t* hidden_slots, const int64_t* seq_start, int64_t n_seqs,
                                 int64_t max_len, const void* w_k, const void* w_v, const void* b_v, int64_t w_stride,
                                 int num_heads, int head_size, float softmax_scale, void* out, int64_t out_stride,
                                 int64_t out_rows, int dtype, void* workspace, int64_t workspace_bytes,
                                 aps_stream_t stream) {
  if (n_seqs < 0 || max_len < 0 || num_heads <= 0 || head_size <= 0) return APS_ERR_INVALID_ARG;
  if (kv_job && (kv_job->magic != kPagedJobMagic || kv_job->batch < 0)) return APS_ERR_INVALID_ARG;
  if (kv_job && kv_job->batch == 0) kv_job = nullptr;
  if (store_job && (store_job->magic != kStoreJobMagic || store_job->n_items < 0)) return APS_ERR_INVALID_ARG;
  if (store_job && store_job->n_items == 0) store_job = nullptr;
  if (n_seqs == 0) {
    const int st = store_job ? aps_cache_job_launch(store_job, stream) : APS_OK;
    return st != APS_OK || !kv_job ? st : aps_attention_job_launch(kv_job, stream);
  }
  if (!q || !seq_rows || !paged_cache || !hidden_slots || !seq_start || !w_k || !w_v || !out || !workspace)
    return APS_ERR_INVALID_ARG;
  if (dtype != APS_F16 && dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  const int64_t hidden = (int64_t)num_heads * head_size;
  if (head_size % 32 != 0 || hidden % 64 != 0 || num_heads > 96) return APS_ERR_UNSUPPORTED;
  if (q_stride < hidden || slot_stride < hidden || w_stride < hidden || out_stride < hidden) return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(q), addr(paged_cache), addr(w_k), addr(w_v), addr(out), addr(workspace),
                        (uint64_t)q_stride * 2, (uint64_t)slot_stride * 2, (uint64_t)w_stride * 2,
                        (uint64_t)out_stride * 2}) != 16)
    return APS_ERR_UNSUPPORTED;
  if (n_seqs > 65535 / ((num_heads + 47) / 48) || max_len > ((int64_t)1 << 24) || num_slots > 0x7fffffff)
    return APS_ERR_UNSUPPORTED;
  const Plan p = make_plan(n_seqs, max_len, num_heads, hidden);
  if (workspace_bytes < p.total) return APS_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const bool bf16 = dtype == APS_BF16;
  // The job's workgroups can ride in the launch of the chunked weighted sum when that launch runs the kernel the
  // job would have run: group path without a ranking launch of its own, 16-bit cache of the queries' dtype,
  // one head per wavefront at the head size the combined kernel is built for.
  const bool ride = kv_job && p.chunked && kWsWaves == kMaxGroupWaves && APS_HPW_F16 == 1 && kv_job->plan.group &&
                    !kv_job->plan.order_scratch && kv_job->head_size == kFusedHeadSize &&
                    kv_job->kv_dtype == kv_job->q_dtype && kv_job->q_dtype == dtype;
  // The stores can ride beside the absorbed queries when that launch is the kernel with the auxiliary rows and
  // the job is the one-row grid of 16-byte accesses.
  MoverGrid mg{};
  bool stores_ride = false;
  if (store_job && head_size <= 128 && store_job->vb == 16) {
    mg = mover_grid(store_job->n_items, store_job->row_bytes, 16, DecodeStepOp::kChunks);
    stores_ride = mg.grid_y == 1 && mg.grid_x <= 4096;
  }
  if (store_job && !stores_ride) {
    const int st = aps_cache_job_launch(store_job, stream);
    if (st != APS_OK) return st;
  }
  char* ws = (char*)workspace;
  char* qt = ws + p.off_qt;
  float* sc = (float*)(ws + p.off_s);
  const int64_t s_part_stride = align_up(n_seqs * num_heads * p.lp * 4, 256) / 4;  // elements between K parts
  char* ctx = ws + p.off_ctx;
  float* partial = (float*)(ws + p.off_partial);

  int32_t* tiles = (int32_t*)(ws + p.off_tiles);
  int32_t* order = n_seqs > 1 && n_seqs <= kMaxOrderedSeqs ? (int32_t*)(ws + p.off_order) : nullptr;
  // 1. qt[s][h][:] = scale*log2(e) * W_k[h]^T q[seq_rows[s]][h], and the plan of the ragged batch (tile list of
  //    the scores kernel, longest-first order of the weighted sum) in the same launch
  if (head_size <= 128) {
    QImageArgs g{};
    g.q = (const char*)q; g.q_stride_b = q_stride * 2; g.seq_rows = seq_rows; g.num_q_rows = num_q_rows;
    g.n_seqs = (int)n_seqs;
    g.w = (const char*)w_k; g.w_stride_b = w_stride * 2;
    g.heads = num_heads; g.hidden = hidden;
    g.qt = qt;
    g.alpha = softmax_scale * 1.4426950408889634f;
    g.row_start = seq_start; g.tile_tokens = kScTokens; g.tile_start = tiles; g.order = order;
    g.zero_row = (u32x4*)(ws + p.off_zero); g.zero_vecs = (int)(p.zero_bytes / 16);
    const unsigned gx = (unsigned)((hidden + 511) / 512);
    // rows in front of the heads: the plan's workgroup and, with the stores on board, the row mover's
    const unsigned aux = stores_ride ? (unsigned)((1 + mg.grid_x + gx - 1) / gx) : 1u;
    const dim3 grid(gx, (unsigned)num_heads + aux);
#define APS_LAUNCH_QI(B)                                                                     \
  switch (head_size / 32) {                                                                  \
    case 1: APS_LAUNCH((query_image_kernel<B, 1>), grid, dim3(256), 0, s, g); break;         \
    case 2: APS_LAUNCH((query_image_kernel<B, 2>), grid, dim3(256), 0, s, g); break;         \
    case 3: APS_LAUNCH((query_image_kernel<B, 3>), grid, dim3(256), 0, s, g); break;         \
    default: APS_LAUNCH((query_image_kernel<B, 4>), grid, dim3(256), 0, s, g); break;        \
  }
#define APS_LAUNCH_QI_STORES(B)                                                                              \
  switch (head_size / 32) {                                                                                  \
    case 1: APS_LAUNCH((query_image_and_stores_kernel<B, 1>), grid, dim3(256), 0, s, g, rider); break;       \
    case 2: APS_LAUNCH((query_image_and_stores_kernel<B, 2>), grid, dim3(256), 0, s, g, rider); break;       \
    case 3: APS_LAUNCH((query_image_and_stores_kernel<B, 3>), grid, dim3(256), 0, s, g, rider); break;       \
    default: APS_LAUNCH((query_image_and_stores_kernel<B, 4>), grid, dim3(256), 0, s, g, rider); break;      \
  }
    if (stores_ride) {
      const StoreRider rider{store_job->op, store_job->n_items, (uint32_t)mg.segs_per_row,
                             (uint32_t)store_job->row_bytes, (uint32_t)mg.items_per_y, (uint32_t)mg.grid_x};
      if (bf16) { APS_LAUNCH_QI_STORES(true) } else { APS_LAUNCH_QI_STORES(false) }
    } else if (bf16) { APS_LAUNCH_QI(true) } else { APS_LAUNCH_QI(false) }
#undef APS_LAUNCH_QI_STORES
#undef APS_LAUNCH_QI
    const int st = launch_status();
    if (st != APS_OK) return st;
  } else {  // heads wider than 128: the generic few-row product (batch = head, K = head_size, B = rows of W_k)
    NnArgs g{};
    g.a = (const char*)q; g.a_batch_stride_b = (int64_t)head_size * 2; g.lda_b = q_stride * 2;
    g.m_rows = (int)n_seqs; g.a_row_ids = seq_rows; g.num_a_rows = num_q_rows;
    g.b = (const char*)w_k; g.b_row_stride_b = w_stride * 2; g.num_b_rows = hidden;
    g.k_fixed = head_size;
    g.n = hidden;
    g.out = qt; g.out_batch_stride = hidden; g.out_row_stride = (int64_t)num_heads * hidden;
    g.batches = num_heads;
    g.m_tiles = (int)((n_seqs + 47) / 48);
    g.alpha = softmax_scale * 1.4426950408889634f;
    int st = bf16 ? launch_nn<true>(g, s) : launch_nn<false>(g, s);
    if (st != APS_OK) return st;
    APS_LAUNCH(seq_plan_kernel, dim3(1), dim3(256), 0, s, seq_start, (int)n_seqs, kScTokens, tiles, order,
               (u32x4*)(ws + p.off_zero), (int)(p.zero_bytes / 16));
    st = launch_status();
    if (st != APS_OK) return st;
  }
  // (the stores are complete or enqueued by now: an attention job that cannot ride goes here, by itself)
  if (kv_job && !ride) {
    const int st = aps_attention_job_launch(kv_job, stream);
    if (st != APS_OK) return st;
  }
  // 2. S[s][h][t] = <qt[s][h], hidden row t of sequence s>
  {
    ScoreArgs g{};
    g.cache = (const char*)paged_cache; g.slot_stride_b = slot_stride * 2; g.num_slots = num_slots;
    g.row_ids = hidden_slots; g.row_start = seq_start;
    g.qt = qt; g.qt_batch_stride_b = (int64_t)num_heads * hidden * 2; g.qt_row_stride_b = hidden * 2;
    g.heads = num_heads;
    g.s = sc; g.s_batch_stride = (int64_t)num_heads * p.lp; g.s_row_stride = p.lp;
    g.k = hidden;
    g.tile_start = tiles; g.n_seqs = (int)n_seqs;
    g.k_per_part = p.score_k_per_part; g.s_part_stride = s_part_stride;
    // upper bound of the tile count that the host can know: every sequence at max_len
    const int64_t max_tiles = ((max_len + kScTokens - 1) / kScTokens) * n_seqs;
    if (max_tiles > 0x7fffffff) return APS_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((max_tiles + 7) / 8 * 8), (unsigned)p.score_parts);  // whole eighths of the list
    const int nht = (num_heads + 15) / 16;
    hipError_t e = hipSuccess;
#define APS_LAUNCH_SCORES(B, N)                                                                                   \
  do {                                                                                                            \
    e = allow_dynamic_lds((const void*)hidden_scores_kernel<B, N>, scores_lds_bytes<N>(), (B ? 6 : 0) + N - 1);   \
    if (e == hipSuccess)                                                                                          \
      APS_LAUNCH((hidden_scores_kernel<B, N>), grid, dim3(kScThreads), scores_lds_bytes<N>(), s, g);      \
  } while (0)
#define APS_LAUNCH_SCORES_N(B)                                                                        \
  switch (nht) {                                                                                      \
    case 1: APS_LAUNCH_SCORES(B, 1); break;                                                           \
    case 2: APS_LAUNCH_SCORES(B, 2); break;                                                           \
    case 3: APS_LAUNCH_SCORES(B, 3); break;                                                           \
    case 4: APS_LAUNCH_SCORES(B, 4); break;                                                           \
    case 5: APS_LAUNCH_SCORES(B, 5); break;                                                           \
    default: APS_LAUNCH_SCORES(B, 6); break;                                                          \
  }
    if (bf16) { APS_LAUNCH_SCORES_N(true) } else { APS_LAUNCH_SCORES_N(false) }
#undef APS_LAUNCH_SCORES_N
#undef APS_LAUNCH_SCORES
    if (e != hipSuccess) return (int)e;
    const int st = launch_status();
    if (st != APS_OK) return st;
  }
  if (p.score_parts > 1) {
    const int64_t n = n_seqs * num_heads * p.lp;   // a multiple of 32
    APS_LAUNCH(score_parts_sum_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, s, sc, n, p.score_parts,
               s_part_stride);
    const int st = launch_status();
    if (st != APS_OK) return st;
  }
  // 3. ctx[s][h][:] = sum_t softmax_t(S[s][h])[t] * hidden row t: online softmax inside the pass over the rows
  {
    WsumArgs g{};
    g.s = sc; g.s_batch_stride = (int64_t)num_heads * p.lp; g.s_row_stride = p.lp;
    g.cache = (const char*)paged_cache; g.slot_stride_b = slot_stride * 2; g.num_slots = num_slots;
    g.row_ids = hidden_slots; g.row_start = seq_start;
    g.zero_row = ws + p.off_zero;
    g.heads = num_heads; g.m_tiles = (num_heads + 47) / 48; g.n_seqs = (int)n_seqs; g.k_per_part = p.k_per_part;
    g.n = hidden;
    g.out = ctx; g.out_batch_stride = (int64_t)num_heads * hidden; g.out_row_stride = hidden;
    g.partial = p.kparts > 1 ? partial : nullptr;
    g.partial_ml = p.kparts > 1 ? (float*)(ws + p.off_ml) : nullptr;
    g.order = order;
    const int mt = g.m_tiles > 1 ? 3 : (num_heads + 15) / 16;
    const dim3 grid((unsigned)((hidden + kWsWaves * 128 - 1) / (kWsWaves * 128)), (unsigned)(n_seqs * g.m_tiles),
                    (unsigned)p.kparts);
#define APS_LAUNCH_WSUM_K(K, B)                                                             \
  switch (mt) {                                                                             \
    case 1: APS_LAUNCH((K<B, 1>), grid, dim3(kWsThreads), 0, s, g); break;                  \
    case 2: APS_LAUNCH((K<B, 2>), grid, dim3(kWsThreads), 0, s, g); break;                  \
    default: APS_LAUNCH((K<B, 3>), grid, dim3(kWsThreads), 0, s, g); break;                 \
  }
#define APS_LAUNCH_WSUM(B) \
  if (p.chunked) { APS_LAUNCH_WSUM_K(hidden_wsum_chunk_kernel, B) } else { APS_LAUNCH_WSUM_K(hidden_wsum_kernel, B) }
#define APS_LAUNCH_WSUM_RIDE(B)                                                                                    \
  switch (mt) {                                                                                                    \
    case 1: APS_LAUNCH((hidden_wsum_chunk_and_paged_kernel<B, 1>), rgrid, dim3(kWsThreads), 0, s, g, kv_job->a,    \
                       (int)grid.z, head_groups, (int)items); break;                                               \
    case 2: APS_LAUNCH((hidden_wsum_chunk_and_paged_kernel<B, 2>), rgrid, dim3(kWsThreads), 0, s, g, kv_job->a,    \
                       (int)grid.z, head_groups, (int)items); break;                                               \
    default: APS_LAUNCH((hidden_wsum_chunk_and_paged_kernel<B, 3>), rgrid, dim3(kWsThreads), 0, s, g, kv_job->a,   \
                        (int)grid.z, head_groups, (int)items); break;                                              \
  }
    if (ride) {   // slices of the grid behind the chunks hold the attention's (head group, sequence) items
      const int head_groups = kv_job->a.num_heads;
      const int64_t items = (int64_t)head_groups * kv_job->batch;
      const int64_t per_slice = (int64_t)grid.x * grid.y;
      const int64_t slices = (items + per_slice - 1) / per_slice;
      if (grid.z + slices > 65535) return APS_ERR_UNSUPPORTED;
      const dim3 rgrid(grid.x, grid.y, (unsigned)(grid.z + slices));
      if (bf16) { APS_LAUNCH_WSUM_RIDE(true) } else { APS_LAUNCH_WSUM_RIDE(false) }
    } else if (bf16) { APS_LAUNCH_WSUM(true) } else { APS_LAUNCH_WSUM(false) }
#undef APS_LAUNCH_WSUM_RIDE
#undef APS_LAUNCH_WSUM
#undef APS_LAUNCH_WSUM_K
    int st = launch_status();
    if (st != APS_OK) return st;
    if (p.kparts > 1) {
      const int64_t quads = n_seqs * num_heads * hidden / 4;
      const dim3 rgrid((unsigned)((quads + 255) / 256));
      if (bf16)
        APS_LAUNCH(wsum_combine_kernel<true>, rgrid, dim3(256), 0, s, partial, g.partial_ml, ctx, p.kparts, (int)n_seqs,
                   num_heads, hidden, g.out_batch_stride, g.out_row_stride);
      else
        APS_LAUNCH(wsum_combine_kernel<false>, rgrid, dim3(256), 0, s, partial, g.partial_ml, ctx, p.kparts,
                   (int)n_seqs, num_heads, hidden, g.out_batch_stride, g.out_row_stride);
      st = launch_status();
      if (st != APS_OK) return st;
    }
  }
  // 5. out[seq_rows[s]][h*D + d] = <W_v[h*D + d], ctx[s][h]> + b_v
  // few sequences: the weight-streaming kernels read W_v once; up to kHeadwiseMaxSeqs where those kernels cover the
  // shape (heads of whole 128-row tiles): K parts fill the chip where (head, 48 sequences) workgroups do not
  if (n_seqs <= 16 || (n_seqs <= kHeadwiseMaxSeqs &&
                       aps_internal_headwise_workspace_bytes(n_seqs, hidden, hidden, head_size) > 0))
    return aps_internal_headwise_linear(ctx, w_v, b_v, out, n_seqs, hidden, hidden, (int64_t)num_heads * hidden,
                                        hidden, head_size, w_stride, out_stride, seq_rows, out_rows, dtype,
                                        ws + p.off_vp, p.total - p.off_vp, (int32_t*)(ws + p.off_vp_counters), s);
  {
    HeadProjArgs g{};
    g.w = (const char*)w_v; g.w_stride_b = w_stride * 2; g.head_rows = head_size; g.heads = num_heads;
    g.x = ctx; g.x_row_stride_b = (int64_t)num_heads * hidden * 2; g.x_head_stride_b = hidden * 2;
    g.m_rows = (int)n_seqs;
    g.bias = (const char*)b_v;
    g.out = (char*)out; g.out_stride = out_stride; g.out_row_map = seq_rows; g.out_rows = out_rows;
    g.k = hidden;
    g.row_tiles = (head_size + kScTokens - 1) / kScTokens;
    // image of 32 or 48 sequences: whichever needs fewer rounds of workgroups over the 256 CUs; on a tie the
    // smaller one, which gives more workgroups (measured at 128 sequences x 40 heads: 56 us against 59 us)
    auto rounds = [&](int nht) {
      const int64_t wgs = (int64_t)num_heads * g.row_tiles * ((n_seqs + 16 * nht - 1) / (16 * nht));
      return (wgs + 255) / 256;
    };
    const int nht = rounds(3) < rounds(2) ? 3 : 2;
    g.m_tiles = (int)((n_seqs + 16 * nht - 1) / (16 * nht));
    const dim3 grid((unsigned)(g.m_tiles * num_heads * g.row_tiles));
    hipError_t e = hipSuccess;
#define APS_LAUNCH_PROJ(B, N)                                                                                    \
  do {                                                                                                           \
    e = allow_dynamic_lds((const void*)head_proj_kernel<B, N>, scores_lds_bytes<N>(), 12 + (B ? 2 : 0) + N - 2); \
    if (e == hipSuccess)                                                                                         \
      APS_LAUNCH((head_proj_kernel<B, N>), grid, dim3(kScThreads), scores_lds_bytes<N>(), s, g);         \
  } while (0)
#define APS_LAUNCH_PROJ_N(B)                                                                          \
  if (nht == 2) APS_LAUNCH_PROJ(B, 2); else APS_LAUNCH_PROJ(B, 3);
    if (bf16) { APS_LAUNCH_PROJ_N(true) } else { APS_LAUNCH_PROJ_N(false) }
#undef APS_LAUNCH_PROJ_N
#undef APS_LAUNCH_PROJ
    if (e != hipSuccess) return (int)e;
    return launch_status();
  }
}


int aps_absorbed_attention(const void* q, int64_t q_stride, const int64_t* seq_rows, int64_t num_q_rows,
                           const void* paged_cache, int64_t slot_stride, int64_t num_slots,
                           const int64_t* hidden_slots, const int64_t* seq_start, int64_t n_seqs, int64_t max_len,
                           const void* w_k, const void* w_v, const void* b_v, int64_t w_stride, int num_heads,
                           int head_size, float softmax_scale, void* out, int64_t out_stride, int64_t out_rows,
                           int dtype, void* workspace, int64_t workspace_bytes, aps_stream_t stream) {
  return hybrid_attention_impl(nullptr, nullptr, q, q_stride, seq_rows, num_q_rows, paged_cache, slot_stride, num_slots,
                               hidden_slots, seq_start, n_seqs, max_len, w_k, w_v, b_v, w_stride, num_heads, head_size,
                               softmax_scale, out, out_stride, out_rows, dtype, workspace, workspace_bytes, stream);
}

int aps_hybrid_decode_attention(const void* store_job, const void* kv_job, const void* q, int64_t q_stride,
                                const int64_t* seq_rows, int64_t num_q_rows, const void* paged_cache, int64_t slot_stride, int64_t num_slots,
                                const int64_t* hidden_slots, const int64_t* seq_start, int64_t n_seqs,
                                int64_t max_len, const void* w_k, const void* w_v, const void* b_v, int64_t w_stride,
                                int num_heads, int head_size, float softmax_scale, void* out, int64_t out_stride,
                                int64_t out_rows, int dtype, void* workspace, int64_t workspace_bytes,
                                aps_stream_t stream) {
  if ((kv_job && (addr(kv_job) & 7)) || (store_job && (addr(store_job) & 7))) return APS_ERR_INVALID_ARG;
  return hybrid_attention_impl((const StoreJob*)store_job, (const PagedJob*)kv_job, q, q_stride, seq_rows, num_q_rows, paged_cache, slot_stride,
                               num_slots, hidden_slots, seq_start, n_seqs, max_len, w_k, w_v, b_v, w_stride,
                               num_heads, head_size, softmax_scale, out, out_stride, out_rows, dtype, workspace,
                               workspace_bytes, stream);
}

}  // extern "C"
