// Decode attention of hidden-cached sequences computed on the cached hidden rows themselves
// ("absorbed" projection weights), for gfx950.
//
// For a hidden-cached sequence the K and V of a context token are W_k h_t + b_k and W_v h_t + b_v.
// Instead of re-projecting every cached row in every layer,
//     s[h][t] = scale * <W_k[h]^T q[h], h_t>      (the b_k term is the same for all t: softmax drops it)
//     out[h]  = W_v[h] (sum_t p[h][t] h_t) + b_v[h]
// so the hidden rows are read twice (scores, then the weighted sum) and the projections shrink to
// products with one row per sequence and head:
//   1. qt[s][h][:]  = scale*log2(e) * W_k[h]^T q[s][h]            nn_few_rows_kernel (B = rows of W_k)
//   2. S[s][h][t]   = <qt[s][h], h_t>                               seq_plan_kernel (work list of the ragged
//                                                                   batch), hidden_scores_kernel (paged rows)
//   3. P[s][h][:]   = softmax_t, 16-bit, zero padded to 32 tokens   softmax_rows_kernel
//   4. ctx[s][h][:] = sum_t P[s][h][t] h_t                          nn_few_rows_kernel (B = paged rows)
//   5. out[s][h*D+d] = <W_v[h*D+d], ctx[s][h]> + b_v                head_proj_kernel; up to 16 sequences: the
//                                                                   weight-streaming kernels of the projection
//                                                                   file, x chosen per head
// Per cached token and layer that is 2 x Hd x 2 bytes of HBM reads and ~4*H*Hd flops, against a
// gather, a 4*Hd*Hd-flop GEMM, a cache write and an attention read for the re-projection flow.
#include "aps_common.h"
#include "mfma_common.h"
#include "row_stream_core.h"

namespace aps {
namespace {

// ------------------------------------------------------------------ NN product with few rows
// out[z][m][n] = alpha * sum_k A[z][m][k] * B[row(z,k)][n],  m < m_rows (tiles of 16*MT rows), k < K(z).
// B rows are n-contiguous; row(z,k) = row_ids[row_start[z] + k] (paged rows) or z*k_fixed + k.
// A is K-contiguous and readable (finite, normally zero) up to the next multiple of 32 in k.
//
// The matrix core wants, per lane, 8 consecutive k of one column.  A lane therefore loads an 8x8
// block (8 rows k, 16 bytes = 8 columns each; the 16 lanes of a quarter-wave read 256 contiguous
// bytes of a row), transposes it in registers with v_perm_b32 and feeds 8 MFMAs, MFMA j taking
// column 8c+j from lane (g, c).  No LDS for the data; a workgroup of 4 wavefronts covers 512 columns.
struct NnArgs {
  const char* a; int64_t a_batch_stride_b, lda_b; int m_rows;
  const int64_t* a_row_ids; int64_t num_a_rows;  // nullable: row m of A is row a_row_ids[m] (rows of lda_b bytes)
  const char* b; int64_t b_row_stride_b, num_b_rows;
  const int64_t* row_ids; const int64_t* row_start; int k_fixed;
  int64_t n;
  char* out; int64_t out_batch_stride, out_row_stride;  // elements
  float* partial;  // non-null: fp32 partial sums [k part][batch][m_rows][n] instead of out
  int batches, k_per_part, m_tiles;
  float alpha;
  const int32_t* batch_order;  // nullable: the y-th batch dispatched is batch_order[y] (longest first)
};

// 4 wavefronts per workgroup, two workgroups per CU (256 registers per wavefront: a 3-deep ring of row blocks
// beside 96 accumulator registers).  Eight wavefronts per CU with two blocks in flight each stream faster than four
// with three (188 against 205 us on 87 591 rows): loads return in order per wavefront, so the number of
// independent streams counts, not only the bytes in flight.
constexpr int kNnWaves = 4;
constexpr int kNnRing = 3;
constexpr int kNnMaxPart = 4096;  // rows of B per k-partition when they are addressed through row_ids

template <bool BF16, int MT>
__global__ __launch_bounds__(kNnWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void nn_few_rows_kernel(
    const NnArgs g) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int zi = blockIdx.y / g.m_tiles;
  const int z = g.batch_order ? g.batch_order[zi] : zi;
  const int m0 = (blockIdx.y % g.m_tiles) * (16 * MT);
  int64_t rs = 0;
  int K = g.k_fixed;
  if (g.row_ids) {
    rs = g.row_start[z];
    K = (int)(g.row_start[z + 1] - rs);
  }
  const int kbeg = blockIdx.z * g.k_per_part;
  const int kend = min(K, kbeg + g.k_per_part);
  // Row ids of this partition go to LDS first: read from there they cost an LDS access instead of a global
  // load whose result every row load would have to wait for, one after the other.
  __shared__ __attribute__((aligned(16))) int64_t ids[kNnMaxPart];
  if (g.row_ids) {
    const int staged = (kend - kbeg + 31) / 32 * 32;
    for (int i = tid; i < staged; i += kNnWaves * 64) ids[i] = kbeg + i < kend ? g.row_ids[rs + kbeg + i] : -1;
    __syncthreads();
  }
  const int64_t col0 = (int64_t)blockIdx.x * (kNnWaves * 128) + wave * 128 + 8 * c;
  const bool col_ok = col0 < g.n;
  const char* a_base = g.a + (int64_t)z * g.a_batch_stride_b;  // uniform; rows of a batch lie within 4 GiB of it
  uint32_t a_off[MT];
  bool a_ok[MT];
#pragma unroll
  for (int ht = 0; ht < MT; ++ht) {
    const int m = m0 + 16 * ht + c;
    a_ok[ht] = m < g.m_rows;
    int64_t arow = m;
    if (a_ok[ht] && g.a_row_ids) {
      arow = g.a_row_ids[m];
      a_ok[ht] = arow >= 0 && arow < g.num_a_rows;
    }
    if (!a_ok[ht]) arow = g.a_row_ids ? 0 : m0;  // a row that exists; its product is discarded
    a_off[ht] = (uint32_t)(arow * g.lda_b + g4 * 16);
  }
  float4v acc[MT][8];
#pragma unroll
  for (int ht = 0; ht < MT; ++ht)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[ht][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // Loads are unconditional (a row or column that does not exist reads row 0 / column 0 and is replaced by
  // zeros afterwards): with per-lane branches around them the wait counts before the MFMAs degrade to
  // "everything outstanding", which serialises the two register sets.
  const char* b_col = g.b + (col_ok ? col0 : 0) * 2;
  auto load_step = [&](int t0, u32x4(&r)[8], u32x4(&pf)[MT], uint32_t& bad) {
    int64_t row[8];
    if (g.row_ids) {
      const u32x4* src = (const u32x4*)(ids + (t0 - kbeg + 8 * g4));  // 8 ids = 64 bytes, 64-byte aligned
      const u32x4 q0 = src[0], q1 = src[1], q2 = src[2], q3 = src[3];
      row[0] = (int64_t)q0[0] | ((int64_t)q0[1] << 32); row[1] = (int64_t)q0[2] | ((int64_t)q0[3] << 32);
      row[2] = (int64_t)q1[0] | ((int64_t)q1[1] << 32); row[3] = (int64_t)q1[2] | ((int64_t)q1[3] << 32);
      row[4] = (int64_t)q2[0] | ((int64_t)q2[1] << 32); row[5] = (int64_t)q2[2] | ((int64_t)q2[3] << 32);
      row[6] = (int64_t)q3[0] | ((int64_t)q3[1] << 32); row[7] = (int64_t)q3[2] | ((int64_t)q3[3] << 32);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) row[i] = (int64_t)z * g.k_fixed + t0 + 8 * g4 + i;
    }
    bad = 0;  // bit i: row i of this lane does not exist; applied when the block is consumed
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const bool ok = col_ok && (t0 + 8 * g4 + i < kend) && row[i] >= 0 && row[i] < g.num_b_rows;
      if (!ok) bad |= 1u << i;
      const int64_t rr = ok ? row[i] : 0;
      r[i] = __builtin_nontemporal_load((const u32x4*)(b_col + rr * g.b_row_stride_b));
    }
#pragma unroll
    for (int ht = 0; ht < MT; ++ht) pf[ht] = *(const u32x4*)(a_base + (a_off[ht] + (uint32_t)t0 * 2));
  };
  auto mac_step = [&](u32x4(&r)[8], u32x4(&pf)[MT], uint32_t bad) {
    if (__builtin_amdgcn_ballot_w64(bad != 0) != 0) {  // rare: the last step of a sequence
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
  int t0 = kbeg;
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
      if (g.partial) {
        float* dst = g.partial + (((int64_t)blockIdx.z * g.batches + z) * g.m_rows + m) * g.n + col0;
        *(float4v*)dst = float4v{acc[ht][0][i], acc[ht][1][i], acc[ht][2][i], acc[ht][3][i]};
        *(float4v*)(dst + 4) = float4v{acc[ht][4][i], acc[ht][5][i], acc[ht][6][i], acc[ht][7][i]};
      } else {
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
}

// out[z][m][n] = alpha * sum_p partial[p][z][m][n], 4 columns per thread
template <bool BF16>
__global__ __launch_bounds__(256) void nn_reduce_kernel(const float* __restrict__ partial, char* out, int parts,
                                                        int batches, int m_rows, int64_t n, int64_t out_batch_stride,
                                                        int64_t out_row_stride, float alpha) {
  const int64_t per_part = (int64_t)batches * m_rows * n;
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (idx >= per_part) return;
  float4v s = *(const float4v*)(partial + idx);
  int p = 1;
  for (; p + 3 < parts; p += 4) {  // four independent loads in flight; additions in the order of one at a time
    const float4v v0 = *(const float4v*)(partial + p * per_part + idx);
    const float4v v1 = *(const float4v*)(partial + (p + 1) * per_part + idx);
    const float4v v2 = *(const float4v*)(partial + (p + 2) * per_part + idx);
    const float4v v3 = *(const float4v*)(partial + (p + 3) * per_part + idx);
#pragma unroll
    for (int i = 0; i < 4; ++i) s[i] = (((s[i] + v0[i]) + v1[i]) + v2[i]) + v3[i];
  }
  for (; p < parts; ++p) {
    const float4v v = *(const float4v*)(partial + p * per_part + idx);
    s[0] += v[0]; s[1] += v[1]; s[2] += v[2]; s[3] += v[3];
  }
  const int64_t col = idx % n, zm = idx / n;
  const int64_t m = zm % m_rows, z = zm / m_rows;
  uint16_t* o = (uint16_t*)out + z * out_batch_stride + m * out_row_stride + col;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = BF16 ? f32_to_bf16_bits(s[i] * alpha) : f32_to_f16_bits(s[i] * alpha);
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
__global__ __launch_bounds__(256) void seq_plan_kernel(const int64_t* __restrict__ row_start, int n_seqs,
                                                       int tile_tokens, int32_t* __restrict__ tile_start,
                                                       int32_t* __restrict__ order) {
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

// ------------------------------------------------------------------ softmax over the tokens of a row
// P[z][h][t] = exp2(S - max) / sum for t < L(z), 0 for L <= t < the next multiple of 32; S already carries
// scale*log2(e).
template <bool BF16>
__global__ __launch_bounds__(256) void softmax_rows_kernel(float* __restrict__ s, uint16_t* __restrict__ p,
                                                           const int64_t* __restrict__ row_start, int heads,
                                                           int64_t lp, int parts, int64_t part_stride) {
  // Rows up to kCached scores are summed over the K parts once, 4 tokens per thread and step with the loads of
  // all parts of a step independent of each other, and kept in LDS for the other two passes; longer rows keep
  // their sums in part 0 of the global buffer (a thread meets the same tokens in every pass).
  constexpr int kCached = 4096;
  __shared__ __attribute__((aligned(16))) float cache[kCached];
  __shared__ float red[4];
  const int z = blockIdx.y, h = blockIdx.x;
  const int L = (int)min(row_start[z + 1] - row_start[z], lp);  // a sequence longer than the stated maximum: its head
  float* row = s + ((int64_t)z * heads + h) * lp;   // 16-byte aligned: lp is a multiple of 32
  uint16_t* out = p + ((int64_t)z * heads + h) * lp;
  const bool in_lds = L <= kCached;
  float mx = -INFINITY;
  for (int t = threadIdx.x * 4; t < L; t += 1024) {
    float4 v = *(const float4*)(row + t);
    for (int kp = 1; kp < parts; ++kp) {
      const float4 q = *(const float4*)(row + kp * part_stride + t);
      v.x += q.x; v.y += q.y; v.z += q.z; v.w += q.w;
    }
    if (in_lds) *(float4*)(cache + t) = v;
    else if (parts > 1) *(float4*)(row + t) = v;
    mx = fmaxf(mx, v.x);                       // tokens t+1.. past L hold finite padding of the scores kernel or
    if (t + 1 < L) mx = fmaxf(mx, v.y);        // stale values: only tokens below L count
    if (t + 2 < L) mx = fmaxf(mx, v.z);
    if (t + 3 < L) mx = fmaxf(mx, v.w);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  const float* src = in_lds ? cache : row;     // each thread re-reads what it wrote itself
  float sum = 0.f;
  for (int t = threadIdx.x * 4; t < L; t += 1024) {
    const float4 v = *(const float4*)(src + t);
    sum += exp2f(v.x - mx);
    if (t + 1 < L) sum += exp2f(v.y - mx);
    if (t + 2 < L) sum += exp2f(v.z - mx);
    if (t + 3 < L) sum += exp2f(v.w - mx);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
  __syncthreads();
  sum = (red[0] + red[1]) + (red[2] + red[3]);
  const float inv = 1.f / sum;
  // zero padded to the next multiple of 32 tokens: the weighted sum reads a row's probabilities 32 at a time and
  // never past its sequence
  const int64_t pad_to = min(lp, (int64_t)((L + 31) / 32 * 32));
  for (int64_t t = threadIdx.x * 4; t < pad_to; t += 1024) {
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (t < L) v = *(const float4*)(src + t);
    uint16_t o[4];
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float pv = t + i < L ? exp2f(e[i] - mx) * inv : 0.f;
      o[i] = BF16 ? f32_to_bf16_bits(pv) : f32_to_f16_bits(pv);
    }
    *(uint2*)(out + t) = uint2{(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
  }
}

template <bool BF16>
int launch_nn(const NnArgs& g, int kparts, hipStream_t s) {
  const int mt = g.m_tiles > 1 ? 3 : (g.m_rows <= 16 ? 1 : (g.m_rows <= 32 ? 2 : 3));  // row tiles are 16*mt rows
  const dim3 grid((unsigned)((g.n + kNnWaves * 128 - 1) / (kNnWaves * 128)), (unsigned)(g.batches * g.m_tiles),
                  (unsigned)kparts);
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
  int64_t lp;        // padded row length of S and P
  int kparts;        // token partitions of the weighted sum
  int score_parts;   // parts of K in the scores kernel (partial scores summed by the softmax)
  int64_t score_k_per_part;
  int k_per_part;
  int64_t off_qt, off_s, off_p, off_ctx, off_tiles, off_order, off_partial, total;
};

Plan make_plan(int64_t n_seqs, int64_t max_len, int heads, int64_t hidden) {
  Plan p{};
  p.lp = align_up(max_len > 0 ? max_len : 1, 32);
  const int64_t col_tiles = (hidden + kNnWaves * 128 - 1) / (kNnWaves * 128);
  int64_t parts = 1;
  // Fewer workgroups than CUs (few sequences): split the tokens.  A workgroup walks its tokens one after the
  // other at ~29 GB/s, so without a split the longest sequence sets the kernel's time.  The host knows only the
  // longest length; with lengths spread like a serving batch's the rows in all are about a third of
  // n_seqs * longest, and a part should hold about 1/256 of the work of one column tile.
  if (n_seqs * col_tiles < 256) {
    int64_t target = n_seqs * p.lp * col_tiles / 3 / 256;
    if (target < 64) target = 64;
    parts = (p.lp + target - 1) / target;
    if (parts > 32) parts = 32;
  }
  while (p.lp / parts > kNnMaxPart) parts *= 2;
  p.k_per_part = (int)align_up((p.lp + parts - 1) / parts, 32);
  p.kparts = (int)((p.lp + p.k_per_part - 1) / p.k_per_part);
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
  p.off_p = o; o += align_up(n_seqs * heads * p.lp * 2, 256);
  p.off_ctx = o; o += align_up(n_seqs * heads * hidden * 2, 256);
  p.off_tiles = o; o += align_up((n_seqs + 1) * 4, 256);
  p.off_order = o; o += align_up(n_seqs * 4, 256);
  p.off_partial = o;
  if (p.kparts > 1) o += align_up((int64_t)p.kparts * n_seqs * heads * hidden * 4, 256);
  p.total = o;
  return p;
}

}  // namespace
}  // namespace aps

using namespace aps;

// the per-head value projection lives with the other weight-streaming kernels
__attribute__((visibility("hidden"))) int aps_internal_headwise_linear(const void* x, const void* weight, const void* bias, void* out, int64_t m, int64_t n,
                                 int64_t k, int64_t x_stride, int64_t x_head_stride, int head_rows, int64_t w_stride,
                                 int64_t out_stride, const int64_t* out_row_map, int64_t out_rows, int dtype,
                                 hipStream_t stream);

extern "C" {

int64_t aps_absorbed_attention_workspace_bytes(int64_t n_seqs, int64_t max_len, int num_heads, int head_size) {
  if (n_seqs <= 0 || max_len <= 0 || num_heads <= 0 || head_size <= 0) return 0;
  return make_plan(n_seqs, max_len, num_heads, (int64_t)num_heads * head_size).total;
}

int aps_absorbed_attention(const void* q, int64_t q_stride, const int64_t* seq_rows, int64_t num_q_rows,
                           const void* paged_cache, int64_t slot_stride, int64_t num_slots,
                           const int64_t* hidden_slots, const int64_t* seq_start, int64_t n_seqs, int64_t max_len,
                           const void* w_k, const void* w_v, const void* b_v, int64_t w_stride, int num_heads,
                           int head_size, float softmax_scale, void* out, int64_t out_stride, int64_t out_rows,
                           int dtype, void* workspace, int64_t workspace_bytes, aps_stream_t stream) {
  if (n_seqs < 0 || max_len < 0 || num_heads <= 0 || head_size <= 0) return APS_ERR_INVALID_ARG;
  if (n_seqs == 0) return APS_OK;
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
  if (n_seqs > 65535 || max_len > ((int64_t)1 << 24)) return APS_ERR_UNSUPPORTED;
  const Plan p = make_plan(n_seqs, max_len, num_heads, hidden);
  if (workspace_bytes < p.total) return APS_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const bool bf16 = dtype == APS_BF16;
  char* ws = (char*)workspace;
  char* qt = ws + p.off_qt;
  float* sc = (float*)(ws + p.off_s);
  const int64_t s_part_stride = align_up(n_seqs * num_heads * p.lp * 4, 256) / 4;  // elements between K parts
  char* pr = ws + p.off_p;
  char* ctx = ws + p.off_ctx;
  float* partial = (float*)(ws + p.off_partial);

  // 1. qt[s][h][:] = scale*log2(e) * W_k[h]^T q[seq_rows[s]][h]: batch = head, K = head_size, B = rows of W_k
  {
    NnArgs g{};
    g.a = (const char*)q; g.a_batch_stride_b = (int64_t)head_size * 2; g.lda_b = q_stride * 2;
    g.m_rows = (int)n_seqs; g.a_row_ids = seq_rows; g.num_a_rows = num_q_rows;
    g.b = (const char*)w_k; g.b_row_stride_b = w_stride * 2; g.num_b_rows = hidden;
    g.row_ids = nullptr; g.row_start = nullptr; g.k_fixed = head_size;
    g.n = hidden;
    g.out = qt; g.out_batch_stride = hidden; g.out_row_stride = (int64_t)num_heads * hidden;
    g.partial = nullptr; g.batches = num_heads; g.k_per_part = head_size;
    g.m_tiles = (int)((n_seqs + 47) / 48);
    g.alpha = softmax_scale * 1.4426950408889634f;
    const int st = bf16 ? launch_nn<true>(g, 1, s) : launch_nn<false>(g, 1, s);
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
    int32_t* tiles = (int32_t*)(ws + p.off_tiles);
    int32_t* order = n_seqs > 1 && n_seqs <= kMaxOrderedSeqs ? (int32_t*)(ws + p.off_order) : nullptr;
    APS_LAUNCH(seq_plan_kernel, dim3(1), dim3(256), 0, s, seq_start, (int)n_seqs, kScTokens, tiles, order);
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
  // 3. P = softmax over the tokens, zero padded to whole groups of 32 tokens
  {
    const dim3 grid((unsigned)num_heads, (unsigned)n_seqs);
    if (bf16)
      APS_LAUNCH(softmax_rows_kernel<true>, grid, dim3(256), 0, s, sc, (uint16_t*)pr, seq_start, num_heads, p.lp,
                         p.score_parts, s_part_stride);
    else
      APS_LAUNCH(softmax_rows_kernel<false>, grid, dim3(256), 0, s, sc, (uint16_t*)pr, seq_start, num_heads, p.lp,
                         p.score_parts, s_part_stride);
    const int st = launch_status();
    if (st != APS_OK) return st;
  }
  // 4. ctx[s][h][:] = sum_t P[s][h][t] * hidden row t: batch = sequence, K = its length, B = paged rows
  {
    NnArgs g{};
    g.a = pr; g.a_batch_stride_b = (int64_t)num_heads * p.lp * 2; g.lda_b = p.lp * 2;
    g.m_rows = num_heads; g.a_row_ids = nullptr; g.num_a_rows = num_heads;
    g.b = (const char*)paged_cache; g.b_row_stride_b = slot_stride * 2; g.num_b_rows = num_slots;
    g.row_ids = hidden_slots; g.row_start = seq_start; g.k_fixed = 0;
    g.n = hidden;
    g.out = ctx; g.out_batch_stride = (int64_t)num_heads * hidden; g.out_row_stride = hidden;
    g.partial = p.kparts > 1 ? partial : nullptr;
    g.batches = (int)n_seqs; g.k_per_part = p.k_per_part;
    g.m_tiles = (num_heads + 47) / 48;
    g.alpha = 1.f;
    if (n_seqs > 1 && n_seqs <= kMaxOrderedSeqs) g.batch_order = (const int32_t*)(ws + p.off_order);  // from step 2
    int st = bf16 ? launch_nn<true>(g, p.kparts, s) : launch_nn<false>(g, p.kparts, s);
    if (st != APS_OK) return st;
    if (p.kparts > 1) {
      const int64_t quads = n_seqs * num_heads * hidden / 4;
      const dim3 rgrid((unsigned)((quads + 255) / 256));
      if (bf16)
        APS_LAUNCH(nn_reduce_kernel<true>, rgrid, dim3(256), 0, s, partial, ctx, p.kparts, (int)n_seqs,
                           num_heads, hidden, g.out_batch_stride, g.out_row_stride, 1.f);
      else
        APS_LAUNCH(nn_reduce_kernel<false>, rgrid, dim3(256), 0, s, partial, ctx, p.kparts, (int)n_seqs,
                           num_heads, hidden, g.out_batch_stride, g.out_row_stride, 1.f);
      st = launch_status();
      if (st != APS_OK) return st;
    }
  }
  // 5. out[seq_rows[s]][h*D + d] = <W_v[h*D + d], ctx[s][h]> + b_v
  if (n_seqs <= 16)  // few sequences: the weight-streaming kernels read W_v once
    return aps_internal_headwise_linear(ctx, w_v, b_v, out, n_seqs, hidden, hidden, (int64_t)num_heads * hidden,
                                        hidden, head_size, w_stride, out_stride, seq_rows, out_rows, dtype, s);
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

}  // extern "C"
