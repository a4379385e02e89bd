// Row-streaming MFMA core shared by the kernels whose large operand is a set of K-contiguous rows read once
// from HBM (cached hidden rows, weight rows) and whose small operand (the "image": a few dozen rows) is reused
// by every streamed row.
#pragma once
#include "mfma_common.h"

namespace aps {
namespace {

// A workgroup is 8 wavefronts x 16 streamed rows; the image is staged 512 elements of K at a time; every
// wavefront keeps a ring of 16 wave-wide loads (16 KiB) in flight, one trip round the ring per chunk (a ring of
// 32 loads, tried with 32- and 48-row images where one workgroup fits a CU, made long products slower and short
// ones no faster).
constexpr int kScWaves = 8, kScTokens = kScWaves * 16, kScThreads = kScWaves * 64, kScChunk = 512;
// dynamic LDS of a kernel that calls the core: two buffers of [16*NHT image rows][512 k]
template <int NHT>
constexpr int scores_lds_bytes() { return 2 * NHT * 16 * kScChunk * 2; }

// acc[ht][i] (lane (g4, c)) = sum_k row_c[k] * image[16*ht + 4*g4 + i][k]: row_c = the c-th of the 16 rows that
// this wavefront streams, image rows = q_base + r * q_row_stride_b for r < q_rows (zero beyond), staged through
// lds (scores_lds_bytes<NHT>()).  k is a multiple of 64.  Called by all 8 wavefronts of the workgroup (barriers).
//
// Loading layout: a wave-wide load takes 128 contiguous bytes (64 k) of each of 8 rows, lane l = row l/8, piece
// l%8; rowp0 is this lane's pointer into row l/8, rowp1 into row 8 + l/8 (both + 16 bytes * (l % 8)).  On this
// part scattered rows stream a third faster in 128-byte visits than in 64-byte ones.  Two loads (a pair) hold
// 16 rows x 64 k = two MFMA k-steps.  Operand order for a step is lane 16*g + c: row c, k piece g of the step's
// four.  For the even step (pieces 0-3) one DPP move first puts pieces 0-3 of rows 8-15 (second load, lanes
// with l%8 < 4) over the lanes with l%8 >= 4 of the first load, so that a single ds_bpermute per dword finds
// every (row, piece) in one register; the odd step mirrors that.
template <bool BF16, int NHT>
__device__ __forceinline__ void stream_rows_times_image(const char* rowp0, const char* rowp1, const char* q_base,
                                                        int64_t q_row_stride_b, int q_rows, int64_t k, char* lds,
                                                        float4v (&acc)[NHT]) {
  constexpr int kBuf = NHT * 16 * kScChunk * 2;
  constexpr int kPieces = NHT * 16 * 64;                          // 16-byte pieces of a chunk
  static_assert(kPieces % kScThreads == 0, "pieces are spread evenly over the threads");
  constexpr int kPerThread = kPieces / kScThreads;
  constexpr int kChunkPairs = kScChunk / 64;
  constexpr int kPairs = kChunkPairs;                             // pairs of loads in the ring = pairs of a chunk, so
  constexpr int kScRing = 2 * kPairs;                             // that ring positions are static in the unrolled body
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int last_pair = (int)(k / 64) - 1;
  const int nchunks = (int)((k + kScChunk - 1) / kScChunk);
  const int upper = c >> 3;                                        // rows 8-15 come from the second load
  const int src_even = (8 * (c & 7) + g4 + 4 * upper) * 4;         // byte address of the source lane, even step
  const int src_odd = (8 * (c & 7) + g4 + 4 * (1 - upper)) * 4;

  // image: piece p = (row p / 64, chunk p % 64); thread tid moves pieces tid + j*threads.  Rows past the last
  // one and k past the end of K read the first 16 bytes of the image instead (the one address that is valid
  // whatever the row count, the row length and the row stride are) and are replaced by zeros.
  const char* qsrc[kPerThread];
  bool qok[kPerThread];
  uint32_t qdst[kPerThread];
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    const int p = tid + j * kScThreads;
    const int r = p >> 6, ch = p & 63;
    qok[j] = r < q_rows;
    qsrc[j] = q_base + (int64_t)(qok[j] ? r : 0) * q_row_stride_b + ch * 16;
    qdst[j] = (uint32_t)(r * (kScChunk * 2) + ((ch & ~15) | ((ch ^ r) & 15)) * 16);
  }
  const int64_t k_bytes = k * 2;
  auto fetch_q = [&](int chunk, u32x4(&q)[kPerThread]) {
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const int64_t off = (int64_t)chunk * (kScChunk * 2);
      const bool in_k = off + ((tid + j * kScThreads) & 63) * 16 < k_bytes;   // a short last chunk ends early
      q[j] = *(const u32x4*)(in_k ? qsrc[j] + off : q_base);
    }
  };
  auto store_q = [&](int buf, int chunk, const u32x4(&q)[kPerThread]) {
    char* dst = lds + (buf & 1) * kBuf;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const bool in_k = (int64_t)chunk * (kScChunk * 2) + ((tid + j * kScThreads) & 63) * 16 < k_bytes;
      *(u32x4*)(dst + qdst[j]) = (qok[j] && in_k) ? q[j] : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto pair_at = [&](int i) { return (int64_t)min(i, last_pair) * 128; };  // byte offset of the i-th pair, clamped

#pragma unroll
  for (int ht = 0; ht < NHT; ++ht) acc[ht] = float4v{0.f, 0.f, 0.f, 0.f};
  u32x4 qreg[kPerThread];
  fetch_q(0, qreg);
  u32x4 ring[kScRing];
#pragma unroll
  for (int d = 0; d < kPairs - 1; ++d) {
    ring[2 * d] = __builtin_nontemporal_load((const u32x4*)(rowp0 + pair_at(d)));
    ring[2 * d + 1] = __builtin_nontemporal_load((const u32x4*)(rowp1 + pair_at(d)));
  }
  // the image's first chunk goes to LDS only now: the first rows are already on their way while the workgroup
  // waits for it (loads return in order, so this waits for the image alone), one memory round trip instead of two
  // before the first product
  __builtin_amdgcn_sched_barrier(0);
  store_q(0, 0, qreg);
  APS_WAIT_LGKM0();  // own LDS writes done; no fence: it would also wait for the row loads in flight
  APS_BARRIER();     // chunk 0 of the image is in LDS

  // operands of MFMA step st (0..15 within a chunk) from pair u of the ring and the current image buffer
  auto fetch_operands = [&](const char* qrow, int u, int st, u32x4& bf, u32x4(&af)[NHT]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int lo = (int)ring[2 * u][d], hi = (int)ring[2 * u + 1][d];
      // even step: lanes l%8 >= 4 (banks 1, 3 of a 16-lane row) take the second load from 4 lanes below;
      // odd step: lanes l%8 < 4 (banks 0, 2) take it from 4 lanes above
      const int merged = (st & 1) == 0 ? __builtin_amdgcn_update_dpp(lo, hi, 0x114 /* row_shr:4 */, 0xf, 0xa, false)
                                       : __builtin_amdgcn_update_dpp(lo, hi, 0x104 /* row_shl:4 */, 0xf, 0x5, false);
      bf[d] = (uint32_t)__builtin_amdgcn_ds_bpermute((st & 1) == 0 ? src_even : src_odd, merged);
    }
    const int ch = 4 * st + g4;  // 16-byte piece of the image row within the 512-element chunk
#pragma unroll
    for (int ht = 0; ht < NHT; ++ht)
      af[ht] = *(const u32x4*)(qrow + ht * 16 * (kScChunk * 2) + ((ch & ~15) | ((ch ^ c) & 15)) * 16);
  };

  for (int chunk = 0; chunk < nchunks; ++chunk) {
    fetch_q(min(chunk + 1, nchunks - 1), qreg);
    const char* qrow = lds + (chunk & 1) * kBuf + c * (kScChunk * 2);
    const int i0 = chunk * kChunkPairs;
    // The operands of step st+1 (a DPP move, a ds_bpermute and NHT LDS reads) are fetched while the MFMAs of
    // step st run.
    u32x4 bf[2], af[2][NHT];
#pragma unroll
    for (int st = 0; st < 2 * kChunkPairs; ++st) {
      const int u = st >> 1;   // pair within the ring
      if ((st & 1) == 0) {
        const int64_t ahead = pair_at(i0 + u + kPairs - 1);
        ring[2 * ((u + kPairs - 1) % kPairs)] = __builtin_nontemporal_load((const u32x4*)(rowp0 + ahead));
        ring[2 * ((u + kPairs - 1) % kPairs) + 1] = __builtin_nontemporal_load((const u32x4*)(rowp1 + ahead));
        __builtin_amdgcn_sched_barrier(0);  // keep the loads here: the scheduler would sink them to their use
      }
      if (st == 0) fetch_operands(qrow, u, 0, bf[0], af[0]);
      if (st + 1 < 2 * kChunkPairs) fetch_operands(qrow, (st + 1) >> 1, st + 1, bf[(st + 1) & 1], af[(st + 1) & 1]);
#pragma unroll
      for (int ht = 0; ht < NHT; ++ht)
        acc[ht] = mfma16<BF16>(af[st & 1][ht], bf[st & 1], acc[ht]);  // k past the end meets the image's zeros
      if (st & 1) __builtin_amdgcn_sched_barrier(0);
    }
    store_q(chunk + 1, chunk + 1, qreg);  // the other buffer: last read one chunk ago, which every wavefront has left
    APS_WAIT_LGKM0();
    APS_BARRIER();
  }
}

}  // namespace
}  // namespace aps
