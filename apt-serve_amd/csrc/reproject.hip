// K/V re-projection GEMM for gfx950:  C[M,N] = A[M,K] * W[N,K]^T + bias[N]
// fp16 or bf16 operands, fp32 accumulation on the matrix cores, result in the
// operand dtype.  Both operands are K-contiguous ("NT"), which is how the
// fused QKV weight [3*Hd, Hd] and the holder of gathered hidden rows [T, Hd]
// are laid out.
//
// Tiling: one 512-thread workgroup (8 wavefronts, 2 x 4) owns a 256 x 256 tile
// of C; each wavefront owns 128 x 64 = 8 x 4 tiles of v_mfma_f32_16x16x32 (128
// fp32 accumulator registers per lane), so two wavefronts fit on every SIMD.
// That matters more than the larger per-wave tile it replaces: a wavefront issues
// in order, and while it is held at a global load the matrix core of its SIMD is
// only kept busy by the other wavefront (with one wavefront per SIMD the main
// loop took 1.4x the cycles).  The instruction shape is a matter of power: on
// random operands the part lowers its clock until the matrix cores fit its power
// limit, and 16x16x32 (32 multiply-adds per accumulator element and instruction)
// needs less energy per flop than 32x32x16 (16): alone, with operands in
// registers, they sustain 1.8 against 1.4-1.6 PFLOP/s (aps_mfma_probe).
// The K loop moves BK = 64 at a time through a two-stage LDS ring (2 x (32 + 32)
// KiB of the 160 KiB per CU; 144 KiB with the epilogue images): tile t+1 is
// copied global -> LDS by buffer_load ... lds (no VGPR round trip) while the
// matrix cores consume tile t.
//
// LDS layout: a tile is [256 rows][8 chunks of 16 B]; chunk c of row r lives at
// position c ^ ((r >> 1) % 8).  The LDS of gfx950 serves a 128-bit read to 16
// lanes per cycle over 64 banks, so the 16 consecutive rows those lanes read
// (2 rows x 8 chunks per 256 B of banks) must all land in different 16-byte
// bank groups; with an 8-row swizzle half of all LDS cycles were conflicts
// (SQ_LDS_BANK_CONFLICT).  The DMA writes 1 KiB per wavefront in lane order,
// so the swizzle is applied on the global side: lane l of a wave-wide load
// fetches chunk (l%8) ^ ((row>>1)%8) of row l/8 of its 8-row group.
//
// Schedule: a tile is two k-steps of 32; fragments live in two register sets;
// while the matrix cores work on k-step s the 12 ds_read_b128 of k-step s+1 are
// in flight (32 MFMA : 12 reads).
// Before the last k-step of a tile every wave has its fragments in registers,
// so after one barrier the stage can be refilled with tile t+2 while the last
// k-step runs and the first fragments of tile t+1 stream in.  Waits and the
// barrier are written as asm so that no fence forces all DMA traffic to drain.
//
// Workgroups are renumbered so that the 32 workgroups an XCD runs together
// form an 8 x 4 block of tiles and share their A and W panels in that XCD's L2.
#include "aps_common.h"
#include "mfma_common.h"
#include "row_stream_core.h"

namespace aps {
namespace {

constexpr int BM = 256, BN = 256, BK = 64;      // BM: rows of the full-size tile (MI = 4)
constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int WN = 64;                            // columns of a wavefront tile
constexpr int kWTileBytes = BN * BK * 2;          // 32 KiB
constexpr int kStages = 2;
constexpr int kEpiPitch = WN * 2 + 16;            // bytes per row of a wave's epilogue image
// The tile has 2 x 4 wavefronts of (32*MI rows) x 64 columns: 64*MI rows in all.  MI = 4 is the tile for large
// M; with 49..128 rows it would spend most of its matrix-core time on rows that do not exist (and that time,
// not the weight stream, bounds the product there), hence MI = 1, 2 and 3.
template <int MI>
struct TileShape {
  static constexpr int kWm = 32 * MI, kBm = 2 * kWm;
  static constexpr int kATileBytes = kBm * BK * 2;
  static constexpr int kStageBytes = kATileBytes + kWTileBytes;
  static constexpr int kEpiWaveBytes = kWm * kEpiPitch;
  static constexpr int kLdsBytes =
      kWaves * kEpiWaveBytes > kStages * kStageBytes ? kWaves * kEpiWaveBytes : kStages * kStageBytes;
};
constexpr int kNumXcd = 8;
constexpr int kNumCus = 256;
constexpr int kGroupM = 8;
constexpr int kSkinnyMaxRows = 16;  // at most this many rows: the weight-streaming MFMA kernel without workspace
constexpr int kRsMaxRows = 2;       // at most this many rows: the dot-product kernel

// Where a result row goes.  Plain: row t of C is row t (or map[t], negative skipped) of base[0], ld elements
// apart.  Cache mode (n_split > 0): columns below n_split are the K part of the row and columns from n_split
// on its V part; map[t] >= 0 is a slot of the workspace caches base[0] (K) / base[1] (V), map[t] <= -2 is
// slot -(map[t]+2) of the private caches base[2] / base[3], -1 is skipped; a slot is ld elements.
struct OutMap {
  char* base[4];
  int64_t ld;
  int64_t n_split;
  const int64_t* map;
  int64_t limit0, limit1;  // rows (plain) or workspace slots; private slots
  int aligned16;           // every base and the pitch allow 128-bit stores
  int relu;                // negative results are stored as zero (the activation between fc1 and fc2)
};

// max(v, 0) that keeps a NaN, as the element-wise activation on the rounded result would
__device__ __forceinline__ float act(const OutMap& o, float v) { return (o.relu && v < 0.f) ? 0.f : v; }

// Start of result row `row` for the column half `half`; nullptr when the row is skipped.
__device__ __forceinline__ uint16_t* out_row(const OutMap& o, int64_t row, int half) {
  int64_t r = row;
  char* base = half ? o.base[1] : o.base[0];
  if (o.map) {
    r = o.map[row];
    if (o.n_split && r <= -2) {
      r = -(r + 2);
      if (r >= o.limit1) return nullptr;
      base = half ? o.base[3] : o.base[2];
    } else if (r < 0 || r >= o.limit0) {
      return nullptr;
    }
  }
  return base ? (uint16_t*)base + r * o.ld : nullptr;
}

struct GemmArgs {
  const char* a; const char* w; const void* bias;
  int64_t lda_b, ldw_b;  // bytes
  int64_t m, n, k;
  int tiles_m, tiles_n;
  OutMap out;
  // weight-streaming kernels only: weight rows come in groups of head_rows (a head); the rows of group h are
  // multiplied with x[m] + h * x_head_stride_b instead of x[m] (0: one x for all rows)
  int64_t x_head_stride_b;
  int head_rows;
  // split-K (small M): workgroup (tile, z) handles k-tiles [z*kt_per_split, ...) and stores its fp32
  // partial tile to partial[z][m][n]; a second kernel adds the splits and the bias
  float* partial;
  int kt_per_split;
  // weight_stream_kernel only: one zero-initialised counter per output tile.  With it the workgroup that
  // stores a tile's last partial product adds the parts itself (and puts the counter back to zero) instead of
  // leaving them to a second launch.
  int* tile_counters;
  // weight_stream_kernel only: weight rows of a workgroup (a multiple of 16, at most 128; 0 = 128).  The wavefronts
  // beyond them only help to stage the activations.
  int rows_per_wg;
  // tail split (large M): logical tiles from tail_from on are cut into tail_ways parts of tail_kt k-tiles each;
  // part p of tail tile i stores its fp32 result tile at tail_partial[(i * tail_ways + p)][256][256]
  float* tail_partial;
  int tail_from, tail_ways, tail_kt;
  // gathered A operand (GATHER kernels only): row t of A is not a + t*lda but
  //   row_src[t] >= 0:     slot row_src[t] of the paged cache, slot_base + row_src[t] * slot_stride_b
  //   row_src[t] = -(b+1): row b of the step's input, alt_base + b * alt_stride_b  (b < alt_rows)
  // anything else (and rows >= m) reads row 0 of the input: such rows must not be stored (kv_dest = -1).
  const int64_t* row_src;
  const char* slot_base; const char* alt_base;
  int64_t slot_stride_b, alt_stride_b, num_slots, alt_rows;
};

// Logical tile number -> tile coordinates: groups of kGroupM tile rows, column-major inside a group, so that
// consecutive logical tiles share their A and W panels.
__host__ __device__ __forceinline__ void tile_coords(int logical, int tiles_m, int tiles_n, int& pid_m, int& pid_n) {
  const int in_group = kGroupM * tiles_n;
  const int group = logical / in_group;
  const int first_m = group * kGroupM;
  const int gsz = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
  const int r = logical - group * in_group;
  pid_m = first_m + r % gsz;
  pid_n = r / gsz;
}

template <bool BF16, int MI, bool GATHER = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_nt_kernel(
    const GemmArgs g) {
  using T = TileShape<MI>;
  constexpr int WM = T::kWm, TBM = T::kBm, kStageBytes = T::kStageBytes, kTileBytes = T::kATileBytes;
  constexpr int kEpiWaveBytes = T::kEpiWaveBytes;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave >> 2, wn = wave & 3;

  // ---- tile assignment: XCD-contiguous, grouped 8 tiles along M.  Workgroups go to the XCDs round-robin by
  // their linear id, so XCD x gets the ids x, x+8, ...: it is given a contiguous run of logical tiles (and, with
  // a tail split, a contiguous run of the tail parts, which come last).
  int pid_m, pid_n, tail_part = -1, tail_slot = 0;
  {
    const int total = g.tiles_m * g.tiles_n;
    const int w = blockIdx.x;
    const int xcd = w % kNumXcd, idx = w / kNumXcd;
    int logical;
    if (g.tail_ways > 1) {
      const int full_per_xcd = g.tail_from / kNumXcd;  // tail_from is a multiple of the CU count
      const int tail_items = (total - g.tail_from) * g.tail_ways;
      const int tail_per_xcd = (tail_items + kNumXcd - 1) / kNumXcd;
      if (idx < full_per_xcd) {
        logical = xcd * full_per_xcd + idx;
      } else {
        tail_slot = xcd * tail_per_xcd + (idx - full_per_xcd);
        if (idx - full_per_xcd >= tail_per_xcd || tail_slot >= tail_items) return;
        logical = g.tail_from + tail_slot / g.tail_ways;
        tail_part = tail_slot % g.tail_ways;
      }
    } else {
      const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
      logical = xcd * per_xcd + idx;
      if (logical >= total) return;
    }
    tile_coords(logical, g.tiles_m, g.tiles_n, pid_m, pid_n);
  }

  // ---- global -> LDS DMA addressing
  const int64_t row0 = (int64_t)pid_m * TBM, col0 = (int64_t)pid_n * BN;
  const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(g.a + row0 * g.lda_b, (g.m - row0 - 1) * g.lda_b + g.k * 2);
  const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(g.w + col0 * g.ldw_b, (g.n - col0 - 1) * g.ldw_b + g.k * 2);
  const int lrow = lane >> 3;  // row within the 8-row group of a wave-wide load
  // (row >> 1) % 8 of row 8*i + lane/8 is 4*(i&1) + lane/16: two swizzles, for even and odd groups
  const int lchunk0 = (lane & 7) ^ ((lane >> 4) & 7);
  const int lchunk1 = (lane & 7) ^ ((4 + (lane >> 4)) & 7);
  const uint32_t voff_a0 = (uint32_t)(lrow * g.lda_b + lchunk0 * 16), voff_a1 = (uint32_t)(lrow * g.lda_b + lchunk1 * 16);
  const uint32_t voff_w0 = (uint32_t)(lrow * g.ldw_b + lchunk0 * 16), voff_w1 = (uint32_t)(lrow * g.ldw_b + lchunk1 * 16);
  const uint32_t grp_a = (uint32_t)(8 * g.lda_b), grp_w = (uint32_t)(8 * g.ldw_b);
  // gathered A: this lane's row of each of the MI 8-row groups the wavefront loads, swizzled chunk included
  const char* a_row[GATHER ? MI : 1];
  if constexpr (GATHER) {
#pragma unroll
    for (int j = 0; j < MI; ++j) {
      const int i = wave * MI + j;
      const int64_t row = row0 + i * 8 + lrow;
      const char* p = g.alt_base;
      if (row < g.m) {
        const int64_t src = g.row_src[row];
        if (src >= 0) {
          if (src < g.num_slots) p = g.slot_base + src * g.slot_stride_b;
        } else if (-(src + 1) < g.alt_rows) {
          p = g.alt_base + (-(src + 1)) * g.alt_stride_b;
        }
      }
      a_row[j] = p + (((i & 1) ? lchunk1 : lchunk0) * 16);
    }
  }

  const int kt_base_ = tail_part >= 0 ? tail_part * g.tail_kt : (g.partial ? (int)blockIdx.y * g.kt_per_split : 0);
  auto issue_loads = [&](int kt) {
    char* sa = lds + (kt & 1) * kStageBytes;
    char* sw = sa + kTileBytes;
    const uint32_t koff = (uint32_t)(kt_base_ + kt) * (BK * 2);
#pragma unroll
    for (int j = 0; j < MI; ++j) {
      const int i = wave * MI + j;  // 8-row group of the A tile handled by this wave-wide load (8*MI groups)
      if constexpr (GATHER)   // every lane brings the 64-bit address of its own row
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_row[j] + koff),
                                         (__attribute__((address_space(3))) void*)(sa + i * 1024), 16, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(sa + i * 1024), 16,
                                                 (i & 1) ? voff_a1 : voff_a0, koff + i * grp_a, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = wave * 4 + j;   // 8-row group of the W tile (32 groups)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void*)(sw + i * 1024), 16,
                                               (j & 1) ? voff_w1 : voff_w0, koff + i * grp_w, 0, 0);
    }
  };

  // ---- LDS -> register fragment addressing.  v_mfma_f32_16x16x32: lane l holds row (or weight row) l%16 and
  // the 8 elements k = 8*(l/16) .. +7 of a 32-wide k-step, i.e. chunk 4*ks + l/16 of the row, swizzled.  The 16
  // lanes the LDS serves per cycle read 16 consecutive rows at one chunk: 16 different 16-byte bank groups.
  const int frow = lane & 15, fq = lane >> 4;
  const uint32_t a_row_off = (uint32_t)((wm * WM + frow) * (BK * 2));
  const uint32_t w_row_off = (uint32_t)((wn * WN + frow) * (BK * 2));
  uint32_t chunk_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) chunk_off[ks] = (uint32_t)(((4 * ks + fq) ^ ((frow >> 1) & 7)) * 16);

  constexpr int RT = 2 * MI;   // 16-row tiles of a wavefront (its 64 columns are 4 tiles)
  float4v acc[RT][4];
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;

  auto read_frags = [&](int kt, int ks, u32x4(&af)[RT], u32x4(&wf)[4]) {
    const char* sa = lds + (kt & 1) * kStageBytes;
    const char* sw = sa + kTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) wf[i] = *(const u32x4*)(sw + w_row_off + i * (16 * BK * 2) + chunk_off[ks]);
#pragma unroll
    for (int i = 0; i < RT; ++i) af[i] = *(const u32x4*)(sa + a_row_off + i * (16 * BK * 2) + chunk_off[ks]);
  };
  auto mfma_step = [&](const u32x4(&af)[RT], const u32x4(&wf)[4]) {
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mfma16<BF16>(af[i], wf[j], acc[i][j]);
  };
  auto interleave = [&]() {  // scheduling hint: the 12 LDS reads spread over the 32 MFMA of a k-step
    if constexpr (MI != 4) return;  // the small tiles are bound by the weight stream: the compiler's order will do
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 3, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  };

  const int nk_total = (int)(g.k / BK);
  const int kt_base = kt_base_;
  const int nk = tail_part >= 0 ? min(g.tail_kt, nk_total - kt_base)
                                : (g.partial ? min(g.kt_per_split, nk_total - kt_base) : nk_total);
  u32x4 a0[RT], w0[4], a1[RT], w1[4];
  issue_loads(0);
  if (nk > 1) {
    issue_loads(1);
    // tile 0 has landed, tile 1 (4 + MI loads per wavefront) may still be in flight
    if constexpr (MI == 4) APS_WAIT_VM(8); else if constexpr (MI == 3) APS_WAIT_VM(7);
    else if constexpr (MI == 2) APS_WAIT_VM(6); else APS_WAIT_VM(5);
  } else {
    APS_WAIT_VM(0);
  }
  APS_BARRIER();
  read_frags(0, 0, a0, w0);
  int kt = 0;
  for (; kt + 2 < nk; ++kt) {  // steady state: a tile kt+2 exists, the body has no branches
    read_frags(kt, 1, a1, w1); mfma_step(a0, w0); interleave();
    APS_WAIT_LGKM0();  // every fragment of tile kt is in registers: its stage is free
    APS_WAIT_VM(0);    // tile kt+1 has landed (this wave's part; the barrier covers the others)
    APS_BARRIER();
    issue_loads(kt + 2);
    read_frags(kt + 1, 0, a0, w0); mfma_step(a1, w1); interleave();
  }
  for (; kt < nk; ++kt) {  // last two tiles: nothing left to issue
    read_frags(kt, 1, a1, w1); mfma_step(a0, w0); interleave();
    APS_WAIT_LGKM0();
    APS_WAIT_VM(0);
    APS_BARRIER();
    if (kt + 1 < nk) read_frags(kt + 1, 0, a0, w0);
    mfma_step(a1, w1);
  }

  // ---- epilogue: bias, round once, transpose through LDS, 128-bit row stores.
  // Lane l of a 16x16 result tile holds column l%16 and rows 4*(l/16) + e, e = 0..3.
  // Each wave owns a [32*MI rows][64 cols] fp16 image (row pitch 144 B).  Neighbouring lanes swap one value
  // so that every lane writes a 32-bit pair; the image is then read back 16 bytes per lane, 8 lanes per row.
  if (tail_part >= 0) {  // part of a tail tile: raw fp32 sums into its own [TBM][256] image
    float* pz = g.tail_partial + (int64_t)tail_slot * (TBM * BN);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = wn * WN + j * 16 + frow;
#pragma unroll
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int row = wm * WM + i * 16 + 4 * fq + e;
          pz[row * BN + col] = acc[i][j][e];
        }
    }
    return;
  }
  if (g.partial) {  // split-K: raw fp32 partial sums, lanes of a half-wave write 128 contiguous bytes
    float* pz = g.partial + (int64_t)blockIdx.y * g.m * g.n;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t col = col0 + wn * WN + j * 16 + frow;
#pragma unroll
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int64_t row = row0 + wm * WM + i * 16 + 4 * fq + e;
          if (row < g.m) pz[row * g.n + col] = acc[i][j][e];
        }
    }
    return;
  }
  APS_WAIT_LGKM0();
  APS_BARRIER();  // the main-loop tiles are dead; the LDS is reused for the images
  char* img = lds + wave * kEpiWaveBytes;
  const bool odd = lane & 1;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = j * 16 + frow;  // column inside the wave's 64-column strip
    float bv = 0.f;
    if (g.bias) {
      const uint16_t bb = ((const uint16_t*)g.bias)[col0 + wn * WN + col];
      bv = BF16 ? __uint_as_float((uint32_t)bb << 16) : (float)__builtin_bit_cast(_Float16, bb);
    }
#pragma unroll
    for (int i = 0; i < RT; ++i) {
#pragma unroll
      for (int e = 0; e < 4; e += 2) {
        const float v0 = act(g.out, acc[i][j][e] + bv), v1 = act(g.out, acc[i][j][e + 1] + bv);
        const uint32_t h0 = BF16 ? f32_to_bf16_bits(v0) : f32_to_f16_bits(v0);
        const uint32_t h1 = BF16 ? f32_to_bf16_bits(v1) : f32_to_f16_bits(v1);
        // even lanes keep row e and receive the neighbour's row-e value; odd lanes keep row e+1
        const uint32_t send = odd ? h0 : h1;
        const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1, 0xf, 0xf, true);
        const uint32_t pair = odd ? (recv | (h1 << 16)) : (h0 | (recv << 16));
        const int row = i * 16 + 4 * fq + e + (odd ? 1 : 0);
        *(uint32_t*)(img + row * kEpiPitch + (col & ~1) * 2) = pair;
      }
    }
  }
  // same wave wrote and reads: only the LDS counter has to drain
  const int half = (g.out.n_split && col0 >= g.out.n_split) ? 1 : 0;  // a tile never straddles the split
  const int64_t ocol = col0 - (half ? g.out.n_split : 0) + wn * WN;
  const int rrow = lane >> 3, rchunk = lane & 7;
#pragma unroll 4
  for (int it = 0; it < WM / 8; ++it) {
    const int lr = it * 8 + rrow;
    const u32x4 v = *(const u32x4*)(img + lr * kEpiPitch + rchunk * 16);
    const int64_t row = row0 + wm * WM + lr;
    if (row >= g.m) continue;
    uint16_t* dst = out_row(g.out, row, half);
    if (!dst) continue;
    dst += ocol + rchunk * 8;
    if (g.out.aligned16)
      __builtin_nontemporal_store(v, (u32x4*)dst);   // 4 MB per XCD and round: as much as its L2 holds
    else {
      uint32_t* d = (uint32_t*)dst;
      d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
    }
  }
}

// ---------------------------------------------------------------- few rows (a decode step's projections)
// out[m, n] for m <= 16: the product is a stream of the weights.  One workgroup owns 16 weight rows;
// its 8 wavefronts split K, each feeding v_mfma_f32_16x16x32 with the 16 weight rows as the A operand
// (lane l: row l%16, k-chunk l/16 of 8 elements) and the <=16 activation rows as B (rows beyond m read
// as zero through the buffer bounds); the 8 partial 16x16 results are added in LDS in a fixed order.
// No workspace and no second launch.
// Weights are not loaded in operand order (a wave-wide load of 16 rows x 64 bytes streams at 4.4 TB/s on this
// part) but as 8 rows x 128 bytes (lane l: row l/8, 16-byte piece l%8; 5.9 TB/s): two such loads hold
// 16 rows x 64 k = two MFMA steps.  For the even step one DPP move puts pieces 0-3 of rows 8-15 (second
// load, lanes with l%8 < 4) over the lanes with l%8 >= 4 of the first load, and one ds_bpermute per dword
// then fetches (row, piece) for every lane from that single register; the odd step mirrors it.
// The activations are small and stay in L2; they are loaded in operand order.
constexpr int kSkWaves = 8, kSkU = 4;   // kSkU pairs of steps per register set

template <bool BF16>
__global__ __launch_bounds__(kSkWaves * 64) void skinny_nt_kernel(const GemmArgs g, int pairs_per_wave) {
  __shared__ float4v red[kSkWaves][64];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int64_t n0 = (int64_t)blockIdx.x * 16;
  const int64_t m0 = (int64_t)blockIdx.y * 16;  // 16 activation rows per workgroup row
  const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(g.w + n0 * g.ldw_b, (g.n - n0 - 1) * g.ldw_b + g.k * 2);
  const int64_t x_head_b = g.head_rows ? (n0 / g.head_rows) * g.x_head_stride_b : 0;
  const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(g.a + m0 * g.lda_b + x_head_b, (g.m - m0 - 1) * g.lda_b + g.k * 2);
  const int row = lane & 15, kg = lane >> 4;
  const uint32_t voff_w0 = (uint32_t)((lane >> 3) * g.ldw_b + (lane & 7) * 16);  // rows >= n: out of bounds, zero
  const uint32_t voff_w1 = voff_w0 + (uint32_t)(8 * g.ldw_b);
  const uint32_t voff_x = (uint32_t)(row * g.lda_b + kg * 16);                   // rows >= m: zero
  const int upper = row >> 3;
  const int src_even = (8 * (row & 7) + kg + 4 * upper) * 4;       // byte address of the source lane, even step
  const int src_odd = (8 * (row & 7) + kg + 4 * (1 - upper)) * 4;
  const int total_steps = (int)(g.k / 32);                         // k is a multiple of 32
  const int total_pairs = (total_steps + 1) / 2;                   // an odd last step: its pair reads zeros past k
  const int p_begin = wave * pairs_per_wave;
  const int p_end = min(total_pairs, p_begin + pairs_per_wave);
  float4v acc = {0.f, 0.f, 0.f, 0.f};
  struct Set { u32x4 w0[kSkU], w1[kSkU], x0[kSkU], x1[kSkU]; };
  Set sa, sb;
  // Loads are unconditional: pairs past the wavefront's range are clamped to its last pair and skipped in the
  // multiply (a branch around a load makes the compiler wait for everything outstanding).  The row limit of
  // the buffer descriptors cannot bound k, so the second step of an odd tail is zeroed by hand.
  auto load_block = [&](int q0, Set& t) {
#pragma unroll
    for (int u = 0; u < kSkU; ++u) {
      const uint32_t koff = (uint32_t)min(q0 + u, p_end - 1) * 128;
      t.w0[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, voff_w0, koff, 2));
      t.w1[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, voff_w1, koff, 2));
      t.x0[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, voff_x, koff, 0));
      t.x1[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, voff_x, koff + 64, 0));
    }
  };
  auto mac_block = [&](int q0, const Set& t) {
#pragma unroll
    for (int u = 0; u < kSkU; ++u) {
      if (q0 + u >= p_end) continue;   // uniform
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (j == 1 && 2 * (q0 + u) + 1 >= total_steps) continue;  // odd number of steps: no second half
        u32x4 wf;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int lo = (int)t.w0[u][d], hi = (int)t.w1[u][d];
          const int merged = j == 0 ? __builtin_amdgcn_update_dpp(lo, hi, 0x114 /* row_shr:4 */, 0xf, 0xa, false)
                                    : __builtin_amdgcn_update_dpp(lo, hi, 0x104 /* row_shl:4 */, 0xf, 0x5, false);
          wf[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(j == 0 ? src_even : src_odd, merged);
        }
        acc = mfma16<BF16>(wf, j == 0 ? t.x0[u] : t.x1[u], acc);
      }
    }
  };
  int q = p_begin;
  if (q < p_end) load_block(q, sa);
  while (q < p_end) {
    load_block(q + kSkU, sb);
    mac_block(q, sa);
    q += kSkU;
    if (q >= p_end) break;
    load_block(q + kSkU, sa);
    mac_block(q, sb);
    q += kSkU;
  }
  red[wave][lane] = acc;
  __syncthreads();
  if (wave != 0) return;
  float4v sum = red[0][lane];
#pragma unroll
  for (int w = 1; w < kSkWaves; ++w) {
    const float4v p = red[w][lane];
    sum[0] += p[0]; sum[1] += p[1]; sum[2] += p[2]; sum[3] += p[3];
  }
  // lane l holds out[token l%16][n0 + 4*(l/16) + i], i = 0..3
  const int64_t token = m0 + row;
  if (token >= g.m) return;
  const int64_t n = n0 + 4 * kg;
  const int half = (g.out.n_split && n >= g.out.n_split) ? 1 : 0;
  uint16_t* dst = out_row(g.out, token, half);
  if (!dst) return;
  dst += n - (half ? g.out.n_split : 0);
  uint16_t h[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float v = sum[i];
    if (g.bias) {
      const uint16_t bb = ((const uint16_t*)g.bias)[n + i];
      v += BF16 ? __uint_as_float((uint32_t)bb << 16) : (float)__builtin_bit_cast(_Float16, bb);
    }
    v = act(g.out, v);
    h[i] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
  }
  if (g.out.aligned16) {  // 8-byte store
    uint2 v2 = {(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
    *(uint2*)dst = v2;
  } else {
    dst[0] = h[0]; dst[1] = h[1]; dst[2] = h[2]; dst[3] = h[3];
  }
}

// ---------------------------------------------------------------- at most 8 rows: weights as a pure stream
// Every wavefront owns 2 whole weight rows and reads them as contiguous 1 KiB wave-wide loads (lane l:
// 8 elements at k = 512*j + 8*l), straight into registers: on this part a wave-wide load that covers
// 16 rows x 64 B streams at 4.4 TB/s, one that covers 1 KiB of a row at 7 TB/s.  The activations are tiny
// and shared: the workgroup stages them in LDS, 2048 elements of K at a time ([MT][2048], copied
// global -> LDS without a register round trip), from where a lane reads the 8 elements that match its
// weight chunk (consecutive lanes, consecutive 16 bytes).  v_dot2 with fp32 accumulation does the
// arithmetic (4*MT per weight load); the 64 partial sums of a row are added once, at the end.
// Chunk c+1 (weights into a second register set, activations into the other LDS buffer) is in flight
// while chunk c is multiplied; one barrier per chunk.
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
constexpr int kRsWaves = 8, kRsRows = 2, kRsKc = 2048, kRsJ = kRsKc / 512;

template <bool BF16>
__device__ __forceinline__ float dot8(const u32x4& a, const u32x4& b, float c) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t ai = a[i], bi = b[i];
    if constexpr (BF16)
      c = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, ai), __builtin_bit_cast(bf16x2, bi), c, false);
    else
      c = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, ai), __builtin_bit_cast(half2v, bi), c, false);
  }
  return c;
}

__device__ __forceinline__ float wave_total(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true));
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

template <bool BF16, int MT>
__global__ __launch_bounds__(kRsWaves * 64) void rowstream_nt_kernel(const GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) char xs[2][MT][kRsKc * 2];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int64_t n_first = ((int64_t)blockIdx.x * kRsWaves + wave) * kRsRows;
  const char* wrow = g.w + n_first * g.ldw_b + lane * 16;
  const int64_t x_head_b =
      g.head_rows ? (((int64_t)blockIdx.x * kRsWaves * kRsRows) / g.head_rows) * g.x_head_stride_b : 0;
  const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(g.a + x_head_b, (g.m - 1) * g.lda_b + g.k * 2);
  float acc[kRsRows][MT];
#pragma unroll
  for (int i = 0; i < kRsRows; ++i)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[i][m] = 0.f;
  const int nchunks = (int)((g.k + kRsKc - 1) / kRsKc);

  // 1 KiB pieces of the activation chunk (MT rows x kRsJ pieces) are spread over the wavefronts
  auto stage_x = [&](int c) {
    const int64_t k0 = (int64_t)c * kRsKc;
    const int kcur = (int)min((int64_t)kRsKc, g.k - k0);
#pragma unroll
    for (int p = 0; p < (MT * kRsJ + kRsWaves - 1) / kRsWaves; ++p) {
      const int piece = p * kRsWaves + wave;
      const int m = piece / kRsJ, q = piece % kRsJ;
      if (piece < MT * kRsJ && q * 512 < kcur)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (__attribute__((address_space(3))) void*)(&xs[c & 1][m][q * 1024]),
                                                 16, (uint32_t)(lane * 16), (uint32_t)(m * g.lda_b + (k0 + q * 512) * 2),
                                                 0, 0);
    }
  };
  auto load_w = [&](int c, u32x4(&wq)[kRsRows][kRsJ]) {
    const int64_t k0 = (int64_t)c * kRsKc;
    const int kcur = (int)min((int64_t)kRsKc, g.k - k0);
#pragma unroll
    for (int i = 0; i < kRsRows; ++i)
#pragma unroll
      for (int j = 0; j < kRsJ; ++j) {
        wq[i][j] = u32x4{0u, 0u, 0u, 0u};
        if (j * 512 + lane * 8 < kcur)
          wq[i][j] = __builtin_nontemporal_load((const u32x4*)(wrow + i * g.ldw_b + (k0 + j * 512) * 2));
      }
  };
  auto multiply = [&](int c, const u32x4(&wq)[kRsRows][kRsJ]) {
    const int kcur = (int)min((int64_t)kRsKc, g.k - (int64_t)c * kRsKc);
#pragma unroll
    for (int j = 0; j < kRsJ; ++j) {
      if (j * 512 + lane * 8 < kcur) {  // lanes past the end of K hold no weights and stale activations
        u32x4 xv[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) xv[m] = *(const u32x4*)(&xs[c & 1][m][j * 1024 + lane * 16]);
#pragma unroll
        for (int i = 0; i < kRsRows; ++i)
#pragma unroll
          for (int m = 0; m < MT; ++m) acc[i][m] = dot8<BF16>(wq[i][j], xv[m], acc[i][m]);
      }
    }
  };

  u32x4 wa[kRsRows][kRsJ], wb[kRsRows][kRsJ];
  stage_x(0);
  load_w(0, wa);
  for (int c = 0; c < nchunks; c += 2) {
    APS_WAIT_VM(0);  // chunk c has landed (activations in LDS, weights in registers)
    APS_BARRIER();   // ... for every wavefront, and the other LDS buffer is free
    if (c + 1 < nchunks) { stage_x(c + 1); load_w(c + 1, wb); }
    multiply(c, wa);
    if (c + 1 >= nchunks) break;
    APS_WAIT_VM(0);
    APS_BARRIER();
    if (c + 2 < nchunks) { stage_x(c + 2); load_w(c + 2, wa); }
    multiply(c + 1, wb);
  }
#pragma unroll
  for (int i = 0; i < kRsRows; ++i)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[i][m] = wave_total(acc[i][m]);
  // lane i*MT + m stores out[m][n_first + i]
#pragma unroll
  for (int i = 0; i < kRsRows; ++i)
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (lane != i * MT + m) continue;
      const int64_t n = n_first + i;
      const int half = (g.out.n_split && n >= g.out.n_split) ? 1 : 0;
      uint16_t* dst = out_row(g.out, m, half);
      if (!dst) continue;
      float v = acc[i][m];
      if (g.bias) {
        const uint16_t bb = ((const uint16_t*)g.bias)[n];
        v += BF16 ? __uint_as_float((uint32_t)bb << 16) : (float)__builtin_bit_cast(_Float16, bb);
      }
      v = act(g.out, v);
      dst[n - (half ? g.out.n_split : 0)] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
    }
}

template <bool BF16, int MT>
int launch_rowstream(const GemmArgs& g, hipStream_t s) {
  APS_LAUNCH((rowstream_nt_kernel<BF16, MT>), dim3((unsigned)(g.n / (kRsWaves * kRsRows))),
                     dim3(kRsWaves * 64), 0, s, g);
  return launch_status();
}

template <bool BF16>
int launch_rowstream_m(const GemmArgs& g, hipStream_t s) {
  switch (g.m) {
    case 1: return launch_rowstream<BF16, 1>(g, s);
    case 2: return launch_rowstream<BF16, 2>(g, s);
    case 3: return launch_rowstream<BF16, 3>(g, s);
    case 4: return launch_rowstream<BF16, 4>(g, s);
    case 5: return launch_rowstream<BF16, 5>(g, s);
    case 6: return launch_rowstream<BF16, 6>(g, s);
    case 7: return launch_rowstream<BF16, 7>(g, s);
    default: return launch_rowstream<BF16, 8>(g, s);
  }
}

// ---------------------------------------------------------------- 3 .. 48 rows: weight rows through the streaming core
// Workgroup = 128 weight rows (8 wavefronts x 16) x one part of K x up to 16*NHT activation rows.  The weight
// rows are the streamed operand (128-byte visits, 16 KiB in flight per wavefront), the activations the LDS image
// shared by all wavefronts, so neither LDS nor L2 carries more than the weights themselves (the dot-product
// kernel reads the activations from LDS once per weight row and slows down from 3 rows on).  n/128 row tiles
// do not fill the chip: K is split over blockIdx.y into parts of whole 512-element chunks, and the fp32
// partial tiles [part][m][n] are added by splitk_reduce_kernel.
constexpr int kWsMaxRows = 48;
constexpr int kHeadwiseMaxRows = 256;   // head-wise x (the value projection of the attention on hidden rows)

template <bool BF16, int NHT>
__global__ __launch_bounds__(kScThreads) void weight_stream_kernel(const GemmArgs g, int64_t k_per_part) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int rows_wg = g.rows_per_wg ? g.rows_per_wg : kScTokens;
  const bool streams = wave * 16 < rows_wg;   // a wavefront past the workgroup's rows reads row 0 (cache hits), stores nothing
  const int64_t n0 = (int64_t)blockIdx.x * rows_wg;
  const int64_t k0 = (int64_t)blockIdx.y * k_per_part;
  const int64_t klen = min(g.k - k0, k_per_part);
  const int64_t m0 = (int64_t)blockIdx.z * (16 * NHT);
  auto weight_row = [&](int64_t n) {  // rows past the matrix or the workgroup's share: row 0, never stored
    return g.w + ((n < g.n && streams) ? n : 0) * g.ldw_b + (lane & 7) * 16 + k0 * 2;
  };
  float4v acc[NHT];
  // (head-wise x: the 128 weight rows of a workgroup lie inside one head, whose x is the image)
  const int64_t head_off = g.head_rows ? (n0 / g.head_rows) * g.x_head_stride_b : 0;
  stream_rows_times_image<BF16, NHT>(weight_row(n0 + wave * 16 + (lane >> 3)),
                                     weight_row(n0 + wave * 16 + 8 + (lane >> 3)),
                                     g.a + head_off + m0 * g.lda_b + k0 * 2,
                                     g.lda_b, (int)min((int64_t)(16 * NHT), g.m - m0), klen, lds, acc);
  // lane (g4, c) holds activation rows m0 + 16*ht + 4*g4 + i and weight row n0 + 16*wave + c
  const int64_t n = streams ? n0 + wave * 16 + c : g.n;
  const bool own = g.partial && g.tile_counters;   // the last workgroup of a tile adds the parts
  if (n >= g.n && !own) return;
  if (g.partial && n < g.n) {
#pragma unroll
    for (int ht = 0; ht < NHT; ++ht)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t row = m0 + 16 * ht + 4 * g4 + i;
        if (row >= g.m) continue;
        float* dst = g.partial + ((int64_t)blockIdx.y * g.m + row) * g.n + n;
        if (own) coherent_store(dst, acc[ht][i]);   // read by another workgroup of this launch
        else *dst = acc[ht][i];
      }
  }
  if (g.partial) {
    if (!own) return;
    if (!last_arrival(g.tile_counters + blockIdx.z * gridDim.x + blockIdx.x, (int)gridDim.y, (int*)lds) || n >= g.n)
      return;
    // parts 0, 1, 2, ... added in that order (what splitk_reduce_kernel does), eight loads per value in flight
    const int parts = (int)gridDim.y;
    const int64_t plane = g.m * g.n;
    const float* pp[NHT][4];
#pragma unroll
    for (int ht = 0; ht < NHT; ++ht)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t row = min(m0 + 16 * ht + 4 * g4 + i, g.m - 1);   // rows past the end: a valid address, not stored
        pp[ht][i] = g.partial + row * g.n + n;
        acc[ht][i] = coherent_load(pp[ht][i]);
      }
    for (int z0 = 1; z0 < parts; z0 += 8) {
      float t[NHT][4][8];
#pragma unroll
      for (int ht = 0; ht < NHT; ++ht)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int zb = 0; zb < 8; ++zb)
            t[ht][i][zb] = coherent_load(pp[ht][i] + (int64_t)min(z0 + zb, parts - 1) * plane);
#pragma unroll
      for (int zb = 0; zb < 8; ++zb)
        if (z0 + zb < parts) {
#pragma unroll
          for (int ht = 0; ht < NHT; ++ht)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[ht][i] += t[ht][i][zb];
        }
    }
  }
  float b = 0.f;
  if (g.bias) b = load_16bit_as_f32<BF16>(g.bias, n);
  const int half = (g.out.n_split && n >= g.out.n_split) ? 1 : 0;
#pragma unroll
  for (int ht = 0; ht < NHT; ++ht)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t row = m0 + 16 * ht + 4 * g4 + i;
      if (row >= g.m) continue;
      {
        uint16_t* dst = out_row(g.out, row, half);
        if (!dst) continue;
        const float v = act(g.out, acc[ht][i] + b);
        dst[n - (half ? g.out.n_split : 0)] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
      }
    }
}

// Rows per workgroup and parts of K for the kernel above.  Measured (13B layer shapes, 3..48 rows): one round of
// long-lived workgroups beats more, shorter ones even when they could share a CU (n=5120, k=20480: 240 workgroups
// 38 us, 400 workgroups 50 us): a workgroup's first loads meet the full memory latency with nothing to overlap.
// A CU on its own streams ~34 GB/s and the chip ~6.9 TB/s, so a launch wants all 256 CUs; and a K split costs a
// cross-workgroup sum at its end (~3.8 us: store acknowledgement, counter, loads of the parts).  Hence the choice by
// a small cost model over (rows per workgroup in {128, 112, 96, 80, 64}, whole-chunk K parts) with at most one
// workgroup per CU: time of the longest part at min(34 GB/s, 6.9 TB/s / workgroups) plus the sum if K is split.
// 13B shapes at 9..16 rows: n=15360 (qkv) 240 workgroups of 64 rows, no split (was 120 x 2 parts); n=20480 (fc1)
// 214 workgroups of 96 rows (was 160 of 128: 96 CUs idle); n=5120, k=5120 46 x 5 parts of 112 rows; n=5120,
// k=20480 64 x 4 parts of 80 rows.  (3..8 rows with K up to 6144 go to weight_ksplit_kernel instead.)
struct WsPlan { int rows, parts; int64_t k_per_part; };
WsPlan weight_stream_plan(int64_t m, int64_t n, int64_t k, bool whole_tiles_only = false) {
  const int nht = m <= 16 ? 1 : (m <= 32 ? 2 : 3);
  const int64_t mt = (m + 16 * nht - 1) / (16 * nht);
  const int64_t chunks = (k + kScChunk - 1) / kScChunk;
  WsPlan best{kScTokens, 1, chunks * kScChunk};
  double best_t = 1e30;
  for (int rows = kScTokens; rows >= (whole_tiles_only ? kScTokens : 64); rows -= 16) {
    const int64_t tiles = ((n + rows - 1) / rows) * mt;
    for (int64_t per = chunks; per >= 1; --per) {
      const int64_t parts = (chunks + per - 1) / per;
      if (tiles * parts > kNumCus) break;
      const int64_t last = chunks - (parts - 1) * per;
      if (last * 2 < per) continue;  // a last part under half a part leaves its workgroups idle early
      const double wgs = (double)(tiles * parts);
      const double rate = 34e9 < 6.9e12 / wgs ? 34e9 : 6.9e12 / wgs;
      const double t = (double)rows * (double)per * kScChunk * 2 / rate + (parts > 1 ? 3.8e-6 : 0.0);
      if (t < best_t * 0.995) {  // (ties go to the larger workgroup: fewer idle wavefronts)
        best_t = t;
        best = WsPlan{rows, (int)parts, per * kScChunk};
      }
    }
  }
  return best;
}

template <bool BF16>
int launch_weight_stream(const GemmArgs& g, int parts, int64_t k_per_part, hipStream_t s) {
  const int nht = g.m <= 16 ? 1 : (g.m <= 32 ? 2 : 3);
  const int rows = g.rows_per_wg ? g.rows_per_wg : kScTokens;
  const dim3 grid((unsigned)((g.n + rows - 1) / rows), (unsigned)parts,
                  (unsigned)((g.m + 16 * nht - 1) / (16 * nht)));
  hipError_t e = hipSuccess;
#define APS_LAUNCH_WS(N)                                                                                          \
  do {                                                                                                            \
    e = allow_dynamic_lds((const void*)weight_stream_kernel<BF16, N>, scores_lds_bytes<N>(), 16 + (BF16 ? 3 : 0) + N - 1); \
    if (e == hipSuccess)                                                                                          \
      APS_LAUNCH((weight_stream_kernel<BF16, N>), grid, dim3(kScThreads), scores_lds_bytes<N>(), s, g,    \
                         k_per_part);                                                                             \
  } while (0)
  if (nht == 1) APS_LAUNCH_WS(1); else if (nht == 2) APS_LAUNCH_WS(2); else APS_LAUNCH_WS(3);
#undef APS_LAUNCH_WS
  if (e != hipSuccess) return (int)e;
  return launch_status();
}

// ---------------------------------------------------------------- 3 .. 8 rows, K up to 6144: K split inside the workgroup
// Workgroup = 16 weight rows; its 8 wavefronts take an eighth of K each (P pairs of wave-wide loads = 64 P elements)
// and add their partial products through LDS, in wavefront order.  Nothing crosses workgroups, so a launch has no
// sum at its end, and the unit of work is small (16 rows x K: 160 KB at K = 5120), so n / 16 workgroups spread
// over the CUs where n / 128 tiles x K parts left some idle.  The price: every workgroup needs the activations of
// its whole K at once - the image is all m rows, staged once (m x K x 2 bytes of LDS, read from L2) - which is why
// this is for few rows and one-digit thousands of K.  A wavefront requests its share of the image copies, then
// everything it streams (2 P loads of 1 KiB), waits for the copies alone, and multiplies as the rows arrive.
constexpr int kKsMaxRows = 8;
constexpr int ksplit_lds_bytes(int m, int pairs) { return m * pairs * 512 * 2 + kScWaves * kKsMaxRows * 16 * 4; }
#ifndef APS_KSPLIT
#define APS_KSPLIT 1
#endif

// ROWS = 16, or 8 (the second wave-wide load of every pair is left out and half of each MFMA multiplies zeros):
// twice the workgroups of half the size, for products whose n / 16 workgroups are too few to balance over the CUs.
template <bool BF16, int P, int ROWS>
__global__ __launch_bounds__(kScThreads) void weight_ksplit_kernel(const GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  constexpr int kRowPieces = 64 * P;   // 16-byte pieces of an image row: K / 8, K = 512 P
  constexpr int kRowBytes = kRowPieces * 16;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int g4 = lane >> 4, c = lane & 15;
  const int m = (int)g.m;
  const int64_t n0 = (int64_t)blockIdx.x * ROWS;
  // The image goes global -> LDS without passing through registers: one wave-wide copy fills 64 consecutive
  // 16-byte slots of a row, and the swizzle (slot s of row r holds piece s ^ (r & 15) of its group of 16) is applied
  // on the source side, every lane fetching the piece that belongs in its slot.  m x P copies, dealt over the
  // wavefronts; they are requested before the weight rows, so that waiting for them leaves the rows in flight.
  // (The copies are issued from assembly: the compiler, seeing a copy into LDS and a later LDS read, waits for
  // every load in flight before the first read, weight rows included; it cannot know which bytes the copy wrote.)
  const int64_t head_off = g.head_rows ? (n0 / g.head_rows) * g.x_head_stride_b : 0;
  const uint64_t xa = (uint64_t)(g.a + head_off);
  u32x4 rsrc;   // buffer descriptor over the m rows of x
  rsrc[0] = __builtin_amdgcn_readfirstlane((uint32_t)xa);
  rsrc[1] = __builtin_amdgcn_readfirstlane((uint32_t)(xa >> 32));
  rsrc[2] = __builtin_amdgcn_readfirstlane((uint32_t)((m - 1) * g.lda_b + g.k * 2));
  rsrc[3] = 0x00020000u;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
#pragma unroll
  for (int j = 0; j < P; ++j) {   // (8 rows x P copies / 8 wavefronts = P copies per wavefront at most)
    const int t = wave + j * kScWaves;
    const int r = t / P, jg = t % P;
    if (r < m) {
      const int slot = 64 * jg + lane;
      const int piece = (slot & ~15) | ((slot ^ r) & 15);
      asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                   :
                   : "s"(__builtin_amdgcn_readfirstlane(lds_base + (uint32_t)(r * kRowBytes + jg * 1024))),
                     "v"((uint32_t)(r * g.lda_b) + (uint32_t)(piece * 16)), "s"(rsrc)
                   : "memory");
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // this wavefront's weight rows: lane l = row l / 8 (and 8 + l / 8), 16-byte piece l % 8 of every 128 bytes
  const char* rowp0 = g.w + (n0 + (lane >> 3)) * g.ldw_b + (lane & 7) * 16 + (int64_t)wave * (P * 128);
  const char* rowp1 = rowp0 + 8 * g.ldw_b;
  constexpr int kLoads = ROWS == 16 ? 2 * P : P;
  u32x4 ring[2 * P];
#pragma unroll
  for (int u = 0; u < P; ++u) {
    ring[2 * u] = __builtin_nontemporal_load((const u32x4*)(rowp0 + u * 128));
    if constexpr (ROWS == 16) ring[2 * u + 1] = __builtin_nontemporal_load((const u32x4*)(rowp1 + u * 128));
    else ring[2 * u + 1] = u32x4{0u, 0u, 0u, 0u};
  }
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");   // the image copies of this wavefront have landed
  APS_BARRIER();
  __builtin_amdgcn_sched_barrier(0);   // (nothing that waits for a weight row moves in front of the barrier)

  const int upper = c >> 3;
  const int src_even = (8 * (c & 7) + g4 + 4 * upper) * 4;
  const int src_odd = (8 * (c & 7) + g4 + 4 * (1 - upper)) * 4;
  const char* qrow = lds + c * kRowBytes;
  float4v acc = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < 2 * P; ++st) {
    const int u = st >> 1;
    u32x4 bf;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int lo = (int)ring[2 * u][d], hi = (int)ring[2 * u + 1][d];
      const int merged = (st & 1) == 0 ? __builtin_amdgcn_update_dpp(lo, hi, 0x114 /* row_shr:4 */, 0xf, 0xa, false)
                                       : __builtin_amdgcn_update_dpp(lo, hi, 0x104 /* row_shl:4 */, 0xf, 0x5, false);
      bf[d] = (uint32_t)__builtin_amdgcn_ds_bpermute((st & 1) == 0 ? src_even : src_odd, merged);
    }
    const int ch = wave * (8 * P) + 4 * st + g4;   // piece of the image row: k = 8 ch .. 8 ch + 7
    u32x4 af = u32x4{0u, 0u, 0u, 0u};
    if (c < m) af = *(const u32x4*)(qrow + ((ch & ~15) | ((ch ^ c) & 15)) * 16);
    acc = mfma16<BF16>(af, bf, acc);
  }
  // lane (g4, c) holds image rows 4 g4 + i (rows 8..15 do not exist) x weight row n0 + c
  float* red = (float*)(lds + m * kRowBytes);
  if (g4 < 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) red[(wave * kKsMaxRows + 4 * g4 + i) * 16 + c] = acc[i];
  }
  __syncthreads();
  if (tid >= 16 * m || (tid & 15) >= ROWS) return;
  const int row = tid >> 4, col = tid & 15;
  float sum = red[row * 16 + col];
#pragma unroll
  for (int w = 1; w < kScWaves; ++w) sum += red[(w * kKsMaxRows + row) * 16 + col];
  const int64_t n = n0 + col;
  if (g.bias) sum += load_16bit_as_f32<BF16>(g.bias, n);
  const int half = (g.out.n_split && n >= g.out.n_split) ? 1 : 0;
  uint16_t* dst = out_row(g.out, row, half);
  if (!dst) return;
  const float v = act(g.out, sum);
  dst[n - (half ? g.out.n_split : 0)] = BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
}

inline bool ksplit_covers(int64_t m, int64_t n, int64_t k) {
  const int64_t pairs = k / 512;
  return m >= 3 && m <= kKsMaxRows && k % 512 == 0 && n % 16 == 0 &&
         (pairs == 4 || pairs == 8 || pairs == 10 || pairs == 12);
}

#ifndef APS_KS_ROWS8_BELOW
#define APS_KS_ROWS8_BELOW 512   // workgroups of 16 rows below which 8-row workgroups are launched instead
#endif
template <bool BF16>
int launch_weight_ksplit(const GemmArgs& g, hipStream_t s) {
  const int pairs = (int)(g.k / 512);
  const int lds_bytes = ksplit_lds_bytes((int)g.m, pairs), lds_max = ksplit_lds_bytes(kKsMaxRows, pairs);
  const bool rows8 = g.n / 16 < APS_KS_ROWS8_BELOW;
  const dim3 grid((unsigned)(g.n / (rows8 ? 8 : 16)));
  hipError_t e = hipSuccess;
#define APS_LAUNCH_KS_R(P_, SLOT, R_)                                                                                \
  do {                                                                                                               \
    e = allow_dynamic_lds((const void*)weight_ksplit_kernel<BF16, P_, R_>, lds_max,                                  \
                          24 + (BF16 ? 8 : 0) + 2 * SLOT + (R_ == 8 ? 1 : 0));                                       \
    if (e == hipSuccess)                                                                                             \
      APS_LAUNCH((weight_ksplit_kernel<BF16, P_, R_>), grid, dim3(kScThreads), lds_bytes, s, g);                     \
  } while (0)
#define APS_LAUNCH_KS(P_, SLOT) \
  if (rows8) APS_LAUNCH_KS_R(P_, SLOT, 8); else APS_LAUNCH_KS_R(P_, SLOT, 16)
  switch (pairs) {
    case 4: APS_LAUNCH_KS(4, 0); break;
    case 8: APS_LAUNCH_KS(8, 1); break;
    case 10: APS_LAUNCH_KS(10, 2); break;
    default: APS_LAUNCH_KS(12, 3); break;
  }
#undef APS_LAUNCH_KS
#undef APS_LAUNCH_KS_R
  if (e != hipSuccess) return (int)e;
  return launch_status();
}

// out[m][n] = sum_z partial[z][m][n] + bias[n], rounded once; 4 columns per thread
template <bool BF16>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, const void* bias,
                                                            const OutMap out, int64_t m, int64_t n, int splits) {
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (idx >= m * n) return;
  const int64_t row = idx / n, col = idx - row * n;
  // four partials at a time: independent loads in flight instead of one memory latency per split
  float4 s = *(const float4*)(partial + idx);
  const int64_t plane = m * n;
  int z = 1;
  for (; z + 3 < splits; z += 4) {
    const float4 p0 = *(const float4*)(partial + (int64_t)z * plane + idx);
    const float4 p1 = *(const float4*)(partial + (int64_t)(z + 1) * plane + idx);
    const float4 p2 = *(const float4*)(partial + (int64_t)(z + 2) * plane + idx);
    const float4 p3 = *(const float4*)(partial + (int64_t)(z + 3) * plane + idx);
    s.x += p0.x; s.y += p0.y; s.z += p0.z; s.w += p0.w;   // same order of additions as one at a time
    s.x += p1.x; s.y += p1.y; s.z += p1.z; s.w += p1.w;
    s.x += p2.x; s.y += p2.y; s.z += p2.z; s.w += p2.w;
    s.x += p3.x; s.y += p3.y; s.z += p3.z; s.w += p3.w;
  }
  for (; z < splits; ++z) {
    const float4 p = *(const float4*)(partial + (int64_t)z * plane + idx);
    s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
  }
  if (bias) {
    const uint16_t* b = (const uint16_t*)bias + col;
    auto cv = [](uint16_t v) { return BF16 ? __uint_as_float((uint32_t)v << 16) : (float)__builtin_bit_cast(_Float16, v); };
    s.x += cv(b[0]); s.y += cv(b[1]); s.z += cv(b[2]); s.w += cv(b[3]);
  }
  s.x = act(out, s.x); s.y = act(out, s.y); s.z = act(out, s.z); s.w = act(out, s.w);
  const int half = (out.n_split && col >= out.n_split) ? 1 : 0;
  uint16_t* o = out_row(out, row, half);
  if (!o) return;
  o += col - (half ? out.n_split : 0);
  if (BF16) { o[0] = f32_to_bf16_bits(s.x); o[1] = f32_to_bf16_bits(s.y); o[2] = f32_to_bf16_bits(s.z); o[3] = f32_to_bf16_bits(s.w); }
  else { o[0] = f32_to_f16_bits(s.x); o[1] = f32_to_f16_bits(s.y); o[2] = f32_to_f16_bits(s.z); o[3] = f32_to_f16_bits(s.w); }
}

// Tail tiles of a large product: out tile = sum of its parts + bias, rounded once.  One thread per 4 columns of a
// row of a tile; 64 workgroups of 256 threads per 256 x 256 tile.
template <bool BF16>
__global__ __launch_bounds__(256) void tail_reduce_kernel(const GemmArgs g) {
  const int tile = blockIdx.x >> 6;  // index among the tail tiles
  const int q = ((blockIdx.x & 63) << 8) + threadIdx.x;  // quad of the tile: row q / 64, columns 4 * (q % 64)
  const int r = q >> 6, c = (q & 63) << 2;
  int pid_m, pid_n;
  tile_coords(g.tail_from + tile, g.tiles_m, g.tiles_n, pid_m, pid_n);
  const int64_t row = (int64_t)pid_m * BM + r, col = (int64_t)pid_n * BN + c;
  if (row >= g.m) return;
  const float* p = g.tail_partial + (int64_t)tile * g.tail_ways * (BM * BN) + r * BN + c;
  float4 s = *(const float4*)p;
  for (int z = 1; z < g.tail_ways; ++z) {
    const float4 t = *(const float4*)(p + (int64_t)z * (BM * BN));
    s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
  }
  if (g.bias) {
    s.x += load_16bit_as_f32<BF16>(g.bias, col); s.y += load_16bit_as_f32<BF16>(g.bias, col + 1);
    s.z += load_16bit_as_f32<BF16>(g.bias, col + 2); s.w += load_16bit_as_f32<BF16>(g.bias, col + 3);
  }
  s.x = act(g.out, s.x); s.y = act(g.out, s.y); s.z = act(g.out, s.z); s.w = act(g.out, s.w);
  const int half = (g.out.n_split && col >= g.out.n_split) ? 1 : 0;
  uint16_t* o = out_row(g.out, row, half);
  if (!o) return;
  o += col - (half ? g.out.n_split : 0);
  const uint32_t lo = BF16 ? (f32_to_bf16_bits(s.x) | ((uint32_t)f32_to_bf16_bits(s.y) << 16))
                           : (f32_to_f16_bits(s.x) | ((uint32_t)f32_to_f16_bits(s.y) << 16));
  const uint32_t hi = BF16 ? (f32_to_bf16_bits(s.z) | ((uint32_t)f32_to_bf16_bits(s.w) << 16))
                           : (f32_to_f16_bits(s.z) | ((uint32_t)f32_to_f16_bits(s.w) << 16));
  ((uint32_t*)o)[0] = lo;   // rows and column offsets are at least 4-byte aligned (checked by the entry points)
  ((uint32_t*)o)[1] = hi;
}

// Tail split of a product of full-size tiles: when the tiles fill the compute units a whole number of times
// plus a remainder of at most half a round, the remaining tiles are cut along K into `ways` parts so that
// their parts fill one short round instead of leaving most compute units idle for a full one (4096 x 10240:
// 640 tiles on 256 compute units = 2.5 rounds run as 3; with the last 128 tiles cut in two, as 2.5).
struct TailPlan { int from, ways, kt; int64_t bytes; };
inline TailPlan plan_tail(int64_t tiles, int64_t nk) {
  TailPlan t{0, 1, 0, 0};
  const int64_t full = tiles / kNumCus * kNumCus, rest = tiles - full;
  if (full == 0 || rest == 0 || tiles >= ((int64_t)1 << 28)) return t;
  int ways = (int)(kNumCus / rest);
  if (ways > 4) ways = 4;
  while (ways > 1 && nk / ways < 8) --ways;
  if (ways < 2) return t;
  t.from = (int)full; t.ways = ways; t.kt = (int)((nk + ways - 1) / ways);
  t.bytes = rest * ways * (int64_t)(BM * BN) * 4;
  return t;
}

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

// Tile rows / 64 for m rows beyond the row-streaming kernels' range.  Up to 128 rows: the smallest tile that
// covers m.  Beyond: 192 or 256 rows, whichever needs less time by the count "rounds of workgroups over the
// CUs x rows per tile" (a tie goes to the 256-row tile, which is the one tuned for large products).  Measured
// on the 13B layer shapes this rule picks the faster of the two at every m from 160 to 4096; the 192-row tile
// wins most of that range because its rounds are shorter and rows past m cost it less matrix-core time.
static int tile_mi(int64_t m, int64_t n) {
  if (m <= 64) return 1;
  if (m <= 128) return 2;
  auto cost = [&](int mi) {
    const int64_t tiles = ((m + 64 * mi - 1) / (64 * mi)) * (n / BN);
    return ((tiles + kNumCus - 1) / kNumCus) * mi;
  };
  return cost(3) < cost(4) ? 3 : 4;
}

int aps_linear_nt_splits(int64_t m, int64_t n, int64_t k) {
  // Few tiles (a decode step's handful of tokens) cannot pull the weights at HBM speed with one workgroup
  // per tile: split K until about two waves of workgroups exist, keeping at least 4 k-tiles per split.
  if (m <= 0 || n <= 0 || k <= 0 || n % BN != 0 || k % BK != 0) return 1;
  if (m <= kRsMaxRows) return 1;  // streamed in one launch
  if (APS_KSPLIT && ksplit_covers(m, n, k)) return 1;   // K split inside the workgroups
  if (m <= kWsMaxRows) return weight_stream_plan(m, n, k).parts;
  const int64_t bm = 64 * tile_mi(m, n);
  const int64_t tiles = ((m + bm - 1) / bm) * (n / BN);
  const int64_t nk = k / BK;
  // as many splits as still give one workgroup per CU (a second, partly filled round costs more than it gains),
  // at least 4 k-tiles each
  int64_t s = kNumCus / tiles;
  if (s > 32) s = 32;
  while (s > 1 && nk / s < 4) --s;
  return (int)(s < 1 ? 1 : s);
}

// Tail plan of a product, or none: only full-size tiles without a uniform K split are cut.
static TailPlan tail_plan_of(int64_t m, int64_t n, int64_t k) {
  if (m <= kWsMaxRows || n <= 0 || k <= 0 || n % BN != 0 || k % BK != 0 || tile_mi(m, n) != 4 ||
      aps_linear_nt_splits(m, n, k) > 1)
    return TailPlan{0, 1, 0, 0};
  return plan_tail(((m + BM - 1) / BM) * (n / BN), k / BK);
}

int64_t aps_linear_nt_workspace_bytes(int64_t m, int64_t n, int64_t k) {
  const int s = aps_linear_nt_splits(m, n, k);
  if (s > 1) return (int64_t)s * m * n * 4;
  return tail_plan_of(m, n, k).bytes;
}

// Where the rows of a gathered A operand live (see GemmArgs::row_src).
struct GatherSrc {
  const int64_t* row_src;
  const void* slot_base; int64_t slot_stride, num_slots;
  const void* alt_base; int64_t alt_stride, alt_rows;
};

static int launch_gemm(const void* x, const void* weight, const void* bias, const OutMap& om, int64_t m, int64_t n,
                       int64_t k, int64_t x_stride, int64_t w_stride, int dtype, void* workspace,
                       int64_t workspace_bytes, aps_stream_t stream, const GatherSrc* gs = nullptr,
                       int32_t* tile_counters = nullptr) {
  if (dtype != APS_F16 && dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  if (n % BN != 0 || k % BK != 0) return APS_ERR_UNSUPPORTED;
  if (x_stride < k || w_stride < k) return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(x), addr(weight), (uint64_t)x_stride * 2, (uint64_t)w_stride * 2}) != 16)
    return APS_ERR_UNSUPPORTED;
  if (gs && common_vec_bytes({addr(gs->slot_base), addr(gs->alt_base), (uint64_t)gs->slot_stride * 2,
                              (uint64_t)gs->alt_stride * 2}) != 16)
    return APS_ERR_UNSUPPORTED;
  // one tile's rows must be addressable with 32-bit byte offsets
  if ((int64_t)BM * x_stride * 2 >= ((int64_t)1 << 31) || (int64_t)BN * w_stride * 2 >= ((int64_t)1 << 31))
    return APS_ERR_UNSUPPORTED;
  GemmArgs g{};
  g.a = (const char*)x; g.w = (const char*)weight; g.bias = bias;
  g.lda_b = x_stride * 2; g.ldw_b = w_stride * 2;
  g.m = m; g.n = n; g.k = k;
  const int mi = tile_mi(m, n);
  g.tiles_m = (int)((m + 64 * mi - 1) / (64 * mi)); g.tiles_n = (int)(n / BN);
  g.out = om;
  hipStream_t s = (hipStream_t)stream;
  if (gs) {   // only the tile kernel reads its A rows through a row map
    g.a = nullptr;
    g.row_src = gs->row_src;
    g.slot_base = (const char*)gs->slot_base; g.alt_base = (const char*)gs->alt_base;
    g.slot_stride_b = gs->slot_stride * 2; g.alt_stride_b = gs->alt_stride * 2;
    g.num_slots = gs->num_slots; g.alt_rows = gs->alt_rows;
  }
  if (!gs && m <= kRsMaxRows)
    return dtype == APS_BF16 ? launch_rowstream_m<true>(g, s) : launch_rowstream_m<false>(g, s);
  if (APS_KSPLIT && !gs && ksplit_covers(m, n, k))
    return dtype == APS_BF16 ? launch_weight_ksplit<true>(g, s) : launch_weight_ksplit<false>(g, s);
  if (!gs && m <= kWsMaxRows) {
    const WsPlan wp = weight_stream_plan(m, n, k);
    const int parts = wp.parts;
    const int64_t k_per_part = wp.k_per_part;
    if (parts == 1 || (workspace && workspace_bytes >= (int64_t)parts * m * n * 4 && !(addr(workspace) & 15))) {
      g.rows_per_wg = wp.rows;
      g.partial = parts > 1 ? (float*)workspace : nullptr;
      g.tile_counters = parts > 1 ? (int*)tile_counters : nullptr;   // (at most kNumCus tiles are split)
      int st = dtype == APS_BF16 ? launch_weight_stream<true>(g, parts, k_per_part, s)
                                 : launch_weight_stream<false>(g, parts, k_per_part, s);
      if (st != APS_OK || parts == 1 || g.tile_counters) return st;
      const int64_t quads = m * n / 4;
      const dim3 rgrid((unsigned)((quads + 255) / 256));
      if (dtype == APS_BF16)
        APS_LAUNCH(splitk_reduce_kernel<true>, rgrid, dim3(256), 0, s, (const float*)workspace, bias, om, m, n,
                           parts);
      else
        APS_LAUNCH(splitk_reduce_kernel<false>, rgrid, dim3(256), 0, s, (const float*)workspace, bias, om, m,
                           n, parts);
      return launch_status();
    }
    if (workspace) return APS_ERR_WORKSPACE;
    // no workspace: the single-launch kernels below
    if (m <= 8) return dtype == APS_BF16 ? launch_rowstream_m<true>(g, s) : launch_rowstream_m<false>(g, s);
  }
  if (!gs && m <= kSkinnyMaxRows && n / 16 < ((int64_t)1 << 31) && x_stride * 2 * 16 < ((int64_t)1 << 31) &&
      w_stride * 2 * 16 < ((int64_t)1 << 31)) {
    const int pairs = (int)((k / 32 + 1) / 2);
    const int per_wave = (pairs + kSkWaves - 1) / kSkWaves;
    const dim3 grid((unsigned)(n / 16));
    if (dtype == APS_BF16)
      APS_LAUNCH(skinny_nt_kernel<true>, grid, dim3(kSkWaves * 64), 0, s, g, per_wave);
    else
      APS_LAUNCH(skinny_nt_kernel<false>, grid, dim3(kSkWaves * 64), 0, s, g, per_wave);
    return launch_status();
  }
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  if (total >= ((int64_t)1 << 30)) return APS_ERR_UNSUPPORTED;
  const int64_t per_xcd = (total + kNumXcd - 1) / kNumXcd;
  int splits = 1;
  if (workspace && !(gs && m <= kWsMaxRows)) {   // (the split plan of few rows belongs to the streaming kernels)
    splits = aps_linear_nt_splits(m, n, k);
    if (splits > 1 && (workspace_bytes < (int64_t)splits * m * n * 4 || (addr(workspace) & 15))) return APS_ERR_WORKSPACE;
  }
  const int64_t nk_all = k / BK;
  g.partial = splits > 1 ? (float*)workspace : nullptr;
  g.kt_per_split = (int)((nk_all + splits - 1) / splits);
  if (splits > 1) splits = (int)((nk_all + g.kt_per_split - 1) / g.kt_per_split);  // no empty split
  dim3 grid((unsigned)(per_xcd * kNumXcd), (unsigned)splits);
  g.tail_ways = 1;
  if (workspace && splits == 1) {
    const TailPlan tp = tail_plan_of(m, n, k);
    if (tp.ways > 1) {
      if (workspace_bytes < tp.bytes || (addr(workspace) & 15)) return APS_ERR_WORKSPACE;
      g.tail_partial = (float*)workspace;
      g.tail_from = tp.from; g.tail_ways = tp.ways; g.tail_kt = tp.kt;
      const int64_t tail_items = (total - tp.from) * tp.ways;
      grid.x = (unsigned)((tp.from / kNumXcd + (tail_items + kNumXcd - 1) / kNumXcd) * kNumXcd);
    }
  }
  // more than 64 KiB of dynamic LDS has to be allowed per function (and per device)
  hipError_t e = hipSuccess;
#define APS_LAUNCH_TILE(B, M_)                                                                                     \
  do {                                                                                                            \
    if (gs) {                                                                                                     \
      e = allow_dynamic_lds((const void*)gemm_nt_kernel<B, M_, true>, TileShape<M_>::kLdsBytes,                   \
                            8 + (B ? 4 : 0) + M_ - 1);                                                            \
      if (e == hipSuccess)                                                                                        \
        APS_LAUNCH((gemm_nt_kernel<B, M_, true>), grid, dim3(kThreads), TileShape<M_>::kLdsBytes, s, g);          \
    } else {                                                                                                      \
      e = allow_dynamic_lds((const void*)gemm_nt_kernel<B, M_>, TileShape<M_>::kLdsBytes, (B ? 4 : 0) + M_ - 1);  \
      if (e == hipSuccess)                                                                                        \
        APS_LAUNCH((gemm_nt_kernel<B, M_>), grid, dim3(kThreads), TileShape<M_>::kLdsBytes, s, g);                \
    }                                                                                                             \
  } while (0)
#define APS_LAUNCH_TILE_MI(B)                                                                        \
  if (mi == 1) APS_LAUNCH_TILE(B, 1); else if (mi == 2) APS_LAUNCH_TILE(B, 2);                        \
  else if (mi == 3) APS_LAUNCH_TILE(B, 3); else APS_LAUNCH_TILE(B, 4)
  if (dtype == APS_BF16) { APS_LAUNCH_TILE_MI(true); } else { APS_LAUNCH_TILE_MI(false); }
#undef APS_LAUNCH_TILE_MI
#undef APS_LAUNCH_TILE
  if (e != hipSuccess) return (int)e;
  int st = launch_status();
  if (st == APS_OK && g.tail_ways > 1) {
    const dim3 tgrid((unsigned)((total - g.tail_from) * 64));
    if (dtype == APS_BF16) APS_LAUNCH(tail_reduce_kernel<true>, tgrid, dim3(256), 0, s, g);
    else APS_LAUNCH(tail_reduce_kernel<false>, tgrid, dim3(256), 0, s, g);
    return launch_status();
  }
  if (st != APS_OK || splits <= 1) return st;
  const int64_t quads = (m * n + 3) / 4;
  const dim3 rgrid((unsigned)((quads + 255) / 256));
  if (dtype == APS_BF16)
    APS_LAUNCH(splitk_reduce_kernel<true>, rgrid, dim3(256), 0, s, (const float*)workspace, bias, om, m, n,
                       splits);
  else
    APS_LAUNCH(splitk_reduce_kernel<false>, rgrid, dim3(256), 0, s, (const float*)workspace, bias, om, m, n,
                       splits);
  return launch_status();
}

}  // extern "C"

__attribute__((visibility("hidden"))) int64_t aps_internal_headwise_workspace_bytes(int64_t m, int64_t n, int64_t k,
                                                                                   int head_rows) {
  // (more rows than one image holds go over the grid's z: every 48 rows stream the weights again, from L2)
  if (m < 3 || m > kHeadwiseMaxRows || head_rows <= 0 || head_rows % kScTokens != 0 || n % kScTokens != 0 || k % BK != 0)
    return 0;
  if (APS_KSPLIT && ksplit_covers(m, n, k)) return 16;
  const int parts = weight_stream_plan(m, n, k, true).parts;
  return parts > 1 ? (int64_t)parts * m * n * 4 : 16;   // (a nonzero size says "this shape is covered")
}

// out[map[m]][n] = <weight[n], x[m] + (n / head_rows) * x_head_stride> + bias[n]: the value projection of the
// absorbed attention, where the rows of head h multiply that head's context vector.  Any m: at most 8 rows
// stream the weights through the dot kernel, more go through the MFMA kernel in tiles of 16 rows.
__attribute__((visibility("hidden"))) int aps_internal_headwise_linear(const void* x, const void* weight, const void* bias, void* out, int64_t m, int64_t n,
                                 int64_t k, int64_t x_stride, int64_t x_head_stride, int head_rows, int64_t w_stride,
                                 int64_t out_stride, const int64_t* out_row_map, int64_t out_rows, int dtype,
                                 void* workspace, int64_t workspace_bytes, int32_t* tile_counters, hipStream_t s) {
  if (m <= 0) return APS_OK;
  if (n % 16 != 0 || k % 64 != 0 || head_rows % 16 != 0) return APS_ERR_UNSUPPORTED;
  if (x_stride * 2 * 16 >= ((int64_t)1 << 31) || w_stride * 2 * 16 >= ((int64_t)1 << 31)) return APS_ERR_UNSUPPORTED;
  GemmArgs g{};
  g.a = (const char*)x; g.w = (const char*)weight; g.bias = bias;
  g.lda_b = x_stride * 2; g.ldw_b = w_stride * 2;
  g.m = m; g.n = n; g.k = k;
  g.out.base[0] = (char*)out; g.out.ld = out_stride; g.out.n_split = 0;
  g.out.map = out_row_map; g.out.limit0 = out_rows;
  g.out.aligned16 = common_vec_bytes({addr(out), (uint64_t)out_stride * 2}) == 16;
  g.x_head_stride_b = x_head_stride * 2; g.head_rows = head_rows;
  const bool vec16 = common_vec_bytes({addr(x), addr(weight), (uint64_t)x_stride * 2, (uint64_t)x_head_stride * 2,
                                       (uint64_t)w_stride * 2}) == 16;
  if (APS_KSPLIT && vec16 && ksplit_covers(m, n, k))   // (16 rows of a workgroup lie inside one head)
    return dtype == APS_BF16 ? launch_weight_ksplit<true>(g, s) : launch_weight_ksplit<false>(g, s);
  // 3..48 rows and heads of whole 128-row tiles: the weight rows through the streaming core, K split over
  // enough workgroups to fill the chip, the parts added by the last workgroup of each tile
  const int64_t need = aps_internal_headwise_workspace_bytes(m, n, k, head_rows);
  if (need > 0 && workspace && tile_counters && workspace_bytes >= need && !(addr(workspace) & 15) &&
      common_vec_bytes({addr(x), addr(weight), (uint64_t)x_stride * 2, (uint64_t)x_head_stride * 2,
                        (uint64_t)w_stride * 2}) == 16) {
    const WsPlan wp = weight_stream_plan(m, n, k, true);   // (a workgroup's 128 rows must lie inside one head)
    const int parts = wp.parts;
    g.partial = parts > 1 ? (float*)workspace : nullptr;
    g.tile_counters = parts > 1 ? (int*)tile_counters : nullptr;
    return dtype == APS_BF16 ? launch_weight_stream<true>(g, parts, wp.k_per_part, s)
                             : launch_weight_stream<false>(g, parts, wp.k_per_part, s);
  }
  if (m <= 8 && n % (kRsWaves * kRsRows) == 0)
    return dtype == APS_BF16 ? launch_rowstream_m<true>(g, s) : launch_rowstream_m<false>(g, s);
  const int pairs = (int)((k / 32 + 1) / 2);
  const int per_wave = (pairs + kSkWaves - 1) / kSkWaves;
  const dim3 grid((unsigned)(n / 16), (unsigned)((m + 15) / 16));
  if (dtype == APS_BF16)
    APS_LAUNCH(skinny_nt_kernel<true>, grid, dim3(kSkWaves * 64), 0, s, g, per_wave);
  else
    APS_LAUNCH(skinny_nt_kernel<false>, grid, dim3(kSkWaves * 64), 0, s, g, per_wave);
  return launch_status();
}

extern "C" {

int aps_linear_nt(const void* x, const void* weight, const void* bias, void* out, int64_t m, int64_t n, int64_t k,
                  int64_t x_stride, int64_t w_stride, int64_t out_stride, const int64_t* out_row_map,
                  int64_t out_rows, int dtype, int flags, void* workspace, int64_t workspace_bytes,
                  int32_t* tile_counters, aps_stream_t stream) {
  if (m < 0 || n <= 0 || k <= 0 || (flags & ~APS_LINEAR_RELU)) return APS_ERR_INVALID_ARG;
  if (m == 0) return APS_OK;
  if (!x || !weight || !out) return APS_ERR_INVALID_ARG;
  if (out_stride < n) return APS_ERR_INVALID_ARG;
  const int align = common_vec_bytes({addr(out), (uint64_t)out_stride * 2});
  if (align < 4) return APS_ERR_UNSUPPORTED;
  OutMap om{};
  om.base[0] = (char*)out; om.ld = out_stride; om.n_split = 0;
  om.map = out_row_map; om.limit0 = out_rows; om.aligned16 = align == 16;
  om.relu = (flags & APS_LINEAR_RELU) ? 1 : 0;
  if (addr(tile_counters) & 3) return APS_ERR_INVALID_ARG;
  return launch_gemm(x, weight, bias, om, m, n, k, x_stride, w_stride, dtype, workspace, workspace_bytes, stream,
                     nullptr, tile_counters);
}

int aps_kv_reproject_to_cache(const void* x, const void* w_kv, const void* b_kv, void* ws_k_cache, void* ws_v_cache,
                              void* k_cache, void* v_cache, const int64_t* kv_dest, int64_t m, int64_t hidden_size,
                              int64_t k, int64_t x_stride, int64_t w_stride, int64_t slot_stride, int64_t ws_slots,
                              int64_t cache_slots, int dtype, void* workspace, int64_t workspace_bytes,
                              aps_stream_t stream) {
  if (m < 0 || hidden_size <= 0 || k <= 0 || ws_slots < 0 || cache_slots < 0) return APS_ERR_INVALID_ARG;
  if (m == 0) return APS_OK;
  if (!x || !w_kv || !kv_dest) return APS_ERR_INVALID_ARG;
  if ((ws_slots && (!ws_k_cache || !ws_v_cache)) || (cache_slots && (!k_cache || !v_cache))) return APS_ERR_INVALID_ARG;
  if (slot_stride < hidden_size) return APS_ERR_INVALID_ARG;
  if (hidden_size % BN != 0) return APS_ERR_UNSUPPORTED;  // a column tile must not straddle the K | V boundary
  const int align = common_vec_bytes({addr(ws_k_cache), addr(ws_v_cache), addr(k_cache), addr(v_cache),
                                      (uint64_t)slot_stride * 2});
  if (align < 4) return APS_ERR_UNSUPPORTED;
  OutMap om{};
  om.base[0] = (char*)ws_k_cache; om.base[1] = (char*)ws_v_cache;
  om.base[2] = (char*)k_cache; om.base[3] = (char*)v_cache;
  om.ld = slot_stride; om.n_split = hidden_size; om.map = kv_dest;
  om.limit0 = ws_slots; om.limit1 = cache_slots; om.aligned16 = align == 16;
  return launch_gemm(x, w_kv, b_kv, om, m, 2 * hidden_size, k, x_stride, w_stride, dtype, workspace, workspace_bytes,
                     stream);
}

int aps_kv_reproject_gathered(const void* paged_cache, int64_t cache_slot_stride, int64_t num_cache_slots,
                              const void* hidden_states, int64_t hidden_stride, int64_t num_inputs,
                              const int64_t* holder_src, int64_t m, const void* w_kv, const void* b_kv,
                              void* ws_k_cache, void* ws_v_cache, void* k_cache, void* v_cache,
                              const int64_t* kv_dest, int64_t hidden_size, int64_t k, int64_t w_stride,
                              int64_t slot_stride, int64_t ws_slots, int64_t cache_slots, int dtype, void* workspace,
                              int64_t workspace_bytes, aps_stream_t stream) {
  if (m < 0 || hidden_size <= 0 || k <= 0 || ws_slots < 0 || cache_slots < 0 || num_cache_slots < 0 || num_inputs <= 0)
    return APS_ERR_INVALID_ARG;
  if (m == 0) return APS_OK;
  if (!paged_cache || !hidden_states || !holder_src || !w_kv || !kv_dest) return APS_ERR_INVALID_ARG;
  if ((ws_slots && (!ws_k_cache || !ws_v_cache)) || (cache_slots && (!k_cache || !v_cache))) return APS_ERR_INVALID_ARG;
  if (slot_stride < hidden_size || cache_slot_stride < k || hidden_stride < k) return APS_ERR_INVALID_ARG;
  if (hidden_size % BN != 0) return APS_ERR_UNSUPPORTED;
  const int align = common_vec_bytes({addr(ws_k_cache), addr(ws_v_cache), addr(k_cache), addr(v_cache),
                                      (uint64_t)slot_stride * 2});
  if (align < 4) return APS_ERR_UNSUPPORTED;
  OutMap om{};
  om.base[0] = (char*)ws_k_cache; om.base[1] = (char*)ws_v_cache;
  om.base[2] = (char*)k_cache; om.base[3] = (char*)v_cache;
  om.ld = slot_stride; om.n_split = hidden_size; om.map = kv_dest;
  om.limit0 = ws_slots; om.limit1 = cache_slots; om.aligned16 = align == 16;
  const GatherSrc gs{holder_src, paged_cache, cache_slot_stride, num_cache_slots, hidden_states, hidden_stride,
                     num_inputs};
  // the row pitch checks of the plain path are made on the two sources instead
  return launch_gemm(hidden_states, w_kv, b_kv, om, m, 2 * hidden_size, k, hidden_stride, w_stride, dtype, workspace,
                     workspace_bytes, stream, &gs);
}

}  // extern "C"
