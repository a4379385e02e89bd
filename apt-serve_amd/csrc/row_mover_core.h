// Device side of the row movers: the kernel shape they share, and the operator that moves a decode step's rows
// (newest K/V rows, newest hidden rows, holder assembly).  A header because two translation units use it: the
// cache operators' launcher, and the launch that takes the step's stores in beside the query images.
#pragma once
#include "aps_common.h"

namespace aps {
namespace {

constexpr int kMaxThreads = 256;

struct RowDesc {
  const char* src;  // nullptr with dst != nullptr: fill the row with zeros
  char* dst;        // nullptr: skip the row
};

// A segment is one wave-wide access: 64 consecutive VB-byte chunks of one row.  A wavefront owns U consecutive
// segments (of one row, or of two when U does not divide the segments per row): it resolves the U row
// descriptors first (their index loads are independent and go out together), then issues its U loads, then its
// U stores.  With one chunk per thread a compute unit has at most 32 wavefronts x 1 KiB of loads in flight,
// which at this part's memory latency is about 3 TB/s of reads however many workgroups are queued; U chunks
// per thread put U times as much in flight for the same number of resident wavefronts.  Loads and stores stay
// fully coalesced (a 10 KiB row of OPT-13B is ten 1 KiB segments) and non-temporal.  grid.y splits the rows
// into groups small enough for 32-bit segment arithmetic.
// Measured on MI355X (OPT-13B rows, random fp16 data): operators with one index level run fastest with U = 1
// (292 us for the config-2 gather against 299 / 317 us with U = 2 / 4: the chain index -> data is short enough
// for the 32 resident wavefronts of a compute unit to hide), the ones with two dependent index levels with
// U = 2 (312 against 341 us).  Each operator names its U as kChunks.

// (the body takes its place in the grid as arguments, so that another launch can take the workgroups in)
template <int VB, int U, class Op>
__device__ __forceinline__ void row_mover_body(const Op& op, int64_t n_items, uint32_t segs_per_row,
                                               uint32_t row_bytes, uint32_t items_per_y, const uint32_t bx,
                                               const uint32_t by) {
  typedef typename VecOf<VB>::type vec_t;
  const uint32_t lane = threadIdx.x & 63u;
  // wave-uniform on purpose: the row of a segment, its index loads and its pointers are then scalar work
  const uint32_t wave = __builtin_amdgcn_readfirstlane(bx * (kMaxThreads / 64) + (threadIdx.x >> 6));
  uint32_t local_item = (wave * U) / segs_per_row;
  uint32_t seg = wave * U - local_item * segs_per_row;
  const int64_t item0 = (int64_t)by * items_per_y;
  RowDesc rd[U];
  uint32_t c[U];
#pragma unroll
  for (int j = 0; j < U; ++j) {
    c[j] = (seg * 64u + lane) * VB;
    const int64_t item = item0 + local_item;
    rd[j] = RowDesc{nullptr, nullptr};
    if (local_item < items_per_y && item < n_items) rd[j] = op(item);
    if (c[j] >= row_bytes) rd[j].dst = nullptr;
    if (++seg == segs_per_row) { seg = 0; ++local_item; }
  }
  vec_t v[U];
#pragma unroll
  for (int j = 0; j < U; ++j) {
    v[j] = vec_t{};
    if (rd[j].dst != nullptr && rd[j].src != nullptr) v[j] = load_vec_stream<VB>(rd[j].src + c[j]);
  }
#pragma unroll
  for (int j = 0; j < U; ++j)
    if (rd[j].dst != nullptr) store_vec_stream<VB>(rd[j].dst + c[j], v[j]);
}

template <int VB, int U, class Op>
__global__ __launch_bounds__(kMaxThreads) void row_mover(Op op, int64_t n_items, uint32_t segs_per_row,
                                                         uint32_t row_bytes, uint32_t items_per_y) {
  row_mover_body<VB, U, Op>(op, n_items, segs_per_row, row_bytes, items_per_y, blockIdx.x, blockIdx.y);
}

// slot -> (block, offset).  Block sizes are powers of two in practice: a shift instead of a 64-bit
// division per 16-byte chunk.
struct BlockSplit {
  int block_size, shift;  // shift < 0: not a power of two
  __host__ explicit BlockSplit(int bs) : block_size(bs), shift(-1) {
    for (int s = 0; s < 31; ++s)
      if ((1 << s) == bs) shift = s;
  }
  __device__ __forceinline__ void operator()(int64_t slot, int64_t& blk, int64_t& off) const {
    if (shift >= 0) {
      blk = slot >> shift;
      off = slot & (block_size - 1);
    } else {
      blk = slot / block_size;
      off = slot - blk * block_size;
    }
  }
};

// Holder assembly with the source of every row resolved beforehand:
// row_src[t] >= 0 is a cache slot, -(b+1) is row b of the layer input, anything
// below -num_inputs is a padding row (zero filled).  One dependent index load
// per chunk instead of two: 6.4 instead of 5.6 TB/s on MI355X for 10 KiB rows.
struct ResolvedGatherOp {
  static constexpr int kChunks = 1;
  char* holder; const char* hidden_states; char* cache;
  const int64_t* row_src; const int64_t* slot_mapping;
  const int64_t* use_input; const int64_t* store_tot;
  int64_t n_rows, n_store, n_inputs;
  int64_t holder_stride_b, hidden_stride_b, slot_stride_b, num_slots;
  int64_t n_map;  // entries of slot_mapping (= n_rows unless no holder is assembled)
  // items [0, n_store): the stores of the newest hidden rows (three dependent index loads: first, so that their
  // chains run under the bulk of the launch); items [n_store, n_store + n_rows): the holder rows
  __device__ RowDesc operator()(int64_t item) const {
    RowDesc r{nullptr, nullptr};
    if (item >= n_store) {
      const int64_t i = item - n_store;
      const int64_t s = row_src[i];
      r.dst = holder + i * holder_stride_b;
      if (s >= 0) {
        if (s < num_slots) r.src = cache + s * slot_stride_b;
      } else if (-(s + 1) < n_inputs) {
        r.src = hidden_states + (-(s + 1)) * hidden_stride_b;
      }
    } else {  // newest hidden row is also persisted
      const int64_t j = item;
      const int64_t b = use_input[j];
      const int64_t t = store_tot[j];
      if (b < 0 || b >= n_inputs || t < 0 || t >= n_map) return r;
      const int64_t slot = slot_mapping[t];
      if (slot < 0 || slot >= num_slots) return r;
      r.src = hidden_states + b * hidden_stride_b;
      r.dst = cache + slot * slot_stride_b;
    }
    return r;
  }
};

// The cache traffic of one decode layer as a single launch: the newest K and V rows of the K/V-cached sequences
// (items [0, 2*n_kv): item = 2*i + plane over kv_use_input), the stores of the newest hidden rows (the next n_store
// items) and the holder assembly of ResolvedGatherOp (the last n_rows items).  A K or V row has the width of a
// hidden row (heads * head_size), so all three kinds share one segment grid.  The few rows with the long index
// chains (two and three dependent index loads before the data) come first: wavefronts start in item order, so
// those chains run under the bulk of the launch instead of forming its tail (measured at 87 719 holder rows:
// with them last the 256 K/V rows and 128 stores, 0.2 % of the bytes, added 3 % to the launch).
struct DecodeStepOp {
  static constexpr int kChunks = 1;
  ResolvedGatherOp g;
  const char* key; const char* value; char* k_cache; char* v_cache;
  const int64_t* kv_use_input; const int64_t* new_token_slot;
  int64_t n_kv, key_stride_b, value_stride_b, block_stride_b, row_b, num_blocks;
  BlockSplit split;
  __device__ RowDesc operator()(int64_t i) const {
    if (i >= 2 * n_kv) return g(i - 2 * n_kv);
    RowDesc r{nullptr, nullptr};
    const int64_t b = kv_use_input[i >> 1];
    if (b < 0 || b >= g.n_inputs) return r;
    const int64_t slot = new_token_slot[b];
    if (slot < 0) return r;
    int64_t blk, in_blk;
    split(slot, blk, in_blk);
    if (blk >= num_blocks) return r;
    const int64_t off = blk * block_stride_b + in_blk * row_b;
    if (i & 1) { r.src = value + b * value_stride_b; r.dst = v_cache + off; }
    else       { r.src = key + b * key_stride_b;     r.dst = k_cache + off; }
    return r;
  }
};

// The cache traffic of a decode step, checked and planned but not launched (host side): the operator, the shape
// of its grid, and the width of the accesses its pointers allow.
constexpr uint32_t kStoreJobMagic = 0x4a535041u;
struct StoreJob {
  uint32_t magic;
  int vb;                 // bytes per lane and access (16: the launch another kernel can take in)
  int64_t n_items;        // 0: nothing to do
  int64_t row_bytes;
  DecodeStepOp op;
};

// Grid of a launch of n_items rows of row_bytes: segments per row, rows per grid row, grid.
struct MoverGrid { int64_t segs_per_row, items_per_y, grid_x, grid_y; };
inline MoverGrid mover_grid(int64_t n_items, int64_t row_bytes, int vb, int chunks) {
  MoverGrid m;
  m.segs_per_row = (row_bytes + 64 * vb - 1) / (64 * vb);
  m.items_per_y = ((int64_t)1 << 30) / (m.segs_per_row * 64);
  if (m.items_per_y > n_items) m.items_per_y = n_items;
  m.grid_y = (n_items + m.items_per_y - 1) / m.items_per_y;
  const int64_t waves = (m.items_per_y * m.segs_per_row + chunks - 1) / chunks;
  m.grid_x = (waves + kMaxThreads / 64 - 1) / (kMaxThreads / 64);
  return m;
}

}  // namespace
}  // namespace aps
