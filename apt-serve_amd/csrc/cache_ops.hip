// Row scatter / gather kernels of the hybrid cache for gfx950.
//
// Every operator here moves whole rows (a hidden vector, or the K or V vector
// of one token) between a dense tensor and slots of a paged cache.  They share
// one kernel shape, row_mover: a wavefront owns one 1 KiB segment of a row (or
// two), resolves the row descriptor (source pointer, destination pointer) once
// with scalar index loads and every lane moves its 16-byte chunk with one
// non-temporal 128-bit load and store.  A row of OPT-13B is 10 KiB = ten such
// segments, so loads and stores are fully coalesced.
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>

#include "aps_common.h"
#include "row_mover_core.h"

namespace aps {
namespace {

// ---------------------------------------------------------------- descriptors

struct HiddenToCacheOp {
  static constexpr int kChunks = 2;
  const char* hidden; char* cache;
  const int64_t* slot_mapping; const int64_t* src_idx; const int64_t* tgt_idx;
  int64_t hidden_stride_b, slot_stride_b, num_slots, num_hidden_rows, slot_mapping_len;
  __device__ RowDesc operator()(int64_t b) const {
    RowDesc r{nullptr, nullptr};
    const int64_t tok = src_idx[b];
    const int64_t ti = tgt_idx[b];
    if (tok < 0 || tok >= num_hidden_rows || ti < 0 || ti >= slot_mapping_len) return r;
    const int64_t slot = slot_mapping[ti];
    if (slot < 0 || slot >= num_slots) return r;
    r.src = hidden + tok * hidden_stride_b;
    r.dst = cache + slot * slot_stride_b;
    return r;
  }
};

struct CacheToHiddenOp {
  static constexpr int kChunks = 2;
  char* hidden; const char* cache;
  const int64_t* slot_mapping; const int64_t* dst_idx;
  int64_t hidden_stride_b, slot_stride_b, num_slots, num_hidden_rows, slot_mapping_len;
  __device__ RowDesc operator()(int64_t b) const {
    RowDesc r{nullptr, nullptr};
    const int64_t tok = dst_idx[b];
    if (tok < 0 || tok >= num_hidden_rows || tok >= slot_mapping_len) return r;
    const int64_t slot = slot_mapping[tok];
    if (slot < 0 || slot >= num_slots) return r;
    r.src = cache + slot * slot_stride_b;
    r.dst = hidden + tok * hidden_stride_b;
    return r;
  }
};

struct HybridDecodeGatherOp {
  static constexpr int kChunks = 2;
  char* holder; const char* hidden_states; char* cache;
  const int64_t* slot_mapping; const int64_t* upd; const int64_t* pull;
  const int64_t* use_input; const int64_t* store_tot;
  int64_t n_upd, n_pull, n_store;
  int64_t holder_stride_b, hidden_stride_b, slot_stride_b, num_slots, num_tot;
  __device__ RowDesc operator()(int64_t i) const {
    RowDesc r{nullptr, nullptr};
    if (i < n_upd) {  // newest row of every sequence comes from the layer input
      const int64_t t = upd[i];
      if (t < 0 || t >= num_tot) return r;
      r.src = hidden_states + i * hidden_stride_b;
      r.dst = holder + t * holder_stride_b;
    } else if (i < n_upd + n_pull) {  // context rows of hidden sequences come from the cache
      const int64_t t = pull[i - n_upd];
      if (t < 0 || t >= num_tot) return r;
      r.dst = holder + t * holder_stride_b;
      const int64_t slot = slot_mapping[t];
      if (slot >= 0 && slot < num_slots) r.src = cache + slot * slot_stride_b;  // else zero row
    } else {  // newest hidden row is also persisted
      const int64_t j = i - n_upd - n_pull;
      const int64_t b = use_input[j];
      const int64_t t = store_tot[j];
      if (b < 0 || b >= n_upd || t < 0 || t >= num_tot) return r;
      const int64_t slot = slot_mapping[t];
      if (slot < 0 || slot >= num_slots) return r;
      r.src = hidden_states + b * hidden_stride_b;
      r.dst = cache + slot * slot_stride_b;
    }
    return r;
  }
};

// item = 2*t + plane (0 = K, 1 = V)
struct KvScatterOp {
  static constexpr int kChunks = 1;
  const char* key; const char* value; char* k_cache; char* v_cache;
  const int64_t* slot_mapping; const int64_t* token_idx;
  int64_t num_tokens, key_stride_b, value_stride_b, block_stride_b, row_b, num_blocks;
  BlockSplit split;
  __device__ RowDesc operator()(int64_t item) const {
    RowDesc r{nullptr, nullptr};
    const int64_t t = item >> 1;
    const int64_t tok = token_idx ? token_idx[t] : t;
    if (tok < 0 || tok >= num_tokens) return r;
    const int64_t slot = slot_mapping[tok];
    if (slot < 0) return r;
    int64_t blk, in_blk;
    split(slot, blk, in_blk);
    if (blk >= num_blocks) return r;
    const int64_t off = blk * block_stride_b + in_blk * row_b;
    if (item & 1) { r.src = value + tok * value_stride_b; r.dst = v_cache + off; }
    else          { r.src = key + tok * key_stride_b;     r.dst = k_cache + off; }
    return r;
  }
};

// Write of one step's tokens by cache type: item = 2*t + plane.  A K/V token stores its K row (plane 0)
// and V row (plane 1) by block; a hidden token stores its hidden row (plane 0 only) at its slot of the
// flattened cache.  A null source pointer switches that kind of row off.
struct MixedTokenOp {
  static constexpr int kChunks = 1;
  const char* key; const char* value; const char* hidden;
  char* k_cache; char* v_cache; char* hidden_cache;
  const int64_t* slot_mapping; const uint8_t* is_hidden;
  int64_t key_stride_b, value_stride_b, hidden_stride_b, block_stride_b, row_b, num_blocks;
  int64_t hidden_slot_stride_b, num_hidden_slots;
  BlockSplit split;
  __device__ RowDesc operator()(int64_t item) const {
    RowDesc r{nullptr, nullptr};
    const int64_t t = item >> 1;
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return r;
    if (is_hidden && is_hidden[t]) {
      if ((item & 1) || !hidden || slot >= num_hidden_slots) return r;
      r.src = hidden + t * hidden_stride_b;
      r.dst = hidden_cache + slot * hidden_slot_stride_b;
      return r;
    }
    if (!key) return r;
    int64_t blk, in_blk;
    split(slot, blk, in_blk);
    if (blk >= num_blocks) return r;
    const int64_t off = blk * block_stride_b + in_blk * row_b;
    if (item & 1) { r.src = value + t * value_stride_b; r.dst = v_cache + off; }
    else          { r.src = key + t * key_stride_b;     r.dst = k_cache + off; }
    return r;
  }
};

// Copy of whole cache blocks inside the caches of all layers: item = (layer, pair, plane, token row).
// A K/V block (kind 0) is both planes of block id b < N; a hidden block (kind 1) is one plane slab, its id
// runs over the flattened 2N plane slabs (b < N: K plane of block b, b >= N: V plane of block b - N).
struct BlockCopyOp {
  static constexpr int kChunks = 1;
  const int64_t* layer_base;   // device array: base address of every layer's (2, N, BS, H, D) cache
  const int64_t* pairs;        // [n][2] (source, destination)
  const uint8_t* kinds;        // nullable: all K/V blocks
  int64_t n_pairs, num_blocks, plane_stride_b, block_stride_b, row_b;
  int rows_per_block;
  __device__ RowDesc operator()(int64_t item) const {
    RowDesc r{nullptr, nullptr};
    const int64_t row = item % rows_per_block;
    int64_t rest = item / rows_per_block;
    const int plane = (int)(rest & 1);
    rest >>= 1;
    const int64_t pair = rest % n_pairs, layer = rest / n_pairs;
    const int64_t src = pairs[2 * pair], dst = pairs[2 * pair + 1];
    const bool hidden = kinds && kinds[pair];
    char* base = (char*)layer_base[layer];
    int64_t so, dof;
    if (hidden) {
      if (plane) return r;  // a hidden block is a single slab
      if (src < 0 || dst < 0 || src >= 2 * num_blocks || dst >= 2 * num_blocks) return r;
      so = (src / num_blocks) * plane_stride_b + (src % num_blocks) * block_stride_b;
      dof = (dst / num_blocks) * plane_stride_b + (dst % num_blocks) * block_stride_b;
    } else {
      if (src < 0 || dst < 0 || src >= num_blocks || dst >= num_blocks) return r;
      so = plane * plane_stride_b + src * block_stride_b;
      dof = plane * plane_stride_b + dst * block_stride_b;
    }
    r.src = base + so + row * row_b;
    r.dst = base + dof + row * row_b;
    return r;
  }
};

// item = 2*blk + plane over the reference's grid of 2*nkv + nh blocks
struct MixedKvOp {
  static constexpr int kChunks = 2;
  const char* key; const char* value;
  char* k_cache; char* v_cache; char* sk_cache; char* sv_cache;
  const int64_t* slot_mapping; const int64_t* slot_mapping_shared;
  const int64_t* kv_use_tot; const int64_t* hidden_use_tot;
  int64_t n_kv, n_hidden, num_tot;
  int64_t key_stride_b, value_stride_b, block_stride_b, shared_block_stride_b, row_b;
  int64_t num_blocks, num_shared_blocks;
  BlockSplit split; unsigned flags;
  __device__ RowDesc operator()(int64_t item) const {
    RowDesc r{nullptr, nullptr};
    const int64_t blk = item >> 1;
    int64_t tok, slot;
    bool to_shared;
    if (blk < n_kv) {
      tok = kv_use_tot[blk];
      if (tok < 0 || tok >= num_tot) return r;
      slot = slot_mapping[tok];
      to_shared = false;
    } else if (blk < 2 * n_kv) {
      if (flags & APS_MIXED_SKIP_MIRROR) return r;
      tok = kv_use_tot[blk - n_kv];
      if (tok < 0 || tok >= num_tot) return r;
      slot = slot_mapping[tok];
      to_shared = true;
    } else {
      int64_t off = blk - 2 * n_kv;
      if ((flags & APS_MIXED_LITERAL_MODULO) && n_kv > 0) off = blk % (2 * n_kv);
      if (off >= n_hidden) return r;
      tok = hidden_use_tot[off];
      if (tok < 0 || tok >= num_tot) return r;
      slot = slot_mapping_shared[off];
      to_shared = true;
    }
    if (slot < 0) return r;
    int64_t b, in_blk;
    split(slot, b, in_blk);
    if (b >= (to_shared ? num_shared_blocks : num_blocks)) return r;
    const int64_t off_b = b * (to_shared ? shared_block_stride_b : block_stride_b) + in_blk * row_b;
    if (item & 1) { r.src = value + tok * value_stride_b; r.dst = (to_shared ? sv_cache : v_cache) + off_b; }
    else          { r.src = key + tok * key_stride_b;     r.dst = (to_shared ? sk_cache : k_cache) + off_b; }
    return r;
  }
};

template <int VB, class Op>
int launch_rows_vb(const Op& op, int64_t n_items, int64_t row_bytes, hipStream_t s) {
  constexpr int U = VB == 16 ? Op::kChunks : 1;
  const MoverGrid m = mover_grid(n_items, row_bytes, VB, U);
  if (m.grid_y > 65535) return APS_ERR_UNSUPPORTED;
  APS_LAUNCH((row_mover<VB, U, Op>), dim3((unsigned)m.grid_x, (unsigned)m.grid_y), dim3(kMaxThreads), 0, s, op,
                     n_items, (uint32_t)m.segs_per_row, (uint32_t)row_bytes, (uint32_t)m.items_per_y);
  return launch_status();
}

template <class Op>
int launch_rows(const Op& op, int64_t n_items, int64_t row_bytes, int vb, hipStream_t s) {
  if (n_items <= 0 || row_bytes <= 0) return APS_OK;
  // grid.y = ceil(n_items / floor(2^30 / chunks per row)) must stay below 65536
  if (row_bytes > (int64_t)1 << 24 || n_items >= (int64_t)1 << 31) return APS_ERR_UNSUPPORTED;
  switch (vb) {
    case 16: return launch_rows_vb<16>(op, n_items, row_bytes, s);
    case 8: return launch_rows_vb<8>(op, n_items, row_bytes, s);
    case 4: return launch_rows_vb<4>(op, n_items, row_bytes, s);
    case 2: return launch_rows_vb<2>(op, n_items, row_bytes, s);
    default: return launch_rows_vb<1>(op, n_items, row_bytes, s);
  }
}

inline bool valid_elem(int e) { return e == 1 || e == 2 || e == 4 || e == 8; }

// ------------------------------------------------------- fp8 quantising write

template <class T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<_Float16>(_Float16 v) { return (float)v; }
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
struct bf16_bits { uint16_t u; };
template <> __device__ __forceinline__ float to_f32<bf16_bits>(bf16_bits v) {
  return __uint_as_float((uint32_t)v.u << 16);
}

// code = e4m3fn(clamp(x / scale, +-448)), round to nearest even.  The clamp
// makes the result independent of the conversion instruction's overflow mode;
// NaN is kept NaN (fminf/fmaxf would drop it).
__device__ __forceinline__ float fp8_prepare(float x, float scale) {
  const float y = x / scale;
  const float c = fminf(fmaxf(y, -448.0f), 448.0f);
  return (y != y) ? y : c;
}

__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
  int w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return (uint32_t)w;
}

// One workgroup per (token, plane).  EPT elements per thread per step:
// 8 (128-bit load of f16/bf16, 64-bit store) when everything is aligned, else 1.
template <class InT, int EPT>
__global__ __launch_bounds__(kMaxThreads) void kv_scatter_fp8(
    const InT* __restrict__ key, const InT* __restrict__ value, uint8_t* __restrict__ k_cache,
    uint8_t* __restrict__ v_cache, const int64_t* __restrict__ slot_mapping,
    const int64_t* __restrict__ token_idx, const uint8_t* __restrict__ skip_mask, int64_t num_tokens,
    int64_t key_stride, int64_t value_stride, int64_t block_stride, int64_t num_blocks, int block_size,
    int row_elems, float k_scale, float v_scale) {
  const int64_t item = blockIdx.x;
  const int64_t t = item >> 1;
  const bool is_v = item & 1;
  const int64_t tok = token_idx ? token_idx[t] : t;
  if (tok < 0 || tok >= num_tokens) return;
  if (skip_mask && skip_mask[tok]) return;
  const int64_t slot = slot_mapping[tok];
  if (slot < 0) return;
  const int64_t blk = slot / block_size;
  if (blk >= num_blocks) return;
  const InT* src = is_v ? value + tok * value_stride : key + tok * key_stride;
  uint8_t* dst = (is_v ? v_cache : k_cache) + blk * block_stride + (slot - blk * block_size) * (int64_t)row_elems;
  const float scale = is_v ? v_scale : k_scale;
  if constexpr (EPT == 8) {
    for (int c = threadIdx.x * 8; c < row_elems; c += blockDim.x * 8) {
      InT in[8];
      if constexpr (sizeof(InT) == 2) {
        *reinterpret_cast<VecOf<16>::type*>(in) = *reinterpret_cast<const VecOf<16>::type*>(src + c);
      } else {
        *reinterpret_cast<VecOf<16>::type*>(in) = *reinterpret_cast<const VecOf<16>::type*>(src + c);
        *reinterpret_cast<VecOf<16>::type*>(in + 4) = *reinterpret_cast<const VecOf<16>::type*>(src + c + 4);
      }
      float f[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = fp8_prepare(to_f32<InT>(in[i]), scale);
      VecOf<8>::type out;
      out.x = pack4_e4m3(f[0], f[1], f[2], f[3]);
      out.y = pack4_e4m3(f[4], f[5], f[6], f[7]);
      *reinterpret_cast<VecOf<8>::type*>(dst + c) = out;
    }
  } else {
    for (int c = threadIdx.x; c < row_elems; c += blockDim.x) {
      const float f = fp8_prepare(to_f32<InT>(src[c]), scale);
      dst[c] = (uint8_t)(pack4_e4m3(f, 0.f, 0.f, 0.f) & 0xFFu);
    }
  }
}

template <class InT>
int launch_kv_scatter_fp8(const void* key, const void* value, void* k_cache, void* v_cache,
                          const int64_t* slot_mapping, const int64_t* token_idx, const uint8_t* skip_mask,
                          int64_t n, int64_t num_tokens, int64_t key_stride, int64_t value_stride,
                          int64_t block_stride, int64_t num_blocks, int block_size, int row_elems, float k_scale,
                          float v_scale, hipStream_t s) {
  const int in_b = (int)sizeof(InT);
  const bool aligned = row_elems % 8 == 0 &&
                       common_vec_bytes({addr(key), addr(value), (uint64_t)key_stride * in_b,
                                         (uint64_t)value_stride * in_b}) == 16 &&
                       common_vec_bytes({addr(k_cache), addr(v_cache), (uint64_t)block_stride}) >= 8;
  const int per = aligned ? 8 : 1;
  int threads = ((row_elems + per - 1) / per + 63) / 64 * 64;
  if (threads > kMaxThreads) threads = kMaxThreads;
  const dim3 grid((unsigned)(2 * n));
  if (aligned)
    APS_LAUNCH((kv_scatter_fp8<InT, 8>), grid, dim3(threads), 0, s, (const InT*)key, (const InT*)value,
                       (uint8_t*)k_cache, (uint8_t*)v_cache, slot_mapping, token_idx, skip_mask, num_tokens,
                       key_stride, value_stride, block_stride, num_blocks, block_size, row_elems, k_scale, v_scale);
  else
    APS_LAUNCH((kv_scatter_fp8<InT, 1>), grid, dim3(threads), 0, s, (const InT*)key, (const InT*)value,
                       (uint8_t*)k_cache, (uint8_t*)v_cache, slot_mapping, token_idx, skip_mask, num_tokens,
                       key_stride, value_stride, block_stride, num_blocks, block_size, row_elems, k_scale, v_scale);
  return launch_status();
}

int dispatch_kv_scatter_fp8(const void* key, const void* value, void* key_cache, void* value_cache,
                            const int64_t* slot_mapping, const int64_t* token_idx, const uint8_t* skip_mask,
                            int64_t n, int64_t num_tokens, int64_t key_stride, int64_t value_stride,
                            int64_t block_stride, int64_t num_blocks, int block_size, int64_t row, int in_dtype,
                            float k_scale, float v_scale, hipStream_t s) {
  if (!(k_scale > 0.f) || !(v_scale > 0.f) || row >= (int64_t)1 << 30) return APS_ERR_INVALID_ARG;
  switch (in_dtype) {
    case APS_F16:
      return launch_kv_scatter_fp8<_Float16>(key, value, key_cache, value_cache, slot_mapping, token_idx, skip_mask,
                                             n, num_tokens, key_stride, value_stride, block_stride, num_blocks,
                                             block_size, (int)row, k_scale, v_scale, s);
    case APS_BF16:
      return launch_kv_scatter_fp8<bf16_bits>(key, value, key_cache, value_cache, slot_mapping, token_idx,
                                              skip_mask, n, num_tokens, key_stride, value_stride, block_stride,
                                              num_blocks, block_size, (int)row, k_scale, v_scale, s);
    case APS_F32:
      return launch_kv_scatter_fp8<float>(key, value, key_cache, value_cache, slot_mapping, token_idx, skip_mask, n,
                                          num_tokens, key_stride, value_stride, block_stride, num_blocks,
                                          block_size, (int)row, k_scale, v_scale, s);
    default:
      return APS_ERR_UNSUPPORTED;
  }
}

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

int aps_abi_version(void) { return APS_ABI_VERSION; }

const char* aps_status_string(int status) {
  switch (status) {
    case APS_OK: return "ok";
    case APS_ERR_INVALID_ARG: return "invalid argument";
    case APS_ERR_UNSUPPORTED: return "unsupported shape or dtype";
    case APS_ERR_WORKSPACE: return "workspace too small";
    case APS_ERR_SCRATCH_LIMIT: return "problem needs more scratch than the library's static array holds";
    default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown status";
  }
}

int aps_hidden_to_cache(const void* hidden, void* paged_cache, const int64_t* slot_mapping, const int64_t* src_idx,
                        const int64_t* target_slot_idx, int64_t n, int64_t hidden_size, int64_t hidden_stride,
                        int64_t slot_stride, int64_t num_slots, int64_t num_hidden_rows, int64_t slot_mapping_len,
                        int elem_size, aps_stream_t stream) {
  if (n < 0 || hidden_size < 0 || !valid_elem(elem_size)) return APS_ERR_INVALID_ARG;
  if (n == 0 || hidden_size == 0) return APS_OK;
  if (!hidden || !paged_cache || !slot_mapping || !src_idx || !target_slot_idx) return APS_ERR_INVALID_ARG;
  if (hidden_stride < hidden_size || slot_stride < hidden_size) return APS_ERR_INVALID_ARG;
  const int64_t e = elem_size;
  HiddenToCacheOp op{(const char*)hidden, (char*)paged_cache, slot_mapping, src_idx, target_slot_idx,
                     hidden_stride * e, slot_stride * e, num_slots, num_hidden_rows, slot_mapping_len};
  const int vb = common_vec_bytes({addr(hidden), addr(paged_cache), (uint64_t)(hidden_stride * e),
                                   (uint64_t)(slot_stride * e), (uint64_t)(hidden_size * e)});
  return launch_rows(op, n, hidden_size * e, vb, (hipStream_t)stream);
}

int aps_cache_to_hidden(void* hidden, const void* paged_cache, const int64_t* slot_mapping, const int64_t* dst_idx,
                        int64_t n, int64_t hidden_size, int64_t hidden_stride, int64_t slot_stride,
                        int64_t num_slots, int64_t num_hidden_rows, int64_t slot_mapping_len, int elem_size,
                        aps_stream_t stream) {
  if (n < 0 || hidden_size < 0 || !valid_elem(elem_size)) return APS_ERR_INVALID_ARG;
  if (n == 0 || hidden_size == 0) return APS_OK;
  if (!hidden || !paged_cache || !slot_mapping || !dst_idx) return APS_ERR_INVALID_ARG;
  if (hidden_stride < hidden_size || slot_stride < hidden_size) return APS_ERR_INVALID_ARG;
  const int64_t e = elem_size;
  CacheToHiddenOp op{(char*)hidden, (const char*)paged_cache, slot_mapping, dst_idx,
                     hidden_stride * e, slot_stride * e, num_slots, num_hidden_rows, slot_mapping_len};
  const int vb = common_vec_bytes({addr(hidden), addr(paged_cache), (uint64_t)(hidden_stride * e),
                                   (uint64_t)(slot_stride * e), (uint64_t)(hidden_size * e)});
  return launch_rows(op, n, hidden_size * e, vb, (hipStream_t)stream);
}

int aps_hybrid_decode_gather(void* holder, const void* hidden_states, void* paged_cache,
                             const int64_t* slot_mapping, const int64_t* hidden_holder_upd, int64_t n_upd,
                             const int64_t* hidden_holder_pull, int64_t n_pull,
                             const int64_t* hidden_cache_use_input, const int64_t* hidden_cache_store_tot,
                             int64_t n_store, int64_t hidden_size, int64_t holder_stride, int64_t hidden_stride,
                             int64_t slot_stride, int64_t num_slots, int64_t num_tot_tokens, int elem_size,
                             aps_stream_t stream) {
  if (n_upd < 0 || n_pull < 0 || n_store < 0 || hidden_size < 0 || !valid_elem(elem_size))
    return APS_ERR_INVALID_ARG;
  const int64_t n = n_upd + n_pull + n_store;
  if (n == 0 || hidden_size == 0) return APS_OK;
  if (!holder || !hidden_states || !paged_cache || !slot_mapping) return APS_ERR_INVALID_ARG;
  if ((n_upd && !hidden_holder_upd) || (n_pull && !hidden_holder_pull) ||
      (n_store && (!hidden_cache_use_input || !hidden_cache_store_tot)))
    return APS_ERR_INVALID_ARG;
  if (holder_stride < hidden_size || hidden_stride < hidden_size || slot_stride < hidden_size)
    return APS_ERR_INVALID_ARG;
  const int64_t e = elem_size;
  HybridDecodeGatherOp op{(char*)holder, (const char*)hidden_states, (char*)paged_cache, slot_mapping,
                          hidden_holder_upd, hidden_holder_pull, hidden_cache_use_input, hidden_cache_store_tot,
                          n_upd, n_pull, n_store, holder_stride * e, hidden_stride * e, slot_stride * e,
                          num_slots, num_tot_tokens};
  const int vb = common_vec_bytes({addr(holder), addr(hidden_states), addr(paged_cache),
                                   (uint64_t)(holder_stride * e), (uint64_t)(hidden_stride * e),
                                   (uint64_t)(slot_stride * e), (uint64_t)(hidden_size * e)});
  return launch_rows(op, n, hidden_size * e, vb, (hipStream_t)stream);
}

int aps_gather_hidden_rows(void* holder, const void* hidden_states, void* paged_cache, const int64_t* holder_src,
                           int64_t n_rows, const int64_t* slot_mapping, const int64_t* hidden_cache_use_input,
                           const int64_t* hidden_cache_store_tot, int64_t n_store, int64_t num_inputs,
                           int64_t hidden_size, int64_t holder_stride, int64_t hidden_stride, int64_t slot_stride,
                           int64_t num_slots, int elem_size, aps_stream_t stream) {
  if (n_rows < 0 || n_store < 0 || num_inputs < 0 || hidden_size < 0 || !valid_elem(elem_size))
    return APS_ERR_INVALID_ARG;
  if (n_rows + n_store == 0 || hidden_size == 0) return APS_OK;
  if (!holder || !hidden_states || !paged_cache || (n_rows && !holder_src)) return APS_ERR_INVALID_ARG;
  if (n_store && (!slot_mapping || !hidden_cache_use_input || !hidden_cache_store_tot)) return APS_ERR_INVALID_ARG;
  if (holder_stride < hidden_size || hidden_stride < hidden_size || slot_stride < hidden_size)
    return APS_ERR_INVALID_ARG;
  const int64_t e = elem_size;
  ResolvedGatherOp op{(char*)holder, (const char*)hidden_states, (char*)paged_cache, holder_src, slot_mapping,
                      hidden_cache_use_input, hidden_cache_store_tot, n_rows, n_store, num_inputs,
                      holder_stride * e, hidden_stride * e, slot_stride * e, num_slots, n_rows};
  const int vb = common_vec_bytes({addr(holder), addr(hidden_states), addr(paged_cache),
                                   (uint64_t)(holder_stride * e), (uint64_t)(hidden_stride * e),
                                   (uint64_t)(slot_stride * e), (uint64_t)(hidden_size * e)});
  return launch_rows(op, n_rows + n_store, hidden_size * e, vb, (hipStream_t)stream);
}

// Checks a decode step's cache traffic and writes its plan to `job` (n_items == 0: nothing to do).
static int plan_store_job(void* job, void* holder, const void* hidden_states, void* paged_cache,
                          const int64_t* holder_src, int64_t n_rows, const int64_t* slot_mapping,
                          const int64_t* hidden_cache_use_input, const int64_t* hidden_cache_store_tot, int64_t n_store,
                          int64_t num_inputs, int64_t hidden_size, int64_t holder_stride, int64_t hidden_stride,
                          int64_t slot_stride, int64_t num_slots, const void* key, const void* value, void* key_cache,
                          void* value_cache, const int64_t* kv_cache_use_input, const int64_t* new_token_slot,
                          int64_t n_kv, int64_t key_stride, int64_t value_stride, int block_size, int64_t block_stride,
                          int64_t num_blocks, int elem_size) {
  const DecodeStepOp none{ResolvedGatherOp{}, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0, 0,
                          BlockSplit(1)};
  *(StoreJob*)job = StoreJob{kStoreJobMagic, 16, 0, 0, none};
  if (n_rows < 0 || n_store < 0 || n_kv < 0 || num_inputs < 0 || hidden_size < 0 || !valid_elem(elem_size))
    return APS_ERR_INVALID_ARG;
  if (n_rows + n_store + n_kv == 0 || hidden_size == 0) return APS_OK;
  if ((n_rows || n_store) && (!hidden_states || !paged_cache)) return APS_ERR_INVALID_ARG;
  if (n_rows && holder && !holder_src) return APS_ERR_INVALID_ARG;
  if (n_store && (!slot_mapping || !hidden_cache_use_input || !hidden_cache_store_tot)) return APS_ERR_INVALID_ARG;
  if ((n_rows || n_store) && (hidden_stride < hidden_size || slot_stride < hidden_size)) return APS_ERR_INVALID_ARG;
  if (n_rows && holder && holder_stride < hidden_size) return APS_ERR_INVALID_ARG;
  if (n_kv) {
    if (!key || !value || !key_cache || !value_cache || !kv_cache_use_input || !new_token_slot || block_size <= 0)
      return APS_ERR_INVALID_ARG;
    if (key_stride < hidden_size || value_stride < hidden_size || block_stride < hidden_size * block_size)
      return APS_ERR_INVALID_ARG;
  }
  const int64_t e = elem_size;
  const int64_t n_map = n_rows;   // slot_mapping always has n_rows entries; without a holder no row is gathered
  if (!holder) n_rows = 0;
  DecodeStepOp op{ResolvedGatherOp{(char*)holder, (const char*)hidden_states, (char*)paged_cache, holder_src,
                                   slot_mapping, hidden_cache_use_input, hidden_cache_store_tot, n_rows, n_store,
                                   num_inputs, holder_stride * e, hidden_stride * e, slot_stride * e, num_slots,
                                   n_map},
                  (const char*)key, (const char*)value, (char*)key_cache, (char*)value_cache, kv_cache_use_input,
                  new_token_slot, n_kv, key_stride * e, value_stride * e, block_stride * e, hidden_size * e,
                  num_blocks, BlockSplit(block_size > 0 ? block_size : 1)};
  uint64_t bits = (uint64_t)(hidden_size * e);
  if (n_rows || n_store)
    bits |= addr(hidden_states) | addr(paged_cache) | (uint64_t)(hidden_stride * e) | (uint64_t)(slot_stride * e);
  if (n_rows) bits |= addr(holder) | (uint64_t)(holder_stride * e);
  if (n_kv)
    bits |= addr(key) | addr(value) | addr(key_cache) | addr(value_cache) | (uint64_t)(key_stride * e) |
            (uint64_t)(value_stride * e) | (uint64_t)(block_stride * e);
  const int64_t n_items = n_rows + n_store + 2 * n_kv, row_bytes = hidden_size * e;
  // grid.y = ceil(n_items / floor(2^30 / chunks per row)) must stay below 65536
  if (row_bytes > (int64_t)1 << 24 || n_items >= (int64_t)1 << 31) return APS_ERR_UNSUPPORTED;
  *(StoreJob*)job = StoreJob{kStoreJobMagic, common_vec_bytes({bits}), n_items, row_bytes, op};
  return APS_OK;
}

static int launch_store_job(const StoreJob& job, hipStream_t s) {
  if (job.magic != kStoreJobMagic || job.n_items < 0) return APS_ERR_INVALID_ARG;
  return launch_rows(job.op, job.n_items, job.row_bytes, job.vb, s);
}

#define APS_STEP_STORE_ARGS                                                                                         \
  holder, hidden_states, paged_cache, holder_src, n_rows, slot_mapping, hidden_cache_use_input,                     \
      hidden_cache_store_tot, n_store, num_inputs, hidden_size, holder_stride, hidden_stride, slot_stride, num_slots, \
      key, value, key_cache, value_cache, kv_cache_use_input, new_token_slot, n_kv, key_stride, value_stride,       \
      block_size, block_stride, num_blocks, elem_size

int aps_decode_step_cache_ops(void* holder, const void* hidden_states, void* paged_cache, const int64_t* holder_src,
                              int64_t n_rows, const int64_t* slot_mapping, const int64_t* hidden_cache_use_input,
                              const int64_t* hidden_cache_store_tot, int64_t n_store, int64_t num_inputs,
                              int64_t hidden_size, int64_t holder_stride, int64_t hidden_stride, int64_t slot_stride,
                              int64_t num_slots, const void* key, const void* value, void* key_cache,
                              void* value_cache, const int64_t* kv_cache_use_input, const int64_t* new_token_slot,
                              int64_t n_kv, int64_t key_stride, int64_t value_stride, int block_size,
                              int64_t block_stride, int64_t num_blocks, int elem_size, aps_stream_t stream) {
  alignas(8) unsigned char job[sizeof(StoreJob)];
  const int st = plan_store_job(job, APS_STEP_STORE_ARGS);
  return st != APS_OK ? st : launch_store_job(*(const StoreJob*)job, (hipStream_t)stream);
}

int aps_decode_step_cache_ops_job(void* job, int64_t job_bytes, void* holder, const void* hidden_states,
                                  void* paged_cache, const int64_t* holder_src, int64_t n_rows,
                                  const int64_t* slot_mapping, const int64_t* hidden_cache_use_input,
                                  const int64_t* hidden_cache_store_tot, int64_t n_store, int64_t num_inputs,
                                  int64_t hidden_size, int64_t holder_stride, int64_t hidden_stride,
                                  int64_t slot_stride, int64_t num_slots, const void* key, const void* value,
                                  void* key_cache, void* value_cache, const int64_t* kv_cache_use_input,
                                  const int64_t* new_token_slot, int64_t n_kv, int64_t key_stride,
                                  int64_t value_stride, int block_size, int64_t block_stride, int64_t num_blocks,
                                  int elem_size) {
  static_assert(sizeof(StoreJob) <= APS_CACHE_JOB_BYTES, "a job fits the bytes the header promises");
  if (!job || job_bytes < (int64_t)sizeof(StoreJob) || (addr(job) & 7)) return APS_ERR_INVALID_ARG;
  return plan_store_job(job, APS_STEP_STORE_ARGS);
}
#undef APS_STEP_STORE_ARGS

int aps_cache_job_launch(const void* job, aps_stream_t stream) {
  if (!job || (addr(job) & 7)) return APS_ERR_INVALID_ARG;
  return launch_store_job(*(const StoreJob*)job, (hipStream_t)stream);
}

int aps_reshape_and_cache_flash(const void* key, const void* value, void* key_cache, void* value_cache,
                                const int64_t* slot_mapping, const int64_t* token_idx, int64_t n,
                                int64_t num_tokens, int num_heads, int head_size, int block_size,
                                int64_t key_stride, int64_t value_stride, int64_t block_stride,
                                int64_t num_blocks, int in_dtype, int cache_dtype, float k_scale, float v_scale,
                                aps_stream_t stream) {
  if (n < 0 || num_heads <= 0 || head_size <= 0 || block_size <= 0) return APS_ERR_INVALID_ARG;
  const int in_b = elem_bytes_of(in_dtype);
  if (in_b == 0 || in_dtype == APS_FP8_E4M3) return APS_ERR_INVALID_ARG;
  if (n == 0) return APS_OK;
  if (!key || !value || !key_cache || !value_cache || !slot_mapping) return APS_ERR_INVALID_ARG;
  const int64_t row = (int64_t)num_heads * head_size;
  if (key_stride < row || value_stride < row || block_stride < row * block_size) return APS_ERR_INVALID_ARG;
  if (2 * n >= (int64_t)1 << 31) return APS_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  if (cache_dtype == in_dtype) {
    const int64_t e = in_b;
    KvScatterOp op{(const char*)key, (const char*)value, (char*)key_cache, (char*)value_cache, slot_mapping,
                   token_idx, num_tokens, key_stride * e, value_stride * e, block_stride * e, row * e, num_blocks,
                   BlockSplit(block_size)};
    const int vb = common_vec_bytes({addr(key), addr(value), addr(key_cache), addr(value_cache),
                                     (uint64_t)(key_stride * e), (uint64_t)(value_stride * e),
                                     (uint64_t)(block_stride * e), (uint64_t)(row * e)});
    return launch_rows(op, 2 * n, row * e, vb, s);
  }
  if (cache_dtype != APS_FP8_E4M3) return APS_ERR_UNSUPPORTED;
  return dispatch_kv_scatter_fp8(key, value, key_cache, value_cache, slot_mapping, token_idx, nullptr, n,
                                 num_tokens, key_stride, value_stride, block_stride, num_blocks, block_size, row,
                                 in_dtype, k_scale, v_scale, s);
}

int aps_mixed_reshape_and_cache(const void* key, const void* value, const void* hidden, void* key_cache,
                                void* value_cache, void* hidden_cache, const int64_t* slot_mapping,
                                const uint8_t* is_hidden, int64_t num_tokens, int num_heads, int head_size,
                                int block_size, int64_t key_stride, int64_t value_stride, int64_t hidden_stride,
                                int64_t block_stride, int64_t num_blocks, int64_t hidden_slot_stride,
                                int64_t num_hidden_slots, int in_dtype, int cache_dtype, float k_scale,
                                float v_scale, aps_stream_t stream) {
  if (num_tokens < 0 || num_heads <= 0 || head_size <= 0 || block_size <= 0) return APS_ERR_INVALID_ARG;
  const int in_b = elem_bytes_of(in_dtype);
  if (in_b == 0 || in_dtype == APS_FP8_E4M3) return APS_ERR_INVALID_ARG;
  if (num_tokens == 0) return APS_OK;
  if (!slot_mapping) return APS_ERR_INVALID_ARG;
  const bool have_kv = key != nullptr, have_hidden = hidden != nullptr && is_hidden != nullptr;
  if (have_kv && (!value || !key_cache || !value_cache)) return APS_ERR_INVALID_ARG;
  if (hidden && !hidden_cache) return APS_ERR_INVALID_ARG;
  if (!have_kv && !have_hidden) return APS_OK;
  const int64_t row = (int64_t)num_heads * head_size;
  if (have_kv && (key_stride < row || value_stride < row || block_stride < row * block_size))
    return APS_ERR_INVALID_ARG;
  if (have_hidden && (hidden_stride < row || hidden_slot_stride < row)) return APS_ERR_INVALID_ARG;
  if (2 * num_tokens >= (int64_t)1 << 31) return APS_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  const int64_t e = in_b;
  const bool quantise = have_kv && cache_dtype != in_dtype;
  if (quantise && cache_dtype != APS_FP8_E4M3) return APS_ERR_UNSUPPORTED;
  // hidden rows (always in the activation dtype) and, unless they are quantised, K/V rows: one launch
  MixedTokenOp op{quantise ? nullptr : (const char*)key, (const char*)value, have_hidden ? (const char*)hidden : nullptr,
                  (char*)key_cache, (char*)value_cache, (char*)hidden_cache, slot_mapping, is_hidden,
                  key_stride * e, value_stride * e, hidden_stride * e, block_stride * e, row * e, num_blocks,
                  hidden_slot_stride * e, num_hidden_slots, BlockSplit(block_size)};
  if (op.key || op.hidden) {
    uint64_t bits = (uint64_t)(row * e);
    if (op.key)
      bits |= addr(key) | addr(value) | addr(key_cache) | addr(value_cache) | (uint64_t)(key_stride * e) |
              (uint64_t)(value_stride * e) | (uint64_t)(block_stride * e);
    if (op.hidden) bits |= addr(hidden) | addr(hidden_cache) | (uint64_t)(hidden_stride * e) | (uint64_t)(hidden_slot_stride * e);
    const int st = launch_rows(op, 2 * num_tokens, row * e, common_vec_bytes({bits}), s);
    if (st != APS_OK) return st;
  }
  if (!quantise) return APS_OK;
  return dispatch_kv_scatter_fp8(key, value, key_cache, value_cache, slot_mapping, nullptr, is_hidden, num_tokens,
                                 num_tokens, key_stride, value_stride, block_stride, num_blocks, block_size, row,
                                 in_dtype, k_scale, v_scale, s);
}

int aps_mixed_kv_to_cache(const void* key, const void* value, void* k_cache, void* v_cache, void* shared_k_cache,
                          void* shared_v_cache, const int64_t* slot_mapping, const int64_t* slot_mapping_shared,
                          const int64_t* kv_cache_use_tot, const int64_t* hidden_cache_use_tot, int64_t n_kv,
                          int64_t n_hidden, int64_t num_tot_tokens, int num_heads, int head_size, int block_size,
                          int64_t key_stride, int64_t value_stride, int64_t block_stride, int64_t num_blocks,
                          int64_t shared_block_stride, int64_t num_shared_blocks, int elem_size, unsigned flags,
                          aps_stream_t stream) {
  if (n_kv < 0 || n_hidden < 0 || num_heads <= 0 || head_size <= 0 || block_size <= 0 || !valid_elem(elem_size))
    return APS_ERR_INVALID_ARG;
  const int64_t blocks = 2 * n_kv + n_hidden;
  if (blocks == 0) return APS_OK;
  if (!key || !value || !shared_k_cache || !shared_v_cache) return APS_ERR_INVALID_ARG;
  if (n_kv && (!k_cache || !v_cache || !slot_mapping || !kv_cache_use_tot)) return APS_ERR_INVALID_ARG;
  if (n_hidden && (!slot_mapping_shared || !hidden_cache_use_tot)) return APS_ERR_INVALID_ARG;
  const int64_t row = (int64_t)num_heads * head_size;
  if (key_stride < row || value_stride < row || block_stride < row * block_size ||
      shared_block_stride < row * block_size)
    return APS_ERR_INVALID_ARG;
  const int64_t e = elem_size;
  MixedKvOp op{(const char*)key, (const char*)value, (char*)k_cache, (char*)v_cache, (char*)shared_k_cache,
               (char*)shared_v_cache, slot_mapping, slot_mapping_shared, kv_cache_use_tot, hidden_cache_use_tot,
               n_kv, n_hidden, num_tot_tokens, key_stride * e, value_stride * e, block_stride * e,
               shared_block_stride * e, row * e, num_blocks, num_shared_blocks, BlockSplit(block_size), flags};
  const int vb = common_vec_bytes({addr(key), addr(value), addr(k_cache), addr(v_cache), addr(shared_k_cache),
                                   addr(shared_v_cache), (uint64_t)(key_stride * e), (uint64_t)(value_stride * e),
                                   (uint64_t)(block_stride * e), (uint64_t)(shared_block_stride * e),
                                   (uint64_t)(row * e)});
  return launch_rows(op, 2 * blocks, row * e, vb, (hipStream_t)stream);
}

int aps_copy_cache_blocks(const int64_t* layer_caches, int64_t num_layers, const int64_t* pairs,
                          const uint8_t* kinds, int64_t n_pairs, int64_t num_blocks, int block_size,
                          int64_t row_elems, int elem_size, aps_stream_t stream) {
  if (num_layers < 0 || n_pairs < 0 || num_blocks <= 0 || block_size <= 0 || row_elems <= 0 || !valid_elem(elem_size))
    return APS_ERR_INVALID_ARG;
  if (num_layers == 0 || n_pairs == 0) return APS_OK;
  if (!layer_caches || !pairs) return APS_ERR_INVALID_ARG;
  const int64_t row_b = row_elems * elem_size;
  BlockCopyOp op{layer_caches, pairs, kinds, n_pairs, num_blocks, num_blocks * block_size * row_b,
                 block_size * row_b, row_b, block_size};
  const int64_t items = num_layers * n_pairs * 2 * block_size;
  // layer bases come from the device array: only the row size can be checked here
  return launch_rows(op, items, row_b, common_vec_bytes({(uint64_t)row_b}), (hipStream_t)stream);
}

int aps_swap_cache_blocks(const void* src_cache, void* dst_cache, const int64_t* pairs_host,
                          const uint8_t* kinds_host, int64_t n_pairs, int64_t src_num_blocks,
                          int64_t dst_num_blocks, int64_t block_bytes, aps_stream_t stream) {
  if (n_pairs < 0 || src_num_blocks <= 0 || dst_num_blocks <= 0 || block_bytes <= 0) return APS_ERR_INVALID_ARG;
  if (n_pairs == 0) return APS_OK;
  if (!src_cache || !dst_cache || !pairs_host) return APS_ERR_INVALID_ARG;
  const char* s = (const char*)src_cache;
  char* d = (char*)dst_cache;
  for (int64_t i = 0; i < n_pairs; ++i) {
    const int64_t a = pairs_host[2 * i], b = pairs_host[2 * i + 1];
    const bool hidden = kinds_host && kinds_host[i];
    if (a < 0 || b < 0) continue;
    if (hidden) {
      if (a >= 2 * src_num_blocks || b >= 2 * dst_num_blocks) return APS_ERR_INVALID_ARG;
      const hipError_t e = hipMemcpyAsync(d + ((b / dst_num_blocks) * dst_num_blocks + b % dst_num_blocks) * block_bytes,
                                          s + ((a / src_num_blocks) * src_num_blocks + a % src_num_blocks) * block_bytes,
                                          block_bytes, hipMemcpyDefault, (hipStream_t)stream);
      if (e != hipSuccess) return (int)e;
    } else {
      if (a >= src_num_blocks || b >= dst_num_blocks) return APS_ERR_INVALID_ARG;
      for (int plane = 0; plane < 2; ++plane) {
        const hipError_t e = hipMemcpyAsync(d + (plane * dst_num_blocks + b) * block_bytes,
                                            s + (plane * src_num_blocks + a) * block_bytes, block_bytes,
                                            hipMemcpyDefault, (hipStream_t)stream);
        if (e != hipSuccess) return (int)e;
      }
    }
  }
  return APS_OK;
}

}  // extern "C"
