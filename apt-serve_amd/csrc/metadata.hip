// GPU-side construction of the ragged-batch metadata of the hybrid cache.
//
// Input is one small per-sequence description (length, cache type, block
// tables); everything whose size grows with the number of cached tokens — slot
// mappings and the row-index vectors — is expanded on the device.  One launch,
// one workgroup per sequence: the workgroup first reduces the per-sequence row
// counts of all earlier sequences (its exclusive prefix, O(batch) reads that
// stay in L2), then its threads write the rows of its own sequence.
#include "aps_common.h"

namespace aps {
namespace {

constexpr int kThreads = 256;

struct Prefix {
  int64_t rows;         // "tot" rows of earlier sequences
  int64_t hidden_rows;  // rows of earlier hidden-cached sequences
  int64_t hidden_seqs;  // earlier hidden-cached sequences
  int64_t tokens;       // sum of seq_lens of earlier sequences
};

__device__ __forceinline__ int64_t wave_sum(int64_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

// Sums f(i) over i < upto for the four counters; result valid in every thread.
template <class F>
__device__ Prefix block_prefix(int upto, F f) {
  __shared__ int64_t part[4][kThreads / 64];
  Prefix p{0, 0, 0, 0};
  for (int i = threadIdx.x; i < upto; i += kThreads) {
    const Prefix c = f(i);
    p.rows += c.rows; p.hidden_rows += c.hidden_rows; p.hidden_seqs += c.hidden_seqs; p.tokens += c.tokens;
  }
  p.rows = wave_sum(p.rows); p.hidden_rows = wave_sum(p.hidden_rows);
  p.hidden_seqs = wave_sum(p.hidden_seqs); p.tokens = wave_sum(p.tokens);
  const int w = threadIdx.x / 64;
  if ((threadIdx.x & 63) == 0) {
    part[0][w] = p.rows; part[1][w] = p.hidden_rows; part[2][w] = p.hidden_seqs; part[3][w] = p.tokens;
  }
  __syncthreads();
  Prefix r{0, 0, 0, 0};
#pragma unroll
  for (int k = 0; k < kThreads / 64; ++k) {
    r.rows += part[0][k]; r.hidden_rows += part[1][k]; r.hidden_seqs += part[2][k]; r.tokens += part[3][k];
  }
  return r;
}

struct MetaArgs {
  const int32_t* seq_lens; const int32_t* context_lens; const int32_t* use_hidden;
  const int32_t* block_tables; const int32_t* block_tables_shared;
  int64_t table_stride, shared_stride;
  int table_width, shared_width, batch, block_size;
  int64_t* slot_mapping; int64_t* slot_mapping_shared;
  int64_t* hidden_cache_use_tot; int64_t* kv_cache_use_tot;
  int64_t* hidden_cache_use_input; int64_t* hidden_cache_store_tot;
  int64_t* hidden_holder_upd; int64_t* hidden_holder_pull; int64_t* holder_src; int64_t* kv_dest;
  uint8_t* token_is_hidden;
  int64_t* hidden_slots; int64_t* hidden_seq_start;
  int64_t* kv_cache_use_input; int64_t* new_token_slot; int32_t* kv_seq_lens;
  int32_t* block_tables_out; int64_t out_stride; int out_width;
  uint8_t* block_types_out;   // [batch][out_width], nullable: 1 in every column of a hidden-cached sequence
  int32_t* seq_start_loc; int32_t* query_start_loc; int32_t* context_lens_out; int64_t* input_positions;
  int64_t* totals;
  int64_t cap_rows, cap_hidden_rows, cap_hidden_seqs, cap_kv;
};

__device__ __forceinline__ int64_t slot_of(const int32_t* table, int width, int pos, int block_size) {
  const int bi = pos / block_size;
  if (table == nullptr || bi >= width) return -1;  // no table: padding slot
  return (int64_t)table[bi] * block_size + (pos - bi * block_size);
}

// Decode step: a hidden-cached sequence contributes seq_len rows, a K/V-cached one a single row.
__global__ __launch_bounds__(kThreads) void decode_metadata_kernel(const MetaArgs a) {
  const int b = blockIdx.x;
  const Prefix pre = block_prefix(b, [&](int i) {
    const int64_t L = a.seq_lens[i];
    const bool h = a.use_hidden[i] != 0;
    return Prefix{h ? L : 1, h ? L : 0, h ? 1 : 0, L};
  });
  const int L = a.seq_lens[b];
  const bool hid = a.use_hidden[b] != 0;
  const int32_t* bt = a.block_tables ? a.block_tables + (int64_t)b * a.table_stride : nullptr;
  const int32_t* bts = a.block_tables_shared ? a.block_tables_shared + (int64_t)b * a.shared_stride : nullptr;
  const int64_t row0 = pre.rows;

  if (hid) {
    const int64_t h0 = pre.hidden_rows;
    const int64_t pull0 = pre.hidden_rows - pre.hidden_seqs;  // earlier hidden sequences have L-1 pull rows each
    for (int j = threadIdx.x; j < L; j += kThreads) {
      if (row0 + j < a.cap_rows) {
        const int64_t slot = slot_of(bt, a.table_width, j, a.block_size);
        a.slot_mapping[row0 + j] = slot;
        // context rows come from their slot (padding: a value below every -(b+1)), the newest row from input b
        if (a.holder_src) a.holder_src[row0 + j] = (j == L - 1) ? -(int64_t)(b + 1) : (slot >= 0 ? slot : INT64_MIN);
      }
      const int64_t shared_slot = slot_of(bts, a.shared_width, j, a.block_size);
      if (a.kv_dest && row0 + j < a.cap_rows) a.kv_dest[row0 + j] = shared_slot >= 0 ? shared_slot : -1;
      if (h0 + j < a.cap_hidden_rows) {
        a.slot_mapping_shared[h0 + j] = shared_slot;
        a.hidden_cache_use_tot[h0 + j] = row0 + j;
        if (a.hidden_slots) a.hidden_slots[h0 + j] = slot_of(bt, a.table_width, j, a.block_size);
      }
      if (j < L - 1 && pull0 + j < a.cap_rows - a.batch) a.hidden_holder_pull[pull0 + j] = row0 + j;
    }
    if (threadIdx.x == 0 && L > 0) {
      a.hidden_holder_upd[b] = row0 + L - 1;
      if (pre.hidden_seqs < a.cap_hidden_seqs) {
        a.hidden_cache_use_input[pre.hidden_seqs] = b;
        a.hidden_cache_store_tot[pre.hidden_seqs] = row0 + L - 1;
        if (a.hidden_seq_start) {
          a.hidden_seq_start[pre.hidden_seqs] = h0;
          a.hidden_seq_start[pre.hidden_seqs + 1] = h0 + L;  // the next hidden sequence writes the same value
        }
      }
    }
  } else if (threadIdx.x == 0) {
    if (row0 < a.cap_rows) {
      const int64_t slot = L > 0 ? slot_of(bt, a.table_width, L - 1, a.block_size) : -1;
      a.slot_mapping[row0] = slot;
      if (a.holder_src) a.holder_src[row0] = -(int64_t)(b + 1);
      if (a.kv_dest) a.kv_dest[row0] = slot >= 0 ? -(slot + 2) : -1;
    }
    const int64_t kv_rank = b - pre.hidden_seqs;
    if (kv_rank < a.cap_kv) {
      a.kv_cache_use_tot[kv_rank] = row0;
      if (a.kv_cache_use_input) a.kv_cache_use_input[kv_rank] = b;
    }
    a.hidden_holder_upd[b] = row0;
  }

  // block table handed to attention: the shared table for hidden sequences, the private one otherwise
  const int32_t* src = hid ? bts : bt;
  const int src_w = hid ? a.shared_width : a.table_width;
  for (int w = threadIdx.x; w < a.out_width; w += kThreads) {
    a.block_tables_out[(int64_t)b * a.out_stride + w] = (src && w < src_w) ? src[w] : 0;
    if (a.block_types_out) a.block_types_out[(int64_t)b * a.out_width + w] = hid ? 1 : 0;
  }

  if (threadIdx.x == 0) {
    if (b == 0) { a.seq_start_loc[0] = 0; a.query_start_loc[0] = 0; }
    a.seq_start_loc[b + 1] = (int32_t)(pre.tokens + L);
    a.query_start_loc[b + 1] = b + 1;
    a.context_lens_out[b] = L - 1;
    a.input_positions[b] = L - 1;
    if (a.new_token_slot) a.new_token_slot[b] = L > 0 ? slot_of(bt, a.table_width, L - 1, a.block_size) : -1;
    if (a.kv_seq_lens) a.kv_seq_lens[b] = hid ? 0 : L;
    if (b == a.batch - 1 && a.totals) {
      a.totals[0] = pre.rows + (hid ? L : 1);
      a.totals[1] = pre.hidden_rows + (hid ? L : 0);
      a.totals[2] = pre.hidden_seqs + (hid ? 1 : 0);
      a.totals[3] = b + 1 - a.totals[2];
    }
  }
}

// Prompt step: the row space is the token space; every token of a hidden-cached
// prompt is a hidden row, every other token a K/V row.
__global__ __launch_bounds__(kThreads) void prefill_metadata_kernel(const MetaArgs a) {
  const int b = blockIdx.x;
  const Prefix pre = block_prefix(b, [&](int i) {
    const int64_t L = a.seq_lens[i];
    const int64_t q = L - (a.context_lens ? a.context_lens[i] : 0);
    const bool h = a.use_hidden[i] != 0;
    return Prefix{q, h ? q : 0, h ? 1 : 0, L};
  });
  const int L = a.seq_lens[b];
  const int ctx = a.context_lens ? a.context_lens[b] : 0;
  const int q = L - ctx;
  const bool hid = a.use_hidden[b] != 0;
  const int32_t* bt = a.block_tables ? a.block_tables + (int64_t)b * a.table_stride : nullptr;
  const int64_t tok0 = pre.rows;
  const int64_t h0 = pre.hidden_rows;
  const int64_t kv0 = pre.rows - pre.hidden_rows;
  for (int j = threadIdx.x; j < q; j += kThreads) {
    const int64_t tok = tok0 + j;
    if (tok < a.cap_rows) {
      a.slot_mapping[tok] = slot_of(bt, a.table_width, ctx + j, a.block_size);
      a.input_positions[tok] = ctx + j;
      if (a.token_is_hidden) a.token_is_hidden[tok] = hid ? 1 : 0;
    }
    if (hid) {
      if (h0 + j < a.cap_hidden_rows) a.hidden_cache_use_input[h0 + j] = tok;
    } else {
      if (kv0 + j < a.cap_kv) a.kv_cache_use_tot[kv0 + j] = tok;
    }
  }
  if (threadIdx.x == 0) {
    if (b == 0) { a.seq_start_loc[0] = 0; a.query_start_loc[0] = 0; }
    a.seq_start_loc[b + 1] = (int32_t)(pre.tokens + L);
    a.query_start_loc[b + 1] = (int32_t)(tok0 + q);
    a.context_lens_out[b] = ctx;
    if (b == a.batch - 1 && a.totals) {
      a.totals[0] = tok0 + q;
      a.totals[1] = h0 + (hid ? q : 0);
      a.totals[2] = pre.hidden_seqs + (hid ? 1 : 0);
      a.totals[3] = a.totals[0] - a.totals[1];
    }
  }
}

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

int aps_build_decode_metadata(const int32_t* seq_lens, const int32_t* use_hidden, const int32_t* block_tables,
                              int64_t table_stride, int64_t table_width, const int32_t* block_tables_shared,
                              int64_t shared_stride, int64_t shared_width, int64_t batch, int block_size,
                              int64_t* slot_mapping, int64_t* slot_mapping_shared, int64_t* hidden_cache_use_tot,
                              int64_t* kv_cache_use_tot, int64_t* hidden_cache_use_input,
                              int64_t* hidden_cache_store_tot, int64_t* hidden_holder_upd,
                              int64_t* hidden_holder_pull, int64_t* holder_src, int64_t* kv_dest,
                              int64_t* hidden_slots, int64_t* hidden_seq_start, int64_t* kv_cache_use_input,
                              int64_t* new_token_slot, int32_t* kv_seq_lens, int64_t cap_rows,
                              int64_t cap_hidden_rows,
                              int64_t cap_hidden_seqs, int64_t cap_kv_seqs, int32_t* block_tables_out,
                              int64_t out_stride, int64_t out_width, uint8_t* block_types_out,
                              int32_t* seq_start_loc,
                              int32_t* query_start_loc, int32_t* context_lens, int64_t* input_positions,
                              int64_t* totals, aps_stream_t stream) {
  if (batch < 0 || block_size <= 0 || table_width < 0 || shared_width < 0 || out_width < 0)
    return APS_ERR_INVALID_ARG;
  if (batch == 0) return APS_OK;
  if (batch > 0x7fffffff || table_width > 0x7fffffff || shared_width > 0x7fffffff) return APS_ERR_UNSUPPORTED;
  if (!seq_lens || !use_hidden || !hidden_holder_upd || !seq_start_loc || !query_start_loc || !context_lens ||
      !input_positions)
    return APS_ERR_INVALID_ARG;
  if ((cap_rows && !slot_mapping) || (cap_rows > batch && !hidden_holder_pull) ||
      (cap_hidden_rows && (!slot_mapping_shared || !hidden_cache_use_tot)) ||
      (cap_hidden_seqs && (!hidden_cache_use_input || !hidden_cache_store_tot)) ||
      (cap_kv_seqs && !kv_cache_use_tot) || (out_width && !block_tables_out))
    return APS_ERR_INVALID_ARG;
  if (cap_rows < batch) return APS_ERR_INVALID_ARG;
  MetaArgs a{};
  a.seq_lens = seq_lens; a.context_lens = nullptr; a.use_hidden = use_hidden;
  a.block_tables = table_width ? block_tables : nullptr;
  a.block_tables_shared = shared_width ? block_tables_shared : nullptr;
  a.table_stride = table_stride; a.shared_stride = shared_stride;
  a.table_width = (int)table_width; a.shared_width = (int)shared_width; a.batch = (int)batch;
  a.block_size = block_size;
  a.slot_mapping = slot_mapping; a.slot_mapping_shared = slot_mapping_shared;
  a.hidden_cache_use_tot = hidden_cache_use_tot; a.kv_cache_use_tot = kv_cache_use_tot;
  a.hidden_cache_use_input = hidden_cache_use_input; a.hidden_cache_store_tot = hidden_cache_store_tot;
  a.hidden_holder_upd = hidden_holder_upd; a.hidden_holder_pull = hidden_holder_pull; a.holder_src = holder_src; a.kv_dest = kv_dest;
  a.hidden_slots = hidden_slots; a.hidden_seq_start = hidden_seq_start;
  a.kv_cache_use_input = kv_cache_use_input; a.new_token_slot = new_token_slot; a.kv_seq_lens = kv_seq_lens;
  a.block_tables_out = block_tables_out; a.out_stride = out_stride; a.out_width = (int)out_width;
  a.block_types_out = out_width ? block_types_out : nullptr;
  a.seq_start_loc = seq_start_loc; a.query_start_loc = query_start_loc; a.context_lens_out = context_lens;
  a.input_positions = input_positions; a.totals = totals;
  a.cap_rows = cap_rows; a.cap_hidden_rows = cap_hidden_rows; a.cap_hidden_seqs = cap_hidden_seqs;
  a.cap_kv = cap_kv_seqs;
  APS_LAUNCH(decode_metadata_kernel, dim3((unsigned)batch), dim3(kThreads), 0, (hipStream_t)stream, a);
  return launch_status();
}

int aps_build_prefill_metadata(const int32_t* seq_lens, const int32_t* context_lens_in, const int32_t* use_hidden,
                               const int32_t* block_tables, int64_t table_stride, int64_t table_width,
                               int64_t batch, int block_size, int64_t* slot_mapping, int64_t* input_positions,
                               int64_t* hidden_cache_use_input, int64_t* kv_cache_use_tot,
                               uint8_t* token_is_hidden, int64_t cap_tokens,
                               int64_t cap_hidden_tokens, int64_t cap_kv_tokens, int32_t* seq_start_loc,
                               int32_t* query_start_loc, int32_t* context_lens, int64_t* totals,
                               aps_stream_t stream) {
  if (batch < 0 || block_size <= 0 || table_width < 0) return APS_ERR_INVALID_ARG;
  if (batch == 0) return APS_OK;
  if (batch > 0x7fffffff || table_width > 0x7fffffff) return APS_ERR_UNSUPPORTED;
  if (!seq_lens || !use_hidden || !seq_start_loc || !query_start_loc || !context_lens) return APS_ERR_INVALID_ARG;
  if ((cap_tokens && (!slot_mapping || !input_positions)) || (cap_hidden_tokens && !hidden_cache_use_input) ||
      (cap_kv_tokens && !kv_cache_use_tot))
    return APS_ERR_INVALID_ARG;
  MetaArgs a{};
  a.seq_lens = seq_lens; a.context_lens = context_lens_in; a.use_hidden = use_hidden;
  a.block_tables = table_width ? block_tables : nullptr;
  a.table_stride = table_stride; a.table_width = (int)table_width; a.batch = (int)batch; a.block_size = block_size;
  a.slot_mapping = slot_mapping; a.input_positions = input_positions;
  a.hidden_cache_use_input = hidden_cache_use_input; a.kv_cache_use_tot = kv_cache_use_tot;
  a.token_is_hidden = token_is_hidden;
  a.seq_start_loc = seq_start_loc; a.query_start_loc = query_start_loc; a.context_lens_out = context_lens;
  a.totals = totals;
  a.cap_rows = cap_tokens; a.cap_hidden_rows = cap_hidden_tokens; a.cap_kv = cap_kv_tokens;
  APS_LAUNCH(prefill_metadata_kernel, dim3((unsigned)batch), dim3(kThreads), 0, (hipStream_t)stream, a);
  return launch_status();
}

}  // extern "C"
