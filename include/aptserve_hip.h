/*
 * aptserve_hip.h — C ABI of the MI355X (gfx950) hybrid-cache library.
 *
 * One shared library, libaptserve_hip.so, exports every function below with C
 * linkage.  All pointers are device pointers unless a parameter says "host".
 * All tensors are owned by the caller; the library never allocates, frees or
 * retains device memory and keeps no global state, so calls are re-entrant
 * (one exception, documented there: aps_paged_decode_attention_static).
 * Work is enqueued on the given stream and the call returns without waiting.
 *
 * Return value: 0 on success; a negative aps_status on an argument error
 * (nothing was launched); a positive value is a hipError_t reported by the
 * launch.  Zero-row calls are a no-op that returns 0.
 *
 * Strides are in ELEMENTS of the tensor's dtype unless the name ends in
 * "_bytes".  "ref:" comments cite the reference interface an entry point
 * replaces, relative to additional_designs/ in eddiegaoo/Apt-Serve.
 */
#ifndef APTSERVE_HIP_H
#define APTSERVE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define APS_ABI_VERSION 10

typedef void* aps_stream_t; /* a hipStream_t; NULL = the null stream */

enum aps_status {
  APS_OK = 0,
  APS_ERR_INVALID_ARG = -1, /* null pointer, negative size, bad enum */
  APS_ERR_UNSUPPORTED = -2, /* shape / dtype combination not built */
  APS_ERR_WORKSPACE = -3,    /* workspace too small */
  APS_ERR_SCRATCH_LIMIT = -4 /* aps_paged_decode_attention_static: the problem
                                needs more than APS_STATIC_SCRATCH_BYTES */
};

enum aps_dtype {
  APS_F16 = 0,
  APS_BF16 = 1,
  APS_F32 = 2,
  APS_F64 = 3,
  APS_FP8_E4M3 = 4 /* OCP e4m3fn codes stored as bytes */
};

/* flags of aps_mixed_kv_to_cache */
#define APS_MIXED_LITERAL_MODULO 1u /* reproduce `blk % (2*nkv)` of mixed_cache.cu:88 */
#define APS_MIXED_SKIP_MIRROR 2u    /* do not write range B (the shared mirror) */

/* aps_linear_nt flags */
#define APS_LINEAR_RELU 1 /* store max(result, 0): fc1 with its activation */

int aps_abi_version(void);
const char* aps_status_string(int status);

/* ------------------------------------------------------------------------
 * Row scatter / gather between a dense [rows, width] tensor and the slots of
 * a paged cache.  A "slot" s starts s*slot_stride elements after the cache
 * base; num_slots bounds the slot ids (ids outside [0, num_slots) are
 * skipped, like the negative padding id).  Pure byte moves: any elem_size in
 * {1,2,4,8} (fp8 codes, f16/bf16, f32, f64).
 * ------------------------------------------------------------------------ */

/* ref: mixed_cache_kernels/mixed_cache.cu:119-147 (hidden_to_cache) and
 * :31-53 (kernel).  For b in [0,n): cache[slot_mapping[target_slot_idx[b]]]
 * = hidden[src_idx[b], 0:hidden_size].  Rows whose indices fall outside
 * [0,num_hidden_rows) / [0,slot_mapping_len) are skipped. */
int aps_hidden_to_cache(const void* hidden, void* paged_cache,
                        const int64_t* slot_mapping, const int64_t* src_idx,
                        const int64_t* target_slot_idx, int64_t n,
                        int64_t hidden_size, int64_t hidden_stride,
                        int64_t slot_stride, int64_t num_slots,
                        int64_t num_hidden_rows, int64_t slot_mapping_len,
                        int elem_size, aps_stream_t stream);

/* ref: mixed_cache.cu:150-176 (cache_to_hidden) and :6-28 (kernel).
 * For b in [0,n): t = dst_idx[b]; hidden[t, :] = cache[slot_mapping[t]]. */
int aps_cache_to_hidden(void* hidden, const void* paged_cache,
                        const int64_t* slot_mapping, const int64_t* dst_idx,
                        int64_t n, int64_t hidden_size, int64_t hidden_stride,
                        int64_t slot_stride, int64_t num_slots,
                        int64_t num_hidden_rows, int64_t slot_mapping_len,
                        int elem_size, aps_stream_t stream);

/* ref: model_executor/models/aptserve_opt.py:108-121 — the decode-side
 * sequence hidden_to_cache -> zeros(num_tot,Hd) -> holder[upd]=hidden_states
 * -> cache_to_hidden(holder,...,hidden_cache_use_tot), as ONE launch with
 * disjoint destinations:
 *   holder[upd[b]]              = hidden_states[b]            b in [0,n_upd)
 *   holder[pull[i]]             = cache[slot_mapping[pull[i]]] (zeros if the
 *                                 slot is padding)            i in [0,n_pull)
 *   cache[slot_mapping[store_tot[j]]] = hidden_states[use_input[j]]
 *                                                             j in [0,n_store)
 * Every holder row is written, so the holder needs no prior memset. */
int aps_hybrid_decode_gather(void* holder, const void* hidden_states,
                             void* paged_cache, const int64_t* slot_mapping,
                             const int64_t* hidden_holder_upd, int64_t n_upd,
                             const int64_t* hidden_holder_pull, int64_t n_pull,
                             const int64_t* hidden_cache_use_input,
                             const int64_t* hidden_cache_store_tot,
                             int64_t n_store, int64_t hidden_size,
                             int64_t holder_stride, int64_t hidden_stride,
                             int64_t slot_stride, int64_t num_slots,
                             int64_t num_tot_tokens, int elem_size,
                             aps_stream_t stream);

/* Same result as aps_hybrid_decode_gather with the source of every holder row
 * resolved beforehand (aps_build_decode_metadata writes holder_src):
 *   holder_src[t] >= 0        holder[t] = cache slot holder_src[t]
 *   holder_src[t] = -(b+1)    holder[t] = hidden_states[b], b < num_inputs
 *   anything else             holder[t] = 0 (padding slot)
 * plus the n_store stores of the newest hidden rows into the cache.  One
 * dependent index load per chunk instead of two. */
int aps_gather_hidden_rows(void* holder, const void* hidden_states,
                           void* paged_cache, const int64_t* holder_src,
                           int64_t n_rows, const int64_t* slot_mapping,
                           const int64_t* hidden_cache_use_input,
                           const int64_t* hidden_cache_store_tot,
                           int64_t n_store, int64_t num_inputs,
                           int64_t hidden_size, int64_t holder_stride,
                           int64_t hidden_stride, int64_t slot_stride,
                           int64_t num_slots, int elem_size,
                           aps_stream_t stream);

/* The cache traffic of one decode layer in ONE launch: the holder assembly and
 * hidden stores of aps_gather_hidden_rows (same arguments, same result) plus the
 * write of the newest K/V rows of the K/V-cached sequences.  Replaces the call
 * sequence model_executor/models/aptserve_opt.py:108-121 (hidden_to_cache, zero
 * fill, index_put, cache_to_hidden) and the reshape_and_cache_flash of the new
 * K/V rows, attention/backends/aptserve_flash_attn.py:338-345:
 *   for i in [0, n_kv): b = kv_cache_use_input[i]; s = new_token_slot[b];
 *     key_cache[s/BS, s%BS] = key[b];  value_cache[s/BS, s%BS] = value[b]
 * (s < 0, s >= num_blocks*BS or b outside [0, num_inputs) skipped).  key/value
 * [num_inputs, hidden_size] with row strides key_stride / value_stride; the
 * caches [num_blocks, block_size, hidden_size] with block stride block_stride
 * (they may be the two planes of paged_cache); kv_cache_use_input and
 * new_token_slot as aps_build_decode_metadata writes them.  A K or V row has the
 * width of a hidden row (hidden_size = heads * head_size) and the dtype of the
 * hidden rows.  Bit-identical to aps_reshape_and_cache_flash (token_idx =
 * kv_cache_use_input) followed by aps_gather_hidden_rows; the destinations of
 * the three kinds of rows are disjoint, so no order between them is needed.
 * holder may be NULL (then holder_src too): no holder is assembled, n_rows is
 * only the length of slot_mapping, and the launch is the two kinds of stores —
 * what a flow that attends on the cached hidden rows themselves needs. */
int aps_decode_step_cache_ops(
    void* holder, const void* hidden_states, void* paged_cache,
    const int64_t* holder_src, int64_t n_rows, const int64_t* slot_mapping,
    const int64_t* hidden_cache_use_input,
    const int64_t* hidden_cache_store_tot, int64_t n_store, int64_t num_inputs,
    int64_t hidden_size, int64_t holder_stride, int64_t hidden_stride,
    int64_t slot_stride, int64_t num_slots, const void* key, const void* value,
    void* key_cache, void* value_cache, const int64_t* kv_cache_use_input,
    const int64_t* new_token_slot, int64_t n_kv, int64_t key_stride,
    int64_t value_stride, int block_size, int64_t block_stride,
    int64_t num_blocks, int elem_size, aps_stream_t stream);

/* A call of aps_decode_step_cache_ops that is checked and planned now and
 * launched later: the job (APS_CACHE_JOB_BYTES of host memory that the caller
 * owns, 8-byte aligned, opaque) records the arguments and the shape of the
 * launch.  Same arguments, checks and status codes as
 * aps_decode_step_cache_ops, whose reference call sites it shares
 * (model_executor/models/aptserve_opt.py:108-121,
 * attention/backends/aptserve_flash_attn.py:338-345); nothing is enqueued.
 * aps_cache_job_launch launches a job by itself, with the result of the direct
 * call; aps_hybrid_decode_attention takes one as the cache writes that precede
 * a decode step's attention.  The device memory the arguments point to must be
 * valid when the job is launched. */
#define APS_CACHE_JOB_BYTES 320
int aps_decode_step_cache_ops_job(
    void* job, int64_t job_bytes, void* holder, const void* hidden_states,
    void* paged_cache, const int64_t* holder_src, int64_t n_rows,
    const int64_t* slot_mapping, const int64_t* hidden_cache_use_input,
    const int64_t* hidden_cache_store_tot, int64_t n_store, int64_t num_inputs,
    int64_t hidden_size, int64_t holder_stride, int64_t hidden_stride,
    int64_t slot_stride, int64_t num_slots, const void* key, const void* value,
    void* key_cache, void* value_cache, const int64_t* kv_cache_use_input,
    const int64_t* new_token_slot, int64_t n_kv, int64_t key_stride,
    int64_t value_stride, int block_size, int64_t block_stride,
    int64_t num_blocks, int elem_size);
int aps_cache_job_launch(const void* job, aps_stream_t stream);

/* ------------------------------------------------------------------------
 * K/V row scatter into [num_blocks, block_size, H, D] caches.
 * ------------------------------------------------------------------------ */

/* ref: third-party vllm._custom_ops.reshape_and_cache_flash as called at
 * attention/backends/aptserve_flash_attn.py:338-345, :348-355, :378-385.
 * cache[slot/BS, slot%BS, :, :] = key[t] (and value), t in [0,n); slot<0 or
 * slot >= num_blocks*BS skipped.  in_dtype f16/bf16/f32; cache_dtype equal to
 * in_dtype (byte move) or APS_FP8_E4M3: code = e4m3(clamp(x/scale, +-448)).
 * token_idx (nullable): read key[token_idx[t]] / slot_mapping[token_idx[t]]
 * instead of t — the subset write of :348-355 without the gather copies. */
int aps_reshape_and_cache_flash(const void* key, const void* value,
                                void* key_cache, void* value_cache,
                                const int64_t* slot_mapping,
                                const int64_t* token_idx, int64_t n,
                                int64_t num_tokens, int num_heads,
                                int head_size, int block_size,
                                int64_t key_stride, int64_t value_stride,
                                int64_t block_stride, int64_t num_blocks,
                                int in_dtype, int cache_dtype, float k_scale,
                                float v_scale, aps_stream_t stream);

/* One write for a step whose tokens differ in cache type (the "mixed reshape
 * and cache"): token t with is_hidden[t] != 0 stores hidden[t, :H*D] at slot
 * slot_mapping[t] of the flattened hidden cache (hidden_cache + slot *
 * hidden_slot_stride, as aps_hidden_to_cache does), any other token stores
 * key[t] / value[t] by block as aps_reshape_and_cache_flash does.  Replaces, in
 * one launch, the pair model_executor/models/aptserve_opt.py:125-126
 * (hidden_to_cache over the hidden tokens) and
 * attention/backends/aptserve_flash_attn.py:347-355 (reshape_and_cache_flash
 * over gathered copies of the K/V tokens) of a prompt step.
 * is_hidden nullable (all K/V); key/value nullable (only hidden rows are
 * stored); hidden nullable (only K/V rows).  cache_dtype applies to the K/V
 * rows only (APS_FP8_E4M3: quantised with k_scale / v_scale, then the K/V and
 * the hidden cache are separate allocations); hidden rows keep in_dtype. */
int aps_mixed_reshape_and_cache(
    const void* key, const void* value, const void* hidden, void* key_cache,
    void* value_cache, void* hidden_cache, const int64_t* slot_mapping,
    const uint8_t* is_hidden, int64_t num_tokens, int num_heads, int head_size,
    int block_size, int64_t key_stride, int64_t value_stride,
    int64_t hidden_stride, int64_t block_stride, int64_t num_blocks,
    int64_t hidden_slot_stride, int64_t num_hidden_slots, int in_dtype,
    int cache_dtype, float k_scale, float v_scale, aps_stream_t stream);

/* ref: mixed_cache.cu:179-230 (mixed_kv_to_cache) and :56-116 (kernel).
 * Range A: K/V rows kv_cache_use_tot[i] -> private caches at
 * slot_mapping[tok]; range B: the same rows -> shared caches; range C: rows
 * hidden_cache_use_tot[j] -> shared caches at slot_mapping_shared[j].
 * flags: see APS_MIXED_*. */
int aps_mixed_kv_to_cache(const void* key, const void* value, void* k_cache,
                          void* v_cache, void* shared_k_cache,
                          void* shared_v_cache, const int64_t* slot_mapping,
                          const int64_t* slot_mapping_shared,
                          const int64_t* kv_cache_use_tot,
                          const int64_t* hidden_cache_use_tot, int64_t n_kv,
                          int64_t n_hidden, int64_t num_tot_tokens,
                          int num_heads, int head_size, int block_size,
                          int64_t key_stride, int64_t value_stride,
                          int64_t block_stride, int64_t num_blocks,
                          int64_t shared_block_stride,
                          int64_t num_shared_blocks, int elem_size,
                          unsigned flags, aps_stream_t stream);

/* ------------------------------------------------------------------------
 * Paged decode attention (one query token per sequence) over a hybrid cache.
 * ------------------------------------------------------------------------ */

/* Partition length (tokens) the library would choose for this problem; a
 * sequence longer than one partition is split and recombined (split-KV). */
int aps_decode_attention_partition_size(int64_t batch, int num_heads,
                                        int64_t max_seq_len, int block_size);

/* Bytes of scratch aps_paged_decode_attention needs (0 if every sequence
 * fits one partition).  The caller owns the scratch. */
int64_t aps_decode_attention_workspace_bytes(int64_t batch, int num_heads,
                                             int head_size,
                                             int64_t max_seq_len,
                                             int partition_size);

/* ref: third-party vllm_flash_attn.flash_attn_with_kvcache as called at
 * attention/backends/aptserve_flash_attn.py:452-461 (private cache) and
 * :464-473 (shared cache):  for sequence b, head h, L = seq_lens[b]:
 *   out[b,h,:] = softmax_j(softmax_scale * <q[b,h,:], K_j>) V,  j in [0,L)
 *   K_j / V_j  = cache[block_tables[b, j/BS], j%BS, h, :]
 * in fp32, result rounded to q's dtype.  seq_lens[b] <= 0 gives zeros.
 *
 * Hybrid extension: block_types (nullable, uint8 [batch, >=table_width],
 * row stride types_stride) selects per logical block the persistent cache
 * (0) or the re-projection workspace caches ws_k_cache/ws_v_cache (!= 0),
 * which share the [blocks, BS, H, D] layout and kv_dtype.
 *
 * q/out: [batch, H, D] f16 or bf16, row strides q_stride/out_stride.
 * kv_dtype: equal to q_dtype, or APS_FP8_E4M3 (K = code*k_scale, V = code*
 * v_scale).  head_size in {32,64,128,256} (no 32 with fp8); block_size a
 * multiple of 16.  block ids outside [0, num_*_blocks) contribute nothing.
 * max_seq_len: host-side upper bound of seq_lens (sizes the partition grid).
 * partition_size: 0 = library default, else a multiple of block_size with
 * at most 64 blocks. */
int aps_paged_decode_attention(
    void* out, const void* q, const void* k_cache, const void* v_cache,
    const void* ws_k_cache, const void* ws_v_cache,
    const int32_t* block_tables, const uint8_t* block_types,
    const int32_t* seq_lens, int64_t batch, int num_heads, int head_size,
    int block_size, int64_t table_width, int64_t table_stride,
    int64_t types_stride, int64_t q_stride, int64_t out_stride,
    int64_t cache_block_stride, int64_t num_cache_blocks,
    int64_t ws_block_stride, int64_t num_ws_blocks, int64_t max_seq_len,
    int partition_size, float softmax_scale, int q_dtype, int kv_dtype,
    float k_scale, float v_scale, void* workspace, int64_t workspace_bytes,
    aps_stream_t stream);

/* aps_paged_decode_attention for callers that cannot allocate device memory
 * or bring a workspace: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same
 * arguments and bit-identical results; the partial results of split sequences
 * go to a device array of APS_STATIC_SCRATCH_BYTES that is part of the library
 * image (one copy per GPU, held until the process ends) instead of a caller
 * workspace.  The call allocates and frees nothing.  A problem that needs more
 * (aps_decode_attention_workspace_bytes(...) > APS_STATIC_SCRATCH_BYTES) is
 * rejected with APS_ERR_SCRATCH_LIMIT before anything is launched.  The device
 * of the call is the current device.  Every call on a GPU uses that GPU's one
 * array: calls that overlap in time on the same GPU (two streams, two
 * threads) race; calls on one stream are ordered and safe.  Nothing in the
 * array has to start at zero (every partial that is read was written by the
 * same call), so it is never cleared.  The first call on a device looks the
 * array's device address up (hipGetSymbolAddress, which may load the library's
 * code object): make that call outside a stream capture; every later call on
 * the device only enqueues kernels and may be captured. */
#define APS_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)
int aps_paged_decode_attention_static(
    void* out, const void* q, const void* k_cache, const void* v_cache,
    const void* ws_k_cache, const void* ws_v_cache,
    const int32_t* block_tables, const uint8_t* block_types,
    const int32_t* seq_lens, int64_t batch, int num_heads, int head_size,
    int block_size, int64_t table_width, int64_t table_stride,
    int64_t types_stride, int64_t q_stride, int64_t out_stride,
    int64_t cache_block_stride, int64_t num_cache_blocks,
    int64_t ws_block_stride, int64_t num_ws_blocks, int64_t max_seq_len,
    int partition_size, float softmax_scale, int q_dtype, int kv_dtype,
    float k_scale, float v_scale, aps_stream_t stream);

/* A call of aps_paged_decode_attention that is checked and planned now and
 * launched later: the job (APS_ATTENTION_JOB_BYTES of host memory that the
 * caller owns, 8-byte aligned, opaque) records the arguments, the partitioning
 * and the kernel that the call would have launched.  Same arguments, checks
 * and status codes as aps_paged_decode_attention; nothing is enqueued.
 * aps_attention_job_launch launches a job by itself, with the results of the
 * direct call bit for bit; aps_hybrid_decode_attention takes one as the K/V-
 * cached half of a decode step's attention.  The device memory the arguments
 * point to (workspace included) must be valid when the job is launched; a job
 * may be launched any number of times.  ref: the same call sites as
 * aps_paged_decode_attention (attention/backends/aptserve_flash_attn.py:452-461,
 * :464-473). */
#define APS_ATTENTION_JOB_BYTES 320
int aps_paged_decode_attention_job(
    void* job, int64_t job_bytes, void* out, const void* q,
    const void* k_cache, const void* v_cache, const void* ws_k_cache,
    const void* ws_v_cache, const int32_t* block_tables,
    const uint8_t* block_types, const int32_t* seq_lens, int64_t batch,
    int num_heads, int head_size, int block_size, int64_t table_width,
    int64_t table_stride, int64_t types_stride, int64_t q_stride,
    int64_t out_stride, int64_t cache_block_stride, int64_t num_cache_blocks,
    int64_t ws_block_stride, int64_t num_ws_blocks, int64_t max_seq_len,
    int partition_size, float softmax_scale, int q_dtype, int kv_dtype,
    float k_scale, float v_scale, void* workspace, int64_t workspace_bytes);
int aps_attention_job_launch(const void* job, aps_stream_t stream);

/* ------------------------------------------------------------------------
 * Prompt-step attention on freshly projected q/k/v (no cache read).
 * ref: third-party vllm_flash_attn.flash_attn_varlen_func with causal=True as
 * called at attention/backends/aptserve_flash_attn.py:414-426.  Sequences are
 * packed along the token dimension and delimited by cu_seqlens (int32
 * [num_seqs+1], leading 0); query i of a sequence attends to keys 0..i of the
 * same sequence; softmax in fp32; result in the operand dtype.
 * q/k/v/out: [tokens, H, D] with token-row strides (elements), heads
 * contiguous; f16 or bf16; D in {64, 128}.  num_tokens: rows of q/k/v/out; a
 * sequence whose boundaries do not satisfy 0 <= cu[i] <= cu[i+1] <= num_tokens
 * is skipped (its rows of out are not written).  max_seqlen: host-side bound
 * of the sequence lengths (sizes the grid): queries at positions >= max_seqlen
 * of a longer sequence are not computed, so it must not be an underestimate.
 * softmax_scale must be positive and finite (the kernel takes the running
 * maximum on unscaled scores); anything else is APS_ERR_INVALID_ARG.
 * ------------------------------------------------------------------------ */
int aps_varlen_prefill_attention(void* out, const void* q, const void* k,
                                 const void* v, const int32_t* cu_seqlens,
                                 int64_t num_seqs, int64_t num_tokens,
                                 int64_t max_seqlen,
                                 int num_heads, int head_size,
                                 int64_t q_stride, int64_t k_stride,
                                 int64_t v_stride, int64_t out_stride,
                                 float softmax_scale, int dtype,
                                 aps_stream_t stream);

/* Prompt-step attention that continues a cached prefix (chunked prompts, prefix
 * caching).  ref: third-party vllm_flash_attn.flash_attn_varlen_func with
 * block_table=, as called at attention/backends/aptserve_flash_attn.py:431-447
 * (k=key_cache, v=value_cache, cu_seqlens_q=query_start_loc,
 * cu_seqlens_k=seq_start_loc, causal=True).  The queries are the step's new
 * tokens, packed and delimited by cu_seqlens_q; sequence i has
 * klen = cu_seqlens_k[i+1] - cu_seqlens_k[i] tokens in all (prefix + new), whose
 * K / V rows are read from the [blocks, block_size, H, D] caches through
 * block_tables[i, j / block_size] (the new tokens' rows must have been written
 * already); query j of its qlen new tokens attends to keys 0 .. j + klen - qlen
 * (bottom-right aligned causal mask).  A sequence with klen < qlen, with more
 * blocks than table_width or with bad boundaries is skipped; block ids are
 * clamped into [0, num_cache_blocks).  Otherwise as aps_varlen_prefill_attention
 * (dtypes, head sizes, softmax_scale > 0, max_seqlen_q bounds the qlen). */
int aps_paged_prefill_attention(
    void* out, const void* q, const void* k_cache, const void* v_cache,
    const int32_t* block_tables, const int32_t* cu_seqlens_q,
    const int32_t* cu_seqlens_k, int64_t num_seqs, int64_t num_q_tokens,
    int64_t max_seqlen_q, int num_heads, int head_size, int block_size,
    int64_t table_stride, int64_t table_width, int64_t q_stride,
    int64_t out_stride, int64_t cache_block_stride, int64_t num_cache_blocks,
    float softmax_scale, int dtype, aps_stream_t stream);

/* ------------------------------------------------------------------------
 * Ragged-batch metadata, built on the GPU from a per-sequence description.
 * ref: worker/aptserve_model_runner.py:240-842 (_prepare_model_input), hybrid
 * parts :256-304, :410-437, :516-564, :601-668, :707-733, :772-785.
 * Inputs are int32 device arrays of one entry per sequence (use_hidden: 0/1)
 * and 0-padded block tables; outputs are caller-allocated with the given
 * capacities (entries beyond a capacity are dropped, never written).
 * totals (nullable, int64[4]) receives {rows, hidden rows, hidden sequences,
 * K/V rows or sequences} as computed on the device.
 * ------------------------------------------------------------------------ */

/* Decode step (:525-539, :554-564, :617-645).  Row space "tot": a hidden-cached
 * sequence contributes seq_len rows (its whole context is re-projected), a
 * K/V-cached one a single row.
 *   slot_mapping[row]        private slot of token j (hidden) / of the new token (K/V)
 *   slot_mapping_shared[i]   slot of token j in the shared (workspace) table, hidden rows only
 *   hidden_cache_use_tot / kv_cache_use_tot    rows by cache type, ascending
 *   hidden_holder_upd[b]     row of sequence b's newest token; hidden_holder_pull = the rest
 *   hidden_cache_use_input   batch positions of hidden sequences
 *   hidden_cache_store_tot   their newest rows
 *   holder_src[row]          (nullable, not in the reference) resolved source of the row for
 *                            aps_gather_hidden_rows: slot, -(b+1) for the newest row, INT64_MIN for padding
 *   hidden_slots[i]          (nullable, not in the reference) private slot of hidden row i, in the order of
 *                            hidden_cache_use_tot; hidden_seq_start[j] (nullable, n hidden sequences + 1
 *                            entries) first hidden row of the j-th hidden sequence: aps_absorbed_attention
 *   kv_cache_use_input[i]    (nullable, not in the reference) batch position of the i-th K/V-cached sequence;
 *                            new_token_slot[b] private slot of sequence b's newest token; kv_seq_lens[b]
 *                            (int32) seq_len of a K/V-cached sequence, 0 for a hidden-cached one — what a
 *                            step needs to write and attend the K/V-cached sequences only
 *   kv_dest[row]             (nullable, not in the reference) where the row's re-projected K/V go, for
 *                            aps_kv_reproject_to_cache: shared slot (hidden rows), -(private slot + 2)
 *                            (the new token of a K/V sequence), -1 for padding
 *   block_tables_out[b,:]    shared table for hidden sequences, private otherwise (:415-418);
 *   block_types_out[b,:]     (nullable, uint8 [batch, out_width] contiguous, not in the reference) 1 in every
 *                            column of a hidden-cached sequence: the per-block source mask of
 *                            aps_paged_decode_attention
 *   seq_start_loc / query_start_loc int32 cumulative sums with leading 0;
 *   context_lens = seq_len-1; input_positions = seq_len-1. */
int aps_build_decode_metadata(
    const int32_t* seq_lens, const int32_t* use_hidden,
    const int32_t* block_tables, int64_t table_stride, int64_t table_width,
    const int32_t* block_tables_shared, int64_t shared_stride,
    int64_t shared_width, int64_t batch, int block_size, int64_t* slot_mapping,
    int64_t* slot_mapping_shared, int64_t* hidden_cache_use_tot,
    int64_t* kv_cache_use_tot, int64_t* hidden_cache_use_input,
    int64_t* hidden_cache_store_tot, int64_t* hidden_holder_upd,
    int64_t* hidden_holder_pull, int64_t* holder_src, int64_t* kv_dest,
    int64_t* hidden_slots, int64_t* hidden_seq_start,
    int64_t* kv_cache_use_input, int64_t* new_token_slot, int32_t* kv_seq_lens,
    int64_t cap_rows, int64_t cap_hidden_rows,
    int64_t cap_hidden_seqs, int64_t cap_kv_seqs, int32_t* block_tables_out,
    int64_t out_stride, int64_t out_width, uint8_t* block_types_out,
    int32_t* seq_start_loc,
    int32_t* query_start_loc, int32_t* context_lens, int64_t* input_positions,
    int64_t* totals, aps_stream_t stream);

/* Prompt step (:542-552, :648-666).  Row space = token space; token i of a
 * sequence (i in [context_len, seq_len)) gets slot table[i/BS]*BS + i%BS, or
 * -1 when table_width is 0.  hidden_cache_use_input = tokens of hidden-cached
 * prompts (it also serves as hidden_cache_use_tot and hidden_cache_store_tot),
 * kv_cache_use_tot = the other tokens.  context_lens_in may be NULL (= 0).
 * token_is_hidden (nullable, not in the reference): 1 for every token of a
 * hidden-cached prompt, 0 otherwise: the mask aps_mixed_reshape_and_cache takes. */
int aps_build_prefill_metadata(
    const int32_t* seq_lens, const int32_t* context_lens_in,
    const int32_t* use_hidden, const int32_t* block_tables,
    int64_t table_stride, int64_t table_width, int64_t batch, int block_size,
    int64_t* slot_mapping, int64_t* input_positions,
    int64_t* hidden_cache_use_input, int64_t* kv_cache_use_tot,
    uint8_t* token_is_hidden, int64_t cap_tokens, int64_t cap_hidden_tokens,
    int64_t cap_kv_tokens,
    int32_t* seq_start_loc, int32_t* query_start_loc, int32_t* context_lens,
    int64_t* totals, aps_stream_t stream);

/* ------------------------------------------------------------------------
 * q-only / kv-only projection on the matrix cores.
 * ref: model_executor/layers/aptserve_linear.py:102-132 (UnquantizedLinearMethod
 * .apply with q_only / kv_only = F.linear on a row slice of the fused QKV
 * weight), called at model_executor/models/aptserve_opt.py:116 and :123-124.
 *   out[m, n] = sum_k x[m, k] * weight[n, k] + bias[n]
 * x [m, k] and weight [n, k] are K-contiguous with row strides x_stride /
 * w_stride (pass weight + slice*w_stride for a row slice); bias nullable;
 * f16 or bf16 operands, fp32 accumulation, result rounded once to the operand
 * dtype.  n must be a multiple of 256 and k of 64.
 * out_row_map (nullable): row m is stored at row out_row_map[m] of out (rows of
 * out_stride elements; negative or >= out_rows: skipped) — the epilogue that
 * writes re-projected K/V rows straight into [blocks, BS, H, D] tiles by slot.
 * workspace (nullable): fp32 scratch of aps_linear_nt_workspace_bytes(m,n,k)
 * bytes, 16-byte aligned, owned by the caller.  With it, a problem whose output
 * tiles leave CUs idle (a decode step's rows: anything from 3 rows up to a few
 * hundred) is split along K into aps_linear_nt_splits(m,n,k) partial products
 * that a second kernel adds (in fp32, then bias, then one rounding); without it
 * a single-launch kernel runs.  A workspace that is passed but too small or
 * misaligned is an error (APS_ERR_WORKSPACE), never a silent fallback.
 * flags: APS_LINEAR_RELU stores max(result, 0) — the ReLU between fc1 and fc2
 * of the decoder's MLP (model_executor/models/aptserve_opt.py:204-206:
 * `fc1`, `activation_fn`, `fc2`) without an element-wise launch of its own; the
 * rounded values are those of "linear, then relu" on 16-bit tensors.
 * tile_counters (nullable): APS_LINEAR_TILE_COUNTERS int32 that are zero on
 * entry and zero again when the call's work is done, owned by the caller (one
 * array per stream that calls concurrently).  With them the K split of a decode
 * step's few rows (3..48) needs no second launch: the workgroup that stores the
 * last partial product of an output tile adds the tile's parts itself (in part
 * order: the result is bit for bit the two-launch one).
 * ------------------------------------------------------------------------ */
#define APS_LINEAR_TILE_COUNTERS 256
int aps_linear_nt_splits(int64_t m, int64_t n, int64_t k);
int64_t aps_linear_nt_workspace_bytes(int64_t m, int64_t n, int64_t k);
int aps_linear_nt(const void* x, const void* weight, const void* bias,
                  void* out, int64_t m, int64_t n, int64_t k, int64_t x_stride,
                  int64_t w_stride, int64_t out_stride,
                  const int64_t* out_row_map, int64_t out_rows, int dtype,
                  int flags, void* workspace, int64_t workspace_bytes,
                  int32_t* tile_counters, aps_stream_t stream);

/* K/V re-projection with the cache write fused into the epilogue: one pass that
 * replaces the kv_only projection (model_executor/models/aptserve_opt.py:123-124),
 * the chunk into key/value, and ranges (A) and (C) of mixed_kv_to_cache
 * (mixed_cache_kernels/mixed_cache.cu:56-116, called at
 * attention/backends/aptserve_flash_attn.py:359-373); the mirror range (B) has
 * no reader and is not written.
 *   kv[t, :] = x[t, :] * w_kv[2*hidden_size, k]^T + b_kv;  K = kv[t, :hidden_size], V = the rest
 *   kv_dest[t] >= 0   K -> ws_k_cache slot kv_dest[t], V -> ws_v_cache (slots < ws_slots)
 *   kv_dest[t] <= -2  K -> k_cache slot -(kv_dest[t]+2), V -> v_cache (slots < cache_slots)
 *   kv_dest[t] == -1 or out of range: row not stored
 * A slot is slot_stride elements (= heads*head_size of a [blocks, BS, H, D]
 * cache); hidden_size must be a multiple of 256, k of 64.  The intermediate
 * [m, 2*hidden_size] matrix is never materialised.  workspace as for
 * aps_linear_nt with n = 2*hidden_size. */
int aps_kv_reproject_to_cache(
    const void* x, const void* w_kv, const void* b_kv, void* ws_k_cache,
    void* ws_v_cache, void* k_cache, void* v_cache, const int64_t* kv_dest,
    int64_t m, int64_t hidden_size, int64_t k, int64_t x_stride,
    int64_t w_stride, int64_t slot_stride, int64_t ws_slots,
    int64_t cache_slots, int dtype, void* workspace, int64_t workspace_bytes,
    aps_stream_t stream);

/* aps_kv_reproject_to_cache without the holder: the rows of the product's left
 * operand are fetched where they are cached instead of being gathered into a
 * contiguous [m, k] matrix first (replaces, in addition, the holder assembly
 * model_executor/models/aptserve_opt.py:112-121: zero fill, index_put and
 * cache_to_hidden).  Row t of the operand is
 *   holder_src[t] >= 0       slot holder_src[t] of paged_cache (rows of
 *                            cache_slot_stride elements, < num_cache_slots)
 *   holder_src[t] = -(b+1)   row b of hidden_states (the step's input, rows of
 *                            hidden_stride elements, b < num_inputs)
 * as aps_build_decode_metadata writes it.  Any other value marks a row without
 * a source: it is multiplied with unspecified (valid) data and must not be
 * stored, i.e. its kv_dest must be -1 (the metadata builder guarantees that).
 * The newest hidden rows still have to be stored into the cache by the caller
 * (aps_hidden_to_cache); this call does not depend on that store.  Results are
 * bit-identical to aps_gather_hidden_rows followed by aps_kv_reproject_to_cache.
 * Everything else as for aps_kv_reproject_to_cache. */
int aps_kv_reproject_gathered(
    const void* paged_cache, int64_t cache_slot_stride, int64_t num_cache_slots,
    const void* hidden_states, int64_t hidden_stride, int64_t num_inputs,
    const int64_t* holder_src, int64_t m, const void* w_kv, const void* b_kv,
    void* ws_k_cache, void* ws_v_cache, void* k_cache, void* v_cache,
    const int64_t* kv_dest, int64_t hidden_size, int64_t k, int64_t w_stride,
    int64_t slot_stride, int64_t ws_slots, int64_t cache_slots, int dtype,
    void* workspace, int64_t workspace_bytes, aps_stream_t stream);

/* Decode attention of hidden-cached sequences on their cached hidden rows, the
 * projections absorbed into the query and the output ("next" item 2 of the
 * hybrid path; replaces, for those sequences, the holder gather
 * model_executor/models/aptserve_opt.py:112-121, the kv_only re-projection
 * :123-124, mixed_kv_to_cache and the attention over the shared cache
 * attention/backends/aptserve_flash_attn.py:359-373, :464-473):
 *   s[h][t] = scale * <W_k[h]^T q[h], hidden_t>;  p = softmax_t(s)
 *   out[h]  = W_v[h] (sum_t p[h][t] hidden_t) + b_v[h]
 * (the key bias adds the same amount to every score of a head and drops out).
 *   q [num_q_rows, H*D] (row stride q_stride): query rows of the batch; sequence
 *     i of the n_seqs hidden-cached ones uses row seq_rows[i] and its result is
 *     stored at out[seq_rows[i]] (rows of out_stride elements, < out_rows).
 *   hidden_slots[seq_start[i] .. seq_start[i+1]) : slot of every cached row of
 *     sequence i in the flattened paged cache (row = paged_cache + slot *
 *     slot_stride), oldest first, the newest row included (it must have been
 *     stored already); both written by aps_build_decode_metadata.
 *   w_k, w_v [H*D, H*D] row-major [out, in] with row stride w_stride (row
 *     slices of the fused QKV weight); b_v nullable.
 *   max_len >= the longest sequence.  f16 / bf16; head_size % 32 == 0.
 * workspace: aps_absorbed_attention_workspace_bytes(...) bytes, 16-byte
 * aligned, owned by the caller (query images, fp32 scores,
 * per-head context vectors). */
int64_t aps_absorbed_attention_workspace_bytes(int64_t n_seqs, int64_t max_len,
                                               int num_heads, int head_size);
int aps_absorbed_attention(
    const void* q, int64_t q_stride, const int64_t* seq_rows,
    int64_t num_q_rows, const void* paged_cache, int64_t slot_stride,
    int64_t num_slots, const int64_t* hidden_slots, const int64_t* seq_start,
    int64_t n_seqs, int64_t max_len, const void* w_k, const void* w_v,
    const void* b_v, int64_t w_stride, int num_heads, int head_size,
    float softmax_scale, void* out, int64_t out_stride, int64_t out_rows,
    int dtype, void* workspace, int64_t workspace_bytes, aps_stream_t stream);

/* The attention of a decode step over both kinds of sequence, as one call:
 * aps_absorbed_attention for the hidden-cached sequences (same arguments,
 * same results) and, for the K/V-cached ones, the paged decode attention that
 * kv_job (nullable; from aps_paged_decode_attention_job) describes, with the
 * results of launching that job by itself.  ref: the reference attends both
 * kinds in one flash_attn_with_kvcache call over the shared cache
 * (attention/backends/aptserve_flash_attn.py:464-473) after re-projecting the
 * hidden-cached ones.  The two halves are independent (they write different
 * rows of out), so the library is free to overlap them: for a small batch
 * whose K/V-cached sequences fit the one-workgroup-per-sequence path (f16 /
 * bf16 cache, head size 128) the job's workgroups ride in the launch of the
 * weighted sum over the hidden rows, which leaves most compute units idle;
 * otherwise the job is launched by itself, after the stores.
 * store_job (nullable; from aps_decode_step_cache_ops_job): the step's cache
 * writes, which the reference's attention forward also begins with
 * (attention/backends/aptserve_flash_attn.py:338-345, after
 * model_executor/models/aptserve_opt.py:108-111).  They are complete before
 * either kind of attention reads the caches: inside the launch of the absorbed
 * queries (which touches no cache) when the job moves 16 bytes per lane in one
 * grid row and the head size is at most 128, by a launch of their own before
 * everything else otherwise.  n_seqs == 0: only the jobs, stores first. */
int aps_hybrid_decode_attention(
    const void* store_job, const void* kv_job, const void* q, int64_t q_stride,
    const int64_t* seq_rows, int64_t num_q_rows, const void* paged_cache,
    int64_t slot_stride, int64_t num_slots, const int64_t* hidden_slots,
    const int64_t* seq_start, int64_t n_seqs, int64_t max_len, const void* w_k,
    const void* w_v, const void* b_v, int64_t w_stride, int num_heads,
    int head_size, float softmax_scale, void* out, int64_t out_stride,
    int64_t out_rows, int dtype, void* workspace, int64_t workspace_bytes,
    aps_stream_t stream);

/* Residual add and LayerNorm of a decoder layer in one launch.
 * ref: model_executor/models/aptserve_opt.py:186-211 (OPTDecoderLayer.forward:
 * `hidden_states = residual + hidden_states` followed by the next nn.LayerNorm,
 * which at :188-189 produces the rows a hidden-cached sequence caches).
 *   s[r, :]      = round16(x[r, :] + residual[r, :])        (residual nullable: s = x)
 *   normed[r, :] = LayerNorm(s[r, :]) * gamma + beta        (fp32 statistics over the rounded sum, eps as given)
 * sum (nullable) receives s, the next residual.  f16 / bf16; width a multiple
 * of 8, at most 16384; strides in elements; all pointers 16-byte aligned. */
int aps_add_layer_norm(void* normed, void* sum, const void* x,
                       const void* residual, const void* gamma,
                       const void* beta, int64_t rows, int64_t width,
                       int64_t x_stride, int64_t residual_stride,
                       int64_t normed_stride, int64_t sum_stride, float eps,
                       int dtype, aps_stream_t stream);

/* ------------------------------------------------------------------------
 * Block maintenance, aware of hidden blocks.
 * ref: attention/backends/aptserve_flash_attn.py:44-65 (swap_blocks /
 * copy_blocks over the third-party vllm._custom_ops of the same names, called
 * from worker/aptserve_cache_engine.py:88-99).  The reference copies the K and
 * the V plane of block ids < N; a hidden block is ONE plane slab whose id runs
 * over the 2N slabs (id < N: K plane of block id, id >= N: V plane of block
 * id - N; core/aptserve_block_manager.py:176-192), which those calls cannot
 * address.  kinds[i] = 0: K/V block (both planes), 1: hidden block (one slab).
 * ------------------------------------------------------------------------ */

/* copy_blocks: pairs [n][2] (source, destination) on the device, applied to
 * every layer; layer_caches is a device array of the layers' cache base
 * addresses ((2, N, BS, H, D) contiguous, row_elems = H*D). */
int aps_copy_cache_blocks(const int64_t* layer_caches, int64_t num_layers,
                          const int64_t* pairs, const uint8_t* kinds,
                          int64_t n_pairs, int64_t num_blocks, int block_size,
                          int64_t row_elems, int elem_size,
                          aps_stream_t stream);

/* swap_blocks: pairs and kinds in HOST memory (as the reference passes them);
 * one asynchronous copy per plane slab between two caches (device <-> pinned
 * host, or device <-> device) of src_num_blocks / dst_num_blocks blocks;
 * block_bytes = BS*H*D*elem_size. */
int aps_swap_cache_blocks(const void* src_cache, void* dst_cache,
                          const int64_t* pairs_host, const uint8_t* kinds_host,
                          int64_t n_pairs, int64_t src_num_blocks,
                          int64_t dst_num_blocks, int64_t block_bytes,
                          aps_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* APTSERVE_HIP_H */
