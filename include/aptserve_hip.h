/*
 * aptserve_hip.h — C ABI of the MI355X (gfx950) hybrid-cache library.
 *
 * One shared library, libaptserve_hip.so, exports every function below with C
 * linkage.  All pointers are device pointers unless a parameter says "host".
 * All tensors are owned by the caller; the library never allocates, frees or
 * retains device memory and keeps no global state, so calls are re-entrant.
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

#define APS_ABI_VERSION 1

typedef void* aps_stream_t; /* a hipStream_t; NULL = the null stream */

enum aps_status {
  APS_OK = 0,
  APS_ERR_INVALID_ARG = -1, /* null pointer, negative size, bad enum */
  APS_ERR_UNSUPPORTED = -2, /* shape / dtype combination not built */
  APS_ERR_WORKSPACE = -3    /* workspace too small */
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

/* Plain device copy of nbytes (16-byte aligned pointers): the known-size
 * kernel that hardware counters of the kernels above are scaled against. */
int aps_copy_bytes(void* dst, const void* src, int64_t nbytes,
                   aps_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* APTSERVE_HIP_H */
