"""Attention backend and decoder-attention orchestration over the hybrid cache.

Host-side mirrors of the reference classes on the hot path:

* ``HybridCacheBackend``   <- ``FlashAttentionBackend``
  (additional_designs/attention/backends/aptserve_flash_attn.py:15-65)
* ``allocate_caches``      <- ``CacheEngine._allocate_kv_cache``
  (additional_designs/worker/aptserve_cache_engine.py:61-86)
* ``HybridAttentionImpl``  <- ``FlashAttentionImpl.forward`` (``aptserve_flash_attn.py:290-478``)
* ``HybridOPTAttention``   <- ``OPTAttention.forward``
  (additional_designs/model_executor/models/aptserve_opt.py:99-134)

Two data flows are offered for a decode batch that mixes cache types:

``literal=True`` replays the reference's operator sequence: ``mixed_kv_to_cache`` with the
mirror range, then one attention call over the shared cache for every sequence.  In the
reference the mirror region (shared blocks ``0..N-1``) only ever receives the newest token
of the current layer, so K/V-cached sequences of a mixed batch attend over stale history;
that is kept only so the two flows can be compared where they must agree (all-hidden and
no-hidden batches).

``literal=False`` (default) removes the mirror: K/V-cached sequences read their private
cache, hidden-cached sequences read the re-projected K/V in the shared workspace, selected
per block inside one attention launch.
"""

from __future__ import annotations

from typing import Callable, List, Optional, Tuple

import torch

from . import ops
from .layers import QKVLinear
from .metadata import HybridAttentionMetadata


class HybridCacheBackend:
    @staticmethod
    def get_supported_head_sizes() -> List[int]:
        return [32, 64, 128, 256]

    @staticmethod
    def get_name() -> str:
        return "hybrid-cache-hip"

    @staticmethod
    def get_impl_cls():
        return HybridAttentionImpl

    @staticmethod
    def make_metadata(*args, **kwargs) -> HybridAttentionMetadata:
        return HybridAttentionMetadata(*args, **kwargs)

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int) -> Tuple[int, ...]:
        if block_size % 16 != 0:
            raise ValueError("Block size must be a multiple of 16.")
        return (2, num_blocks, block_size, num_kv_heads, head_size)


def allocate_caches(num_layers: int, num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                    dtype: torch.dtype, device) -> Tuple[List[torch.Tensor], torch.Tensor]:
    """One zeroed ``(2, N, BS, H, D)`` cache per layer and ONE ``(2, 2N, BS, H, D)`` shared
    cache for all layers (blocks ``N..2N-1`` are the per-step K/V workspace)."""
    shape = HybridCacheBackend.get_kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size)
    kv = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(num_layers)]
    shared = torch.zeros((shape[0], 2 * shape[1]) + shape[2:], dtype=dtype, device=device)
    return kv, shared


class HybridAttentionImpl:
    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: Optional[int] = None,
                 alibi_slopes=None, sliding_window=None, kv_cache_dtype: str = "auto", *, literal: bool = False,
                 prefill_attention: Optional[Callable] = None, k_scale: float = 1.0, v_scale: float = 1.0) -> None:
        if alibi_slopes is not None:
            raise ValueError("alibi_slopes is not supported (OPT has none)")
        if sliding_window is not None:
            raise ValueError("Sliding window is not supported.")     # aptserve_flash_attn.py:277-282
        if num_kv_heads not in (None, num_heads):
            raise ValueError("grouped-query attention is outside the OPT path")
        if head_size not in HybridCacheBackend.get_supported_head_sizes():
            raise ValueError(f"Head size {head_size} is not supported. "
                             f"Supported head sizes are: {HybridCacheBackend.get_supported_head_sizes()}.")
        self.num_heads, self.head_size, self.scale = num_heads, head_size, float(scale)
        self.num_kv_heads = num_heads
        if kv_cache_dtype not in ("auto", "fp8", "fp8_e4m3"):
            raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")
        self.kv_cache_dtype = kv_cache_dtype
        self.fp8 = kv_cache_dtype != "auto"
        if self.fp8 and literal:
            raise ValueError("the literal (mirror-writing) flow is a byte move: it has no fp8 form")
        # per-tensor scales of an fp8-e4m3 K/V cache (K = code * k_scale); the reference has none
        # (aptserve_flash_attn.py:311-312 asserts kv_scale == 1.0)
        self.k_scale, self.v_scale = float(k_scale), float(v_scale)
        self.literal = literal
        self.prefill_attention = prefill_attention

    def forward(self, query, key, value, kv_cache, shared_cache, attn_metadata: HybridAttentionMetadata,
                kv_scale: float = 1.0, kv_written: bool = False) -> torch.Tensor:
        """``query [tokens, H*D]``, ``key``/``value [rows, H*D]`` (rows = tokens, or the 'tot' rows of a
        decode batch with hidden-cached sequences) -> ``[tokens, H*D]``.

        ``kv_written``: the caller has already put this step's K/V into the caches
        (``ops.kv_reproject_to_cache`` in a decode step, where ``key = value = None`` is then
        allowed; ``ops.mixed_reshape_and_cache`` in a prompt step), only the attention runs."""
        assert self.fp8 or kv_scale == 1.0, "kv_scale needs an fp8 K/V cache"            # :312
        ks, vs = self.k_scale * kv_scale, self.v_scale * kv_scale
        md = attn_metadata
        # a prompt step that continues a cached prefix (chunked prompts, prefix caching): the reference's prefix
        # branch (aptserve_flash_attn.py:431-447) attends over the K/V cache through the block table
        prefix = bool(md.num_prefills and md.max_prompt_context_len > 0)
        if prefix:
            if md.num_hidden_cache_tokens != 0:
                raise ValueError("a prompt step that continues a cached prefix cannot hold hidden-cached sequences: "
                                 "their prefix is cached as hidden rows, not as K/V")
            if kv_cache is None or self.fp8 or md.block_tables.numel() == 0:
                raise ValueError("the prefix branch needs a K/V cache in the activation dtype and block tables")
        num_tokens, hidden_size = query.shape
        H, D = self.num_heads, self.head_size
        query = query.view(-1, H, D)
        n_hidden, n_prefill, n_decode = md.num_hidden_cache_tokens, md.num_prefill_tokens, md.num_decode_tokens
        written = kv_written or key is None
        if key is None:
            assert value is None and n_prefill == 0
        else:
            key = key.view(-1, H, D)
            value = value.view(-1, H, D)
            if n_hidden == 0:
                assert key.shape[0] == n_prefill + n_decode and value.shape[0] == n_prefill + n_decode

        mixed = False
        if written:
            assert kv_cache is not None and not self.literal
            key_cache, value_cache = kv_cache[0], kv_cache[1]
            if n_hidden != 0 and n_prefill == 0:
                shared_k, shared_v = shared_cache[0], shared_cache[1]
                mixed = md.num_tot_tokens != md.slot_mapping_shared.numel()
        elif kv_cache is not None:
            key_cache, value_cache = kv_cache[0], kv_cache[1]
            if n_hidden == 0:                                                       # :334-345
                ops.reshape_and_cache_flash(key, value, key_cache, value_cache, md.slot_mapping,
                                            self.kv_cache_dtype, ks, vs)
            elif n_prefill != 0:                                                    # :347-355, without the gather copies
                ops.reshape_and_cache_flash(key, value, key_cache, value_cache, md.slot_mapping,
                                            self.kv_cache_dtype, ks, vs, token_idx=md.kv_cache_use_tot)
            else:
                shared_k, shared_v = shared_cache[0], shared_cache[1]
                mixed = md.num_tot_tokens != md.slot_mapping_shared.numel()         # :359
                if self.fp8:
                    # mixed_kv_to_cache is a byte move; the quantising write goes through two scatters whose
                    # slot vectors are indexed like the rows (from kv_dest: workspace slot, or -(private slot + 2))
                    ws_slots, private_slots = md.row_slots_by_destination()
                    ops.reshape_and_cache_flash(key, value, shared_k, shared_v, ws_slots, self.kv_cache_dtype, ks, vs)
                    if mixed:
                        ops.reshape_and_cache_flash(key, value, key_cache, value_cache, private_slots,
                                                    self.kv_cache_dtype, ks, vs)
                elif mixed:
                    ops.mixed_kv_to_cache(key, value, key_cache, value_cache, shared_k, shared_v, md.slot_mapping,
                                          md.slot_mapping_shared, md.kv_cache_use_tot, md.hidden_cache_use_tot,
                                          skip_mirror=not self.literal)
                else:                                                               # :376-385
                    ops.reshape_and_cache_flash(key, value, shared_k, shared_v, md.slot_mapping_shared,
                                                self.kv_cache_dtype)

        output = torch.empty_like(query)
        decode_query = query[n_prefill:]
        if md.prefill_metadata is not None:
            pm = md.prefill_metadata
            if prefix:                                   # aptserve_flash_attn.py:431-447
                ops.flash_attn_varlen_func(
                    q=query[:n_prefill], k=key_cache, v=value_cache, cu_seqlens_q=pm.query_start_loc,
                    max_seqlen_q=pm.max_query_len, cu_seqlens_k=pm.seq_start_loc,
                    max_seqlen_k=pm.max_prefill_seq_len, softmax_scale=self.scale, causal=True,
                    block_table=pm.block_tables, out=output[:n_prefill])
            elif self.prefill_attention is not None:     # caller-supplied prompt attention
                output[:n_prefill] = self.prefill_attention(query[:n_prefill], key[:n_prefill], value[:n_prefill],
                                                            pm.seq_start_loc, pm.max_prefill_seq_len, self.scale)
            else:                                        # aptserve_flash_attn.py:414-426
                ops.flash_attn_varlen_func(
                    q=query[:n_prefill], k=key[:n_prefill], v=value[:n_prefill], cu_seqlens_q=pm.seq_start_loc,
                    cu_seqlens_k=pm.seq_start_loc, max_seqlen_q=pm.max_prefill_seq_len,
                    max_seqlen_k=pm.max_prefill_seq_len, softmax_scale=self.scale, causal=True,
                    out=output[:n_prefill])
        if md.decode_metadata is not None:
            dm = md.decode_metadata
            max_len = dm.max_decode_seq_len or None
            if n_hidden == 0:                                                       # :451-461
                ops.paged_decode_attention(decode_query, key_cache, value_cache, dm.block_tables,
                                           dm.seq_lens_tensor, self.scale, max_seq_len=max_len,
                                           out=output[n_prefill:], k_scale=ks, v_scale=vs)
            elif self.literal or not mixed:                                         # :464-473
                ops.paged_decode_attention(decode_query, shared_k, shared_v, dm.block_tables, dm.seq_lens_tensor,
                                           self.scale, max_seq_len=max_len, out=output[n_prefill:], k_scale=ks,
                                           v_scale=vs)
            else:
                ops.paged_decode_attention(decode_query, key_cache, value_cache, dm.block_tables,
                                           dm.seq_lens_tensor, self.scale, block_types=dm.block_types,
                                           ws_k_cache=shared_k, ws_v_cache=shared_v, max_seq_len=max_len,
                                           out=output[n_prefill:], k_scale=ks, v_scale=vs)
        return output.view(num_tokens, hidden_size)


class PhaseTimes:
    """Optional per-phase GPU timing of the layers (events on the current stream).  ``with PhaseTimes() as t:``
    switches it on for the layers run inside; ``t.totals()`` (after a synchronize) gives milliseconds per phase
    name.  Off by default: the layers then only test one module attribute."""

    active: Optional["PhaseTimes"] = None

    def __init__(self) -> None:
        self.spans = []

    def __enter__(self):
        PhaseTimes.active = self
        return self

    def __exit__(self, *exc):
        PhaseTimes.active = None

    def totals(self):
        torch.cuda.synchronize()
        out = {}
        for name, a, b in self.spans:
            out[name] = out.get(name, 0.0) + a.elapsed_time(b)
        return out


class _Phase:
    __slots__ = ("name", "a")

    def __init__(self, name: str) -> None:
        self.name = name

    def __enter__(self):
        if PhaseTimes.active is not None:
            self.a = torch.cuda.Event(enable_timing=True)
            self.a.record()

    def __exit__(self, *exc):
        t = PhaseTimes.active
        if t is not None:
            b = torch.cuda.Event(enable_timing=True)
            b.record()
            t.spans.append((self.name, self.a, b))


def phase(name: str) -> _Phase:
    return _Phase(name)


class HybridOPTAttention:
    """Self-attention of one OPT decoder layer over the hybrid cache.

    ``fused=False`` issues the reference's operator sequence (``hidden_to_cache``,
    ``torch.zeros`` holder, index_put, ``cache_to_hidden``); ``fused=True`` replaces it by
    one ``gather_hidden_rows`` launch into an uninitialised holder.  Results are identical.

    ``fuse_kv_write=True`` (with ``fused`` and not ``literal``) lets the K/V re-projection write
    its rows straight into the cache slots (``ops.kv_reproject_to_cache``): no ``[T, 2*Hd]``
    intermediate and no ``mixed_kv_to_cache`` pass.  Results are identical again: the same
    values are rounded once and land in the same slots.

    ``holder_free=True`` (with ``fuse_kv_write``) also drops the holder: the re-projection reads every cached
    hidden row where it lies (``ops.kv_reproject_gathered``); only the newest hidden rows are stored first.
    """

    def __init__(self, embed_dim: int, num_heads: int, qkv_weight, qkv_bias, out_weight, out_bias, *,
                 fused: bool = True, literal: bool = False, prefill_attention: Optional[Callable] = None,
                 fuse_kv_write: bool = True, absorbed: bool = False, holder_free: bool = True,
                 kv_cache_dtype: str = "auto", k_scale: float = 1.0, v_scale: float = 1.0) -> None:
        self.embed_dim, self.num_heads = embed_dim, num_heads
        self.head_dim = embed_dim // num_heads
        self.scaling = self.head_dim ** -0.5
        self.qkv_proj = QKVLinear(qkv_weight, qkv_bias)
        self.out_weight, self.out_bias = out_weight, out_bias
        self.fused = fused
        self.fuse_kv_write = fuse_kv_write and fused and not literal
        self.holder_free = holder_free and self.fuse_kv_write
        self.absorbed = absorbed and not literal
        self.attn = HybridAttentionImpl(num_heads, self.head_dim, self.scaling, kv_cache_dtype=kv_cache_dtype,
                                        literal=literal, prefill_attention=prefill_attention, k_scale=k_scale,
                                        v_scale=v_scale)

    def _forward_absorbed(self, hidden_states, kv_cache, hidden_cache, md: HybridAttentionMetadata):
        """Decode step without re-projection: hidden-cached sequences attend on their cached hidden rows
        (projection weights absorbed), K/V-cached sequences on their private cache."""
        w, b = self.qkv_proj.weight, self.qkv_proj.bias
        s = w.shape[0] // 3
        H, D = self.num_heads, self.head_dim
        a = self.attn
        n_kv = md.num_decode_tokens - md.num_hidden_cache_tokens
        attn_output = torch.empty_like(hidden_states)
        # The step's cache writes - the newest hidden row of every hidden-cached sequence, the newest K and V rows of
        # the others - are planned here and launched by the attention call (beside the absorbed queries when the
        # step is small).  An fp8 K/V cache takes the quantising write instead, and the hidden rows a launch of
        # their own.
        one_write = not a.fp8 and (not n_kv or (md.kv_cache_use_input is not None and md.new_token_slot is not None))
        store_job = None
        if not one_write:
            with phase("write"):
                ops.hidden_to_cache(hidden_states, hidden_cache, md.slot_mapping, md.hidden_cache_use_input,
                                    md.hidden_cache_store_tot)
        if n_kv:
            with phase("projections"):
                qkv, _ = self.qkv_proj(hidden_states)
                q, k, v = qkv.chunk(chunks=3, dim=-1)
            if one_write:
                store_job = ops.decode_step_cache_ops(None, hidden_states, hidden_cache, None, md.slot_mapping,
                                                      md.hidden_cache_use_input, md.hidden_cache_store_tot, k, v,
                                                      md.kv_cache_use_input, md.new_token_slot,
                                                      kv_cache=kv_cache, as_job=True)
            else:
                with phase("write"):
                    ops.reshape_and_cache_flash(k, v, kv_cache[0], kv_cache[1], md.new_token_slot, a.kv_cache_dtype,
                                                a.k_scale, a.v_scale, token_idx=md.kv_cache_use_input)
            # planned here, launched by the attention on the hidden rows (the two halves write different rows of
            # attn_output; a small batch runs them in one launch)
            kv_job = ops.paged_decode_attention(q.view(-1, H, D), kv_cache[0], kv_cache[1], md.private_block_tables,
                                                md.kv_seq_lens, self.scaling, max_seq_len=md.max_kv_seq_len or None,
                                                out=attn_output.view(-1, H, D), k_scale=a.k_scale,
                                                v_scale=a.v_scale, as_job=True)
        else:
            kv_job = None
            with phase("projections"):
                q, _ = self.qkv_proj(hidden_states, q_only=True, kv_only=False)
            if one_write:
                store_job = ops.decode_step_cache_ops(None, hidden_states, hidden_cache, None, md.slot_mapping,
                                                      md.hidden_cache_use_input, md.hidden_cache_store_tot, None, None,
                                                      None, None, as_job=True)
        with phase("attention_on_hidden_rows"):
            ops.absorbed_hidden_attention(q, hidden_cache, md.hidden_slots, md.hidden_seq_start,
                                          md.hidden_cache_use_input, md.max_hidden_seq_len, w[s:2 * s], w[2 * s:],
                                          None if b is None else b[2 * s:], self.scaling, attn_output, kv_job=kv_job,
                                          store_job=store_job)
        with phase("projections"):
            return ops.linear_nt(attn_output, self.out_weight, self.out_bias)

    def forward(self, hidden_states, kv_cache, shared_cache, attn_metadata: HybridAttentionMetadata,
                hidden_cache=None):
        """``hidden_cache``: where hidden rows are cached when it is not ``kv_cache`` itself — a separate
        ``(2, N, BS, H, D)`` tensor in the activation dtype, needed with an fp8 K/V cache (whose bytes cannot hold
        16-bit hidden rows)."""
        md = attn_metadata
        hc = kv_cache if hidden_cache is None else hidden_cache
        same = kv_cache is not None and kv_cache.dtype == hidden_states.dtype      # K/V cached in the activation dtype
        fp8 = self.attn.fp8
        if fp8 and md.num_hidden_cache_tokens != 0 and (hidden_cache is None or hidden_cache.dtype != hidden_states.dtype):
            raise ValueError("an fp8 K/V cache cannot hold hidden rows: pass hidden_cache in the activation dtype")
        if md.num_hidden_cache_tokens != 0:
            if (self.absorbed and md.num_decode_tokens != 0 and md.hidden_slots is not None and kv_cache is not None
                    and hc.dtype == hidden_states.dtype):
                return self._forward_absorbed(hidden_states, kv_cache, hc, md)
            if md.num_decode_tokens != 0:
                if (self.holder_free and md.holder_src is not None and md.kv_dest is not None and same
                        and md.num_tot_tokens > 48):   # fewer rows: the weight-streaming kernels on a holder
                    with phase("write"):
                        ops.hidden_to_cache(hidden_states, hc, md.slot_mapping, md.hidden_cache_use_input,
                                            md.hidden_cache_store_tot)
                    with phase("projections"):
                        q, _ = self.qkv_proj(hidden_states, q_only=True, kv_only=False)
                    w, b = self.qkv_proj.weight, self.qkv_proj.bias
                    s = w.shape[0] // 3
                    with phase("kv_gemm"):
                        ops.kv_reproject_gathered(hidden_states, hc, md.holder_src, w[s:],
                                                  None if b is None else b[s:], shared_cache[0], shared_cache[1],
                                                  kv_cache[0], kv_cache[1], md.kv_dest)
                    with phase("attention"):
                        attn_output = self.attn.forward(q, None, None, kv_cache, shared_cache, md, kv_written=True)
                    with phase("projections"):
                        return ops.linear_nt(attn_output, self.out_weight, self.out_bias)
                if self.fused and md.holder_src is not None:
                    holder = torch.empty(md.num_tot_tokens, hidden_states.shape[1], device=hidden_states.device,
                                         dtype=hidden_states.dtype)
                    with phase("gather"):
                        ops.gather_hidden_rows(holder, hidden_states, hc, md.holder_src, md.slot_mapping,
                                               md.hidden_cache_use_input, md.hidden_cache_store_tot)
                else:                                                               # aptserve_opt.py:108-121
                    ops.hidden_to_cache(hidden_states, hc, md.slot_mapping, md.hidden_cache_use_input,
                                        md.hidden_cache_store_tot)
                    holder = torch.zeros(md.num_tot_tokens, hidden_states.shape[1], device=hidden_states.device,
                                         dtype=hidden_states.dtype)
                    holder[md.hidden_holder_upd] = hidden_states
                    ops.cache_to_hidden(holder, hc, md.slot_mapping, md.hidden_cache_use_tot)
                with phase("projections"):
                    q, _ = self.qkv_proj(hidden_states, q_only=True, kv_only=False)
                if self.fuse_kv_write and md.kv_dest is not None and same:
                    w, b = self.qkv_proj.weight, self.qkv_proj.bias
                    s = w.shape[0] // 3
                    with phase("kv_gemm"):
                        ops.kv_reproject_to_cache(holder, w[s:], None if b is None else b[s:], shared_cache[0],
                                                  shared_cache[1], kv_cache[0], kv_cache[1], md.kv_dest)
                    with phase("attention"):
                        attn_output = self.attn.forward(q, None, None, kv_cache, shared_cache, md, kv_written=True)
                    with phase("projections"):
                        return ops.linear_nt(attn_output, self.out_weight, self.out_bias)
                else:
                    kv, _ = self.qkv_proj(holder, q_only=False, kv_only=True)
                    k, v = kv.chunk(chunks=2, dim=-1)
            elif self.fuse_kv_write and md.token_is_hidden is not None and kv_cache is not None and (same or fp8):
                qkv, _ = self.qkv_proj(hidden_states)
                q, k, v = qkv.chunk(chunks=3, dim=-1)
                # hidden rows of hidden-cached prompts and K/V rows of the others, one launch (two with fp8:
                # the byte move of the hidden rows and the quantising write of the K/V rows)
                ops.mixed_reshape_and_cache(k, v, hidden_states, kv_cache, md.slot_mapping, md.token_is_hidden,
                                            self.attn.kv_cache_dtype, self.attn.k_scale, self.attn.v_scale,
                                            hidden_cache=hidden_cache)
                attn_output = self.attn.forward(q, k, v, kv_cache, shared_cache, md, kv_written=True)
                return ops.linear_nt(attn_output, self.out_weight, self.out_bias)
            else:                                                                   # :125-127
                ops.hidden_to_cache(hidden_states, hc, md.slot_mapping, md.hidden_cache_use_input,
                                    md.hidden_cache_store_tot)
                qkv, _ = self.qkv_proj(hidden_states)
                q, k, v = qkv.chunk(chunks=3, dim=-1)
        else:                                                                       # :128-130
            qkv, _ = self.qkv_proj(hidden_states)
            q, k, v = qkv.chunk(chunks=3, dim=-1)
        attn_output = self.attn.forward(q, k, v, kv_cache, shared_cache, md)
        return ops.linear_nt(attn_output, self.out_weight, self.out_bias)

    __call__ = forward


def promote_hidden_to_kv(qkv_weight, qkv_bias, kv_cache, hidden_slots, kv_slots) -> None:
    """Turn hidden-cached rows of one layer into K/V-cached rows without a re-prefill: the rows at
    ``hidden_slots`` (slots of the flattened cache) are re-projected once and written to the K/V slots
    ``kv_slots`` of the same layer cache.  The reference has no such transition: it changes a sequence's
    cache type by preempting it in recompute mode
    (additional_designs/core/aptserve_scheduler.py:748-755).  The opposite direction does not exist
    (hidden states cannot be recovered from K/V).  Source and destination blocks must not overlap."""
    n = hidden_slots.numel()
    if n == 0:
        return
    hd = kv_cache.size(3) * kv_cache.size(4)
    rows = torch.empty(n, hd, dtype=kv_cache.dtype, device=kv_cache.device)
    idx = torch.arange(n, dtype=torch.int64, device=kv_cache.device)
    ops.cache_to_hidden(rows, kv_cache, hidden_slots, idx)
    s = qkv_weight.shape[0] // 3
    ops.kv_reproject_to_cache(rows, qkv_weight[s:], None if qkv_bias is None else qkv_bias[s:], None, None,
                              kv_cache[0], kv_cache[1], -(kv_slots + 2))

