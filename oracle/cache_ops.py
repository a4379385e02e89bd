"""Oracle for the cache scatter/gather operators (test infrastructure only).

All functions mutate their destination in place and return ``None`` like the
reference operators.  Tensors are CPU tensors.  Index tensors are int64.

The addressing model used throughout: a paged cache of shape
``(2, N, BS, H, D)`` is contiguous, so "slot ``s``" of the flattened
``2*N*BS`` slots starts ``s * stride(2)`` elements after the base pointer.
Slots ``>= N*BS`` therefore live in plane 1 (the V plane); that is how a
hidden block numbered ``p + N`` addresses the V half of physical block ``p``
(reference: additional_designs/core/aptserve_block_manager.py:530-541).
"""

from __future__ import annotations

import torch


def _slot_rows(paged_cache: torch.Tensor, width: int) -> torch.Tensor:
    """View of the cache as ``[num_slots, width]`` rows spaced ``stride(2)`` apart.

    Follows additional_designs/mixed_cache_kernels/mixed_cache.cu:129 where the
    slot stride is taken from ``paged_cache.stride(2)`` and element ``i`` of slot
    ``s`` is at flat offset ``s*slot_stride + i`` (``:47-50``).
    """
    assert paged_cache.dim() == 5 and paged_cache.is_contiguous()
    slot_stride = paged_cache.stride(2)
    num_slots = paged_cache.numel() // slot_stride
    assert width <= slot_stride
    return paged_cache.as_strided((num_slots, width), (slot_stride, 1))


def hidden_to_cache(hidden, paged_cache, slot_mapping, src_idx, target_slot_idx) -> None:
    """Scatter rows of ``hidden`` into hidden-cache slots.

    Reference: mixed_cache.cu:31-53 (kernel), :119-147 (launcher).
    For every ``b``: ``tok = src_idx[b]``, ``slot = slot_mapping[target_slot_idx[b]]``;
    a negative slot is skipped; otherwise the ``hidden.size(1)`` elements of row
    ``tok`` are stored at the slot.
    """
    if src_idx.numel() == 0:
        return
    slots = slot_mapping[target_slot_idx]
    keep = slots >= 0
    rows = _slot_rows(paged_cache, hidden.size(1))
    rows.index_put_((slots[keep],), hidden[src_idx[keep]])


def cache_to_hidden(hidden, paged_cache, slot_mapping, dst_idx) -> None:
    """Gather hidden-cache slots back into rows of ``hidden``.

    Reference: mixed_cache.cu:6-28 (kernel), :150-176 (launcher).
    For every ``b``: ``tok = dst_idx[b]``, ``slot = slot_mapping[tok]``; negative
    slots are skipped; otherwise ``hidden[tok, :] = cache_flat[slot, :]``.
    """
    if dst_idx.numel() == 0:
        return
    slots = slot_mapping[dst_idx]
    keep = slots >= 0
    rows = _slot_rows(paged_cache, hidden.size(1))
    hidden.index_put_((dst_idx[keep],), rows.index_select(0, slots[keep]))


def _kv_rows(cache: torch.Tensor) -> torch.Tensor:
    """``[num_blocks, BS, H, D]`` cache as ``[num_blocks*BS, H*D]`` slot rows.

    The target element of (slot, head, d) is
    ``(slot//BS)*block_stride + (slot%BS)*H*D + head*D + d``
    (mixed_cache.cu:96-106); expressed here as a strided 3-D view indexed by
    ``(slot//BS, slot%BS)`` so a padded ``block_stride`` is honoured.
    """
    nb, bs, h, d = cache.shape
    assert cache.stride(3) == 1 and cache.stride(2) == d and cache.stride(1) == h * d
    return cache.as_strided((nb, bs, h * d), (cache.stride(0), h * d, 1))


def _store_rows(cache, slots, src) -> None:
    keep = slots >= 0
    s = slots[keep]
    if s.numel() == 0:          # every slot is padding: nothing is stored
        return
    bs = cache.size(1)
    _kv_rows(cache).index_put_((s // bs, s % bs), src[keep].reshape(int(keep.sum()), -1))


def reshape_and_cache_flash(key, value, key_cache, value_cache, slot_mapping,
                            kv_cache_dtype: str = "auto", k_scale: float = 1.0,
                            v_scale: float = 1.0) -> None:
    """K/V scatter by ``slot_mapping`` into ``[num_blocks, BS, H, D]`` caches.

    The operator itself is third-party (vLLM 0.5.0.post1,
    ``csrc/cache_kernels.cu: reshape_and_cache_flash_kernel``; not under the
    reference tree).  Its published behaviour, anchored on the reference's call
    sites additional_designs/attention/backends/aptserve_flash_attn.py:338-345,
    :348-355, :378-385: token ``t`` goes to
    ``cache[slot//BS, slot%BS, :, :]``; ``slot < 0`` is padding and skipped.

    ``kv_cache_dtype == "fp8"`` (not in the reference, which asserts
    ``kv_scale == 1.0`` at aptserve_flash_attn.py:311-312) stores
    ``e4m3fn(clamp(x / scale, +-448))`` as raw bytes in a uint8 cache.
    """
    if slot_mapping.numel() == 0:
        return
    if kv_cache_dtype in ("fp8", "fp8_e4m3"):
        from .fp8 import quantize_e4m3
        key = quantize_e4m3(key, k_scale)
        value = quantize_e4m3(value, v_scale)
    else:
        assert kv_cache_dtype == "auto"
    n = slot_mapping.numel()
    _store_rows(key_cache, slot_mapping, key[:n])
    _store_rows(value_cache, slot_mapping, value[:n])


def mixed_reshape_and_cache(key, value, hidden, paged_cache, slot_mapping, is_hidden) -> None:
    """The two writes of a prompt step with hidden-cached sequences, as the reference issues them:
    ``hidden_to_cache`` over the tokens of hidden-cached prompts
    (additional_designs/model_executor/models/aptserve_opt.py:125-126) and
    ``reshape_and_cache_flash`` over gathered copies of the other tokens
    (additional_designs/attention/backends/aptserve_flash_attn.py:347-355).  Pinned through the
    two functions it composes."""
    mask = torch.as_tensor(is_hidden).bool()
    hid_idx = torch.nonzero(mask).flatten()
    kv_idx = torch.nonzero(~mask).flatten()
    if hidden is not None:
        hidden_to_cache(hidden, paged_cache, slot_mapping, hid_idx, hid_idx)
    if key is not None:
        reshape_and_cache_flash(key[kv_idx], value[kv_idx], paged_cache[0], paged_cache[1], slot_mapping[kv_idx])


def mixed_kv_to_cache(key, value, k_cache, v_cache, shared_k_cache, shared_v_cache,
                      slot_mapping, slot_mapping_shared, kv_cache_use_tot,
                      hidden_cache_use_tot, literal_modulo: bool = False) -> None:
    """Three-range K/V scatter of a mixed decode batch.

    Reference: mixed_cache.cu:56-116 (kernel), :179-230 (launcher).  The grid is
    ``2*nkv + nh`` blocks, ``nkv = len(kv_cache_use_tot)``,
    ``nh = len(slot_mapping_shared)``:

    * range A, ``blk < nkv``: ``tok = kv_cache_use_tot[blk]``,
      ``slot = slot_mapping[tok]`` -> private ``k_cache`` / ``v_cache``;
    * range B, ``nkv <= blk < 2*nkv``: same token and slot -> shared caches;
    * range C, ``blk >= 2*nkv``: ``off`` -> ``tok = hidden_cache_use_tot[off]``,
      ``slot = slot_mapping_shared[off]`` -> shared caches.

    ``off`` is ``blk - 2*nkv`` (the intended meaning).  The reference computes
    ``blk % (2*nkv)`` (``:88``), which is the same number only while
    ``nh <= 2*nkv``; ``literal_modulo=True`` reproduces that arithmetic (and,
    like the reference, is undefined for ``nkv == 0``).
    """
    nkv = int(kv_cache_use_tot.numel())
    nh = int(slot_mapping_shared.numel())
    if nkv:
        tok = kv_cache_use_tot
        slots = slot_mapping[tok]
        _store_rows(k_cache, slots, key[tok])
        _store_rows(v_cache, slots, value[tok])
        _store_rows(shared_k_cache, slots, key[tok])
        _store_rows(shared_v_cache, slots, value[tok])
    if nh:
        if literal_modulo:
            assert nkv > 0, "blk % 0 is undefined in the reference as well"
            off = (torch.arange(nh, dtype=torch.int64) + 2 * nkv) % (2 * nkv)
            # Later grid blocks may overwrite earlier ones at the same slot; the
            # data are identical for equal offsets, so order is immaterial.
        else:
            off = torch.arange(nh, dtype=torch.int64)
        tok = hidden_cache_use_tot[off]
        slots = slot_mapping_shared[off]
        _store_rows(shared_k_cache, slots, key[tok])
        _store_rows(shared_v_cache, slots, value[tok])


def assemble_hidden_holder(hidden_states, paged_cache, slot_mapping, num_tot_tokens,
                           hidden_holder_upd, hidden_cache_use_tot) -> torch.Tensor:
    """The decode-side holder of every row that is re-projected.

    Reference: additional_designs/model_executor/models/aptserve_opt.py:112-121 —
    ``zeros(num_tot, Hd)``; ``holder[upd] = hidden_states``; then
    ``cache_to_hidden(holder, cache, slot_mapping, hidden_cache_use_tot)``.
    """
    holder = torch.zeros(num_tot_tokens, hidden_states.size(1), dtype=hidden_states.dtype)
    holder[hidden_holder_upd] = hidden_states
    cache_to_hidden(holder, paged_cache, slot_mapping, hidden_cache_use_tot)
    return holder
