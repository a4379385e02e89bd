"""Host-only checks of the attention dispatcher (no GPU call is reached)."""
import pytest
import torch

from aptserve_hip.backend import HybridAttentionImpl
from aptserve_hip.metadata import HybridAttentionMetadata


def _prompt_metadata(context_len):
    e64 = torch.empty(0, dtype=torch.int64)
    lens = [8]
    return HybridAttentionMetadata(
        num_prefills=1, num_prefill_tokens=lens[0] - context_len, num_decode_tokens=0, num_hidden_cache_tokens=0,
        num_tot_tokens=lens[0] - context_len, slot_mapping=torch.arange(lens[0] - context_len), slot_mapping_shared=e64,
        hidden_cache_use_tot=e64, kv_cache_use_tot=torch.arange(lens[0] - context_len), hidden_cache_use_input=e64,
        hidden_cache_store_tot=e64, hidden_holder_upd=e64, hidden_holder_pull=e64, seq_lens=lens,
        seq_lens_tensor=torch.tensor(lens, dtype=torch.int32), max_query_len=lens[0] - context_len,
        max_prefill_seq_len=lens[0], max_decode_seq_len=0,
        query_start_loc=torch.tensor([0, lens[0] - context_len], dtype=torch.int32),
        seq_start_loc=torch.tensor([0, lens[0]], dtype=torch.int32),
        context_lens_tensor=torch.tensor([context_len], dtype=torch.int32),
        block_tables=torch.empty(1, 0, dtype=torch.int32), max_prompt_context_len=context_len)


def test_prefix_branch_without_a_cache_or_with_hidden_sequences_is_rejected_before_any_launch():
    """A prompt step that continues a cached prefix takes the prefix branch
    (additional_designs/attention/backends/aptserve_flash_attn.py:431-447), which reads K/V through the block
    tables: without a K/V cache and tables there is nothing to read (seq_start_loc counts whole sequences while
    q/k/v hold only the new tokens, so the plain prompt attention must not be used either), and a hidden-cached
    sequence keeps no K/V of its prefix."""
    impl = HybridAttentionImpl(2, 64, 0.125)
    md = _prompt_metadata(context_len=3)
    q = torch.zeros(5, 128, dtype=torch.float16)
    with pytest.raises(ValueError, match="prefix branch"):
        impl.forward(q, q, q, None, None, md)                       # no cache
    cache = torch.zeros(2, 4, 16, 2, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="prefix branch"):
        impl.forward(q, q, q, cache, None, md)                      # no block tables
    md.num_hidden_cache_tokens = 5
    with pytest.raises(ValueError, match="hidden-cached"):
        impl.forward(q, q, q, cache, None, md)


def test_constructor_rejects_what_the_reference_rejects():
    with pytest.raises(ValueError):
        HybridAttentionImpl(2, 64, 0.125, sliding_window=128)      # aptserve_flash_attn.py:277-282
    with pytest.raises(ValueError):
        HybridAttentionImpl(2, 48, 0.125)                          # unsupported head size
