"""Pins the metadata oracle: the invariants the reference's own (commented) checks
list at aptserve_model_runner.py:676-695, plus a brute-force rebuild from an
independent per-row definition on small batches."""
import numpy as np
import pytest

from aptserve_hip import workloads
from util import oracle_metadata


def rows_by_definition(batch):
    """Per-row table (sequence, position, is_last, hidden) built directly from the
    meaning of the 'tot' row space, without the reference's list bookkeeping."""
    rows = []
    for b, (L, h) in enumerate(zip(batch.seq_lens, batch.use_hidden)):
        if batch.is_prompt:
            rows += [(b, j, False, h) for j in range(L)]
        elif h:
            rows += [(b, j, j == L - 1, True) for j in range(L)]
        else:
            rows.append((b, L - 1, True, False))
    return rows


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("frac", [0.0, 0.3, 0.5, 1.0])
def test_decode_metadata_invariants_and_brute_force(seed, frac):
    bs = 16
    batch = workloads.small_decode_batch(seed, 4, 50, frac, 32, bs)
    md = oracle_metadata(batch)
    B = len(batch.seq_lens)
    # invariants listed by the reference
    assert len(md["hidden_cache_use_tot"]) + len(md["kv_cache_use_tot"]) == md["num_tot_tokens"] == len(md["slot_mapping"])
    assert len(md["hidden_holder_upd"]) == md["num_decode_tokens"] == B
    assert len(md["hidden_holder_upd"]) + len(md["hidden_holder_pull"]) == md["num_tot_tokens"]
    assert len(md["slot_mapping_shared"]) == len(md["hidden_cache_use_tot"])
    assert len(md["slot_mapping_shared"]) == len(md["hidden_holder_pull"]) + md["num_hidden_cache_tokens"]
    for k in ("hidden_cache_use_tot", "kv_cache_use_tot", "hidden_holder_upd", "hidden_holder_pull",
              "hidden_cache_use_input", "hidden_cache_store_tot"):
        assert np.all(np.diff(md[k]) > 0), k
        assert md[k].dtype == np.int64
    # brute force
    rows = rows_by_definition(batch)
    assert len(rows) == md["num_tot_tokens"]
    for r, (b, j, last, h) in enumerate(rows):
        assert md["slot_mapping"][r] == batch.block_tables[b][j // bs] * bs + j % bs
        assert (r in md["hidden_cache_use_tot"]) == h and (r in md["kv_cache_use_tot"]) == (not h)
        assert (r in md["hidden_holder_upd"]) == last and (r in md["hidden_holder_pull"]) == (not last)
        assert (r in md["hidden_cache_store_tot"]) == (h and last)
    hidden_rows = [(b, j) for (b, j, _, h) in rows if h]
    for i, (b, j) in enumerate(hidden_rows):
        assert md["slot_mapping_shared"][i] == batch.block_tables_4_shared[b][j // bs] * bs + j % bs
    assert list(md["hidden_cache_use_input"]) == [b for b, h in enumerate(batch.use_hidden) if h]
    for b in range(B):
        t = batch.block_tables_4_shared[b] if batch.use_hidden[b] else batch.block_tables[b]
        assert list(md["block_tables"][b, :len(t)]) == t and not md["block_tables"][b, len(t):].any()
    assert md["block_tables"].dtype == np.int32 and md["seq_lens_tensor"].dtype == np.int32
    assert list(md["seq_start_loc"]) == [0] + list(np.cumsum(batch.seq_lens))
    assert list(md["query_start_loc"]) == list(range(B + 1))
    assert list(md["context_lens_tensor"]) == [l - 1 for l in batch.seq_lens]


@pytest.mark.parametrize("seed", range(4))
@pytest.mark.parametrize("frac", [0.0, 0.5, 1.0])
def test_prefill_metadata_brute_force(seed, frac):
    bs = 16
    batch = workloads.small_prefill_batch(seed, 5, 40, frac, 32, bs)
    md = oracle_metadata(batch)
    rows = rows_by_definition(batch)
    assert md["num_tot_tokens"] == md["num_prefill_tokens"] == len(rows) == sum(batch.seq_lens)
    assert md["num_prefills"] == len(batch.seq_lens) and md["num_decode_tokens"] == 0
    for r, (b, j, _, h) in enumerate(rows):
        assert md["slot_mapping"][r] == batch.block_tables[b][j // bs] * bs + j % bs
        assert (r in md["hidden_cache_use_input"]) == h and (r in md["kv_cache_use_tot"]) == (not h)
    assert md["hidden_cache_use_tot"] is md["hidden_cache_use_input"] is md["hidden_cache_store_tot"]
    assert len(md["hidden_holder_upd"]) == len(md["hidden_holder_pull"]) == len(md["slot_mapping_shared"]) == 0
    assert md["num_hidden_cache_tokens"] == sum(l for l, h in zip(batch.seq_lens, batch.use_hidden) if h)
    assert md["block_tables"].shape == (len(batch.seq_lens), 0)
    assert list(md["query_start_loc"]) == list(md["seq_start_loc"]) == [0] + list(np.cumsum(batch.seq_lens))
    assert list(md["input_positions"]) == [j for (_, j, _, _) in rows]


def test_hidden_blocks_alternate_between_the_k_and_v_planes():
    """Slot numbering contract (aptserve_block_manager.py:530-541): logical block 2k of a
    hidden sequence is private block p, 2k+1 is p+N, i.e. the same physical block's V half."""
    N = 64
    batch = workloads.small_decode_batch(3, 3, 70, 1.0, N)
    for t in batch.block_tables:
        for i in range(1, len(t), 2):
            assert t[i] == t[i - 1] + N and t[i - 1] < N
    for t in batch.block_tables_4_shared:
        assert all(N <= x < 2 * N for x in t)


def test_memory_profiling_run_gets_padding_slots():
    from oracle.metadata import SeqRecord, build_metadata
    md = build_metadata([SeqRecord(True, False, 7, 0, [], [])], 16)
    assert list(md["slot_mapping"]) == [-1] * 7 and md["num_tot_tokens"] == 0
