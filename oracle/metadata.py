"""Oracle for the ragged-batch metadata of the hybrid cache (test infrastructure only).

List-based restatement of the hybrid parts of ``ModelRunner._prepare_model_input``
(additional_designs/worker/aptserve_model_runner.py:240-842).  One record per
sequence stands in for a ``SequenceGroupMetadata`` with a single sequence:

    is_prompt, use_hidden, seq_len, context_len, block_table, block_table_4_shared

(``context_len`` is ``seq_len - 1`` in decode, ``:341``; 0 for a non-chunked
prompt, ``:336``.)  Sliding window, prefix caching, LoRA, multi-modal and
graph padding are outside the path and not restated.

Output fields, dtypes as the reference creates them:

* int64: ``slot_mapping`` (``:727-729``), ``slot_mapping_shared`` (``:731-733``),
  ``hidden_cache_use_tot``, ``kv_cache_use_tot``, ``hidden_cache_use_input``,
  ``hidden_cache_store_tot``, ``hidden_holder_upd``, ``hidden_holder_pull``
  (``:613-666``), ``input_positions`` (``:724-726``)
* int32: ``block_tables`` 0-padded (``:601-609``), ``seq_lens_tensor`` (``:707-709``),
  ``context_lens_tensor`` (``:772-774``), ``seq_start_loc`` (``:712-719``),
  ``query_start_loc`` (``:778-785``)
* Python ints: ``num_prefills, num_prefill_tokens, num_decode_tokens,
  num_tot_tokens, num_hidden_cache_tokens, max_query_len, max_prefill_seq_len,
  max_decode_seq_len``
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Sequence

import numpy as np

PAD_SLOT_ID = -1  # aptserve_model_runner.py:32


@dataclass
class SeqRecord:
    is_prompt: bool
    use_hidden: bool
    seq_len: int
    context_len: int
    block_table: List[int] = field(default_factory=list)
    block_table_4_shared: List[int] = field(default_factory=list)


def build_metadata(records: Sequence[SeqRecord], block_size: int) -> Dict[str, object]:
    slot_mapping: List[int] = []
    slot_mapping_shared: List[int] = []
    seq_lens: List[int] = []
    context_lens: List[int] = []
    query_lens: List[int] = []
    prefill_seq_lens: List[int] = []
    decode_seq_lens: List[int] = []
    block_tables: List[List[int]] = []
    input_positions: List[int] = []
    use_tot_flags: List[bool] = []      # hidden_cache_use_tot as the bool list of :299
    use_input_flags: List[bool] = []    # hidden_cache_use_input (:300)
    upd_flags: List[bool] = []          # hidden_holder_upd (:301)
    num_prefills = num_prefill_tokens = num_decode_tokens = num_tot_tokens = 0

    is_prompt = False
    for r in records:
        is_prompt = r.is_prompt  # the branch at :617 sees the last group's flag
        context_len, seq_len = r.context_len, r.seq_len
        # :410-432 — decode uses the shared table for hidden sequences, the
        # private one otherwise; a plain prompt has an empty table
        if not is_prompt:
            block_tables.append(list(r.block_table_4_shared if r.use_hidden else r.block_table))
        else:
            block_tables.append([])
        seq_lens.append(seq_len)
        context_lens.append(context_len)
        query_len = seq_len - context_len
        query_lens.append(query_len)
        input_positions.extend(range(context_len, seq_len))
        if is_prompt:
            num_prefills += 1
            num_prefill_tokens += query_len
            prefill_seq_lens.append(seq_len)
        else:
            assert query_len == 1
            num_decode_tokens += query_len
            decode_seq_lens.append(seq_len)

        if not r.block_table:  # memory-profiling run, :488-495
            slot_mapping.extend([PAD_SLOT_ID] * seq_len)
            continue

        bt, bts = r.block_table, r.block_table_4_shared
        for i in range(context_len, seq_len):  # :519
            if r.use_hidden:
                use_input_flags.append(True)
                if not is_prompt:  # :525-539
                    num_tot_tokens += seq_len
                    use_tot_flags.extend([True] * seq_len)
                    upd_flags.extend([False] * (seq_len - 1) + [True])
                    for j in range(seq_len):
                        slot_mapping_shared.append(bts[j // block_size] * block_size + j % block_size)
                        slot_mapping.append(bt[j // block_size] * block_size + j % block_size)
                else:  # :542-550
                    num_tot_tokens += 1
                    slot_mapping.append(bt[i // block_size] * block_size + i % block_size)
            else:  # :554-564
                num_tot_tokens += 1
                use_input_flags.append(False)
                if not is_prompt:
                    use_tot_flags.append(False)
                    upd_flags.append(True)
                slot_mapping.append(bt[i // block_size] * block_size + i % block_size)

    max_len = max((len(t) for t in block_tables), default=0)
    bt_arr = np.zeros((len(block_tables), max_len), dtype=np.int32)
    for i, t in enumerate(block_tables):
        bt_arr[i, :len(t)] = t

    use_input = np.asarray(use_input_flags, dtype=bool)
    idx_input = np.arange(len(use_input), dtype=np.int64)
    if not is_prompt:  # :617-645
        use_tot = np.asarray(use_tot_flags, dtype=bool)
        upd = np.asarray(upd_flags, dtype=bool)
        idx_tot = np.arange(len(use_tot), dtype=np.int64)
        store_tot = idx_tot[use_tot & upd]
        hidden_cache_use_tot = idx_tot[use_tot]
        kv_cache_use_tot = idx_tot[~use_tot]
        hidden_cache_use_input = idx_input[use_input]
        hidden_holder_upd = idx_tot[upd]
        hidden_holder_pull = idx_tot[~upd]
    else:  # :648-666
        kv_cache_use_tot = idx_input[~use_input]
        hidden_cache_use_input = idx_input[use_input]
        hidden_cache_use_tot = hidden_cache_use_input
        store_tot = hidden_cache_use_input
        hidden_holder_upd = np.zeros(0, dtype=np.int64)
        hidden_holder_pull = hidden_holder_upd

    seq_lens_arr = np.asarray(seq_lens, dtype=np.int32)
    query_lens_arr = np.asarray(query_lens, dtype=np.int64)
    seq_start_loc = np.zeros(len(seq_lens) + 1, dtype=np.int32)
    seq_start_loc[1:] = np.cumsum(seq_lens_arr, dtype=np.int32)
    query_start_loc = np.zeros(len(query_lens) + 1, dtype=np.int32)
    query_start_loc[1:] = np.cumsum(query_lens_arr, dtype=np.int32)

    return dict(
        num_prefills=num_prefills,
        num_prefill_tokens=num_prefill_tokens,
        num_decode_tokens=num_decode_tokens,
        num_tot_tokens=num_tot_tokens,
        num_hidden_cache_tokens=int(len(hidden_cache_use_input)),  # :668
        slot_mapping=np.asarray(slot_mapping, dtype=np.int64),
        slot_mapping_shared=np.asarray(slot_mapping_shared, dtype=np.int64),
        hidden_cache_use_tot=hidden_cache_use_tot,
        kv_cache_use_tot=kv_cache_use_tot,
        hidden_cache_use_input=hidden_cache_use_input,
        hidden_cache_store_tot=store_tot,
        hidden_holder_upd=hidden_holder_upd,
        hidden_holder_pull=hidden_holder_pull,
        seq_lens=list(seq_lens),
        seq_lens_tensor=seq_lens_arr,
        context_lens_tensor=np.asarray(context_lens, dtype=np.int32),
        query_start_loc=query_start_loc,
        seq_start_loc=seq_start_loc,
        input_positions=np.asarray(input_positions, dtype=np.int64),
        block_tables=bt_arr,
        max_query_len=max(query_lens) if query_lens else 0,
        max_prefill_seq_len=max(prefill_seq_lens, default=0),
        max_decode_seq_len=max(decode_seq_lens, default=0),
    )
