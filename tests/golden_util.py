"""Loaders for the committed fixtures (shared by the CPU and GPU golden tests)."""
from pathlib import Path

import numpy as np
import torch

G = Path(__file__).resolve().parent / "golden"


def load(name):
    return np.load(G / name, allow_pickle=False)


def f16(a):
    return torch.from_numpy(np.ascontiguousarray(a)).view(torch.float16)


def tables_of(z, prefix):
    bt = [list(map(int, r[:n])) for r, n in zip(z[f"{prefix}_in_tables"], z[f"{prefix}_in_table_lens"])]
    bts = [list(map(int, r[:n])) for r, n in zip(z[f"{prefix}_in_shared"], z[f"{prefix}_in_shared_lens"])]
    return bt, bts


META_TENSORS = ["slot_mapping", "slot_mapping_shared", "hidden_cache_use_tot", "kv_cache_use_tot",
                "hidden_cache_use_input", "hidden_cache_store_tot", "hidden_holder_upd", "hidden_holder_pull",
                "seq_lens_tensor", "context_lens_tensor", "query_start_loc", "seq_start_loc", "block_tables",
                "input_positions"]
META_SCALARS = ["num_prefills", "num_prefill_tokens", "num_decode_tokens", "num_tot_tokens",
                "num_hidden_cache_tokens", "max_query_len", "max_prefill_seq_len", "max_decode_seq_len"]
