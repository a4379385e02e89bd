"""Helpers shared by the tests (not collected by pytest)."""
from __future__ import annotations

import numpy as np
import torch

from oracle.metadata import SeqRecord, build_metadata


def records_of(batch):
    return [SeqRecord(is_prompt=batch.is_prompt, use_hidden=h, seq_len=l, context_len=c,
                      block_table=bt, block_table_4_shared=bts)
            for l, c, h, bt, bts in zip(batch.seq_lens, batch.context_lens, batch.use_hidden,
                                        batch.block_tables, batch.block_tables_4_shared)]


def oracle_metadata(batch):
    return build_metadata(records_of(batch), batch.block_size)


def t64(a, device="cpu"):
    return torch.as_tensor(np.asarray(a, dtype=np.int64), device=device)


def randn(shape, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def sentinel_cache(shape, dtype=torch.float16, seed=1234):
    """A cache pre-filled with a non-trivial pattern so untouched slots are detectable."""
    g = torch.Generator().manual_seed(seed)
    n = int(np.prod(shape))
    bits = torch.randint(0, 0x3C00, (n,), generator=g, dtype=torch.int32).to(torch.int16)
    if dtype in (torch.float16, torch.bfloat16):
        return bits.view(dtype).reshape(shape).clone()
    if dtype == torch.float32:
        return bits.to(torch.float32).reshape(shape)
    if dtype == torch.float64:
        return bits.to(torch.float64).reshape(shape)
    if dtype == torch.uint8:
        return (bits & 0x7E).to(torch.uint8).reshape(shape)
    raise ValueError(dtype)


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    a, b = a.cpu().contiguous(), b.cpu().contiguous()
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))
