"""Seeded synthetic batches of the shapes the benchmark configurations name.

Only data generation lives here (lengths, cache-type flags, block tables laid
out the way the reference's block manager numbers blocks); index tensors are
derived from a batch by the metadata builder.

Block numbering (additional_designs/core/aptserve_block_manager.py:176-192,
:530-541, :744-749): private blocks are ``0..N-1``; a hidden-cached sequence
takes a new private block ``p`` for every even logical block and ``p + N`` (the
V half of the same physical block) for the following odd one; its per-step
K/V workspace blocks come from the shared pool ``N..2N-1``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List

import numpy as np

OPT_125M = dict(num_heads=12, head_size=64, hidden_size=768)
OPT_13B = dict(num_heads=40, head_size=128, hidden_size=5120)
BLOCK_SIZE = 16


@dataclass
class Batch:
    """One homogeneous batch (all prompts or all decodes), host-side description."""
    is_prompt: bool
    block_size: int
    num_blocks: int                      # N: private blocks per layer
    seq_lens: List[int]
    use_hidden: List[bool]
    block_tables: List[List[int]]
    block_tables_4_shared: List[List[int]] = field(default_factory=list)

    @property
    def context_lens(self) -> List[int]:
        return [0 if self.is_prompt else l - 1 for l in self.seq_lens]

    def packed_tables(self):
        """The block tables as 0-padded int32 ``[batch, width]`` arrays (built once, then kept): the form a
        block manager that updates its tables in place would hand to the metadata builder."""
        if getattr(self, "_packed", None) is None:
            def pack(tables):
                w = max((len(t) for t in tables), default=0)
                out = np.zeros((len(self.seq_lens), w), dtype=np.int32)
                for b, t in enumerate(tables):
                    out[b, :len(t)] = t
                return out
            shared = self.block_tables_4_shared or [[] for _ in self.seq_lens]
            self._packed = (pack(self.block_tables), pack(shared))
            self.seq_lens_np = np.asarray(self.seq_lens, dtype=np.int64)
            self.use_hidden_np = np.asarray(self.use_hidden, dtype=bool)
        return self._packed


def lognormal_lengths(rng: np.random.Generator, n: int, mu: float = 6.2, sigma: float = 0.8,
                      lo: int = 16, hi: int = 2048) -> np.ndarray:
    return np.clip(np.rint(rng.lognormal(mu, sigma, n)), lo, hi).astype(np.int64)


def pick_hidden(rng: np.random.Generator, n: int, fraction: float) -> np.ndarray:
    """Exactly ``round(fraction*n)`` sequences, chosen without replacement."""
    flags = np.zeros(n, dtype=bool)
    k = int(round(fraction * n))
    if k:
        flags[rng.choice(n, k, replace=False)] = True
    return flags


def allocate_blocks(rng: np.random.Generator, seq_lens, use_hidden, num_blocks: int, block_size: int,
                    is_prompt: bool) -> Batch:
    free_private = list(rng.permutation(num_blocks))
    free_shared = list(rng.permutation(num_blocks) + num_blocks)
    tables, shared_tables = [], []
    for length, hid in zip(seq_lens, use_hidden):
        nblk = -(-int(length) // block_size)
        table: List[int] = []
        if hid:
            for i in range(nblk):
                table.append(int(free_private.pop()) if i % 2 == 0 else table[-1] + num_blocks)
            shared_tables.append([int(free_shared.pop()) for _ in range(nblk)])
        else:
            table = [int(free_private.pop()) for _ in range(nblk)]
            shared_tables.append([])
        tables.append(table)
    return Batch(is_prompt=is_prompt, block_size=block_size, num_blocks=num_blocks,
                 seq_lens=[int(x) for x in seq_lens], use_hidden=[bool(x) for x in use_hidden],
                 block_tables=tables, block_tables_4_shared=shared_tables)


def mixed_write_opt125m(seed: int = 0) -> Batch:
    """8 prompts with lengths uniform in [1,128], 512-block pool, 30 % hidden-cached."""
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, 129, 8)
    hid = pick_hidden(rng, 8, 0.3)
    return allocate_blocks(rng, lens, hid, 512, BLOCK_SIZE, is_prompt=True)


def decode_batch_opt13b(seed: int = 0, batch: int = 256, hidden_fraction: float = 0.5,
                        num_blocks: int | None = None, hi: int = 2048) -> Batch:
    """Decode step: ``batch`` sequences, lognormal(6.2, 0.8) lengths clipped to [16, hi]."""
    rng = np.random.default_rng(seed)
    lens = lognormal_lengths(rng, batch, hi=hi)
    hid = pick_hidden(rng, batch, hidden_fraction)
    need = int(sum(-(-int(l) // BLOCK_SIZE) for l in lens))
    if num_blocks is None:
        num_blocks = max(64, need + need // 4)
    return allocate_blocks(rng, lens, hid, num_blocks, BLOCK_SIZE, is_prompt=False)


def small_decode_batch(seed: int, batch: int, max_len: int, hidden_fraction: float, num_blocks: int,
                       block_size: int = BLOCK_SIZE) -> Batch:
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, max_len + 1, batch)
    hid = pick_hidden(rng, batch, hidden_fraction)
    return allocate_blocks(rng, lens, hid, num_blocks, block_size, is_prompt=False)


def small_prefill_batch(seed: int, batch: int, max_len: int, hidden_fraction: float, num_blocks: int,
                        block_size: int = BLOCK_SIZE) -> Batch:
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, max_len + 1, batch)
    hid = pick_hidden(rng, batch, hidden_fraction)
    return allocate_blocks(rng, lens, hid, num_blocks, block_size, is_prompt=True)
