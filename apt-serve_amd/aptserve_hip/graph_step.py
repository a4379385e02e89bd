"""Decode steps of the OPT decoder on the hybrid cache, replayed from HIP graphs.

A decode step of OPT-13B is ~600 launches of a few microseconds each; issued one by one from Python the host needs
6-7 ms to enqueue a step that the GPU finishes in little more.  The operators launch on the caller's stream,
allocate nothing of their own and take every ragged quantity (rows per sequence, slots, tile lists) from device
memory; what they take from the host is fixed by a step's *shape class*: the batch size, the number of
hidden-cached sequences and an upper bound of the sequence lengths.  ``DecodeGraphRunner`` keeps one recorded
graph per shape class (lengths bucketed to ``len_bucket`` tokens, so a class lasts for that many steps of a stable
batch), builds each step's metadata into the class's persistent buffers (``metadata.StaticDecodeBuffers``: the
builder's upload and its one kernel stay outside the graph) and replays.  The data flow is the one in which
hidden-cached sequences attend on their cached hidden rows (``absorbed=True``): in the re-projection flow the
row count of the K/V product changes with every step, which a recorded launch cannot follow.

The graph ends at the decoder's final LayerNorm; the logits product and the argmax stay outside (library
reductions may record memset nodes, which this runtime replays unreliably).

Mirrors what ``CUDAGraphRunner`` does for the reference's stock decode path
(additional_designs/worker/aptserve_model_runner.py:1161-1260, which never passes ``shared_cache`` and is
therefore not usable with hidden-cached sequences there).
"""

from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from . import metadata


class _Recorded:
    __slots__ = ("buffers", "graph", "ids", "hidden", "md", "replays")


class DecodeGraphRunner:
    def __init__(self, model, kv_caches: List[torch.Tensor], shared_cache, block_size: int, device,
                 len_bucket: int = 256, max_graphs: int = 16) -> None:
        if len_bucket % block_size:
            raise ValueError("len_bucket must be a whole number of blocks")
        self.model, self.kv_caches, self.shared_cache = model, kv_caches, shared_cache
        self.block_size, self.device = block_size, torch.device(device)
        self.len_bucket, self.max_graphs = len_bucket, max_graphs
        self.recorded: Dict[Tuple[int, int, int], _Recorded] = {}
        self.stream = torch.cuda.Stream(self.device)     # default priority; captures run on it
        self.captures = 0

    def _key(self, seq_lens: Sequence[int], use_hidden: Sequence[bool]) -> Tuple[int, int, int]:
        cap = -(-max(seq_lens) // self.len_bucket) * self.len_bucket
        return len(seq_lens), int(sum(bool(h) for h in use_hidden)), cap

    def _record(self, key, seq_lens, use_hidden, block_tables, shared_tables, ids: torch.Tensor) -> _Recorded:
        B, n_hidden, cap = key
        if len(self.recorded) >= self.max_graphs:        # oldest class goes (its graph and its buffers)
            self.recorded.pop(next(iter(self.recorded)))
        rec = _Recorded()
        rec.buffers = metadata.StaticDecodeBuffers(B, n_hidden, cap, self.block_size, self.device)
        rec.md = metadata.build_metadata(False, seq_lens, use_hidden, block_tables, shared_tables, self.block_size,
                                         self.device, static=rec.buffers)
        rec.ids = ids.clone()
        cur = torch.cuda.current_stream(self.device)
        self.stream.wait_stream(cur)
        with torch.cuda.stream(self.stream):
            # one eager pass on the capture stream first: one-time set-up (kernel attributes, workspace sizes)
            # must not fall into the capture.  It computes this step for real, and the replay below computes it
            # again: same inputs, same cache slots, same values.
            self.model(rec.ids, rec.md.input_positions, self.kv_caches, self.shared_cache, rec.md)
        cur.wait_stream(self.stream)
        torch.cuda.synchronize(self.device)
        rec.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(rec.graph, stream=self.stream):
            rec.hidden = self.model(rec.ids, rec.md.input_positions, self.kv_caches, self.shared_cache, rec.md)
        rec.replays = 0
        self.captures += 1
        self.recorded[key] = rec
        return rec

    def prepare(self, seq_lens: Sequence[int], use_hidden: Sequence[bool], block_tables, shared_tables,
                input_ids: torch.Tensor) -> _Recorded:
        """Host side of a decode step: the step's metadata and token ids into the persistent buffers of its
        shape class (recording the class's graph first if this is its first step)."""
        key = self._key(seq_lens, use_hidden)
        rec = self.recorded.get(key)
        if rec is None:
            return self._record(key, seq_lens, use_hidden, block_tables, shared_tables, input_ids)
        rec.md = metadata.build_metadata(False, seq_lens, use_hidden, block_tables, shared_tables,
                                         self.block_size, self.device, static=rec.buffers)
        rec.ids.copy_(input_ids, non_blocking=True)
        return rec

    def run(self, rec: _Recorded):
        """Replay the step; returns ``(hidden_states, metadata)``.  ``hidden_states`` is the graph's output
        buffer: read it (or copy it) before the next step of the same shape class."""
        rec.graph.replay()
        rec.replays += 1
        return rec.hidden, rec.md

    def step(self, seq_lens, use_hidden, block_tables, shared_tables, input_ids: torch.Tensor):
        return self.run(self.prepare(seq_lens, use_hidden, block_tables, shared_tables, input_ids))
