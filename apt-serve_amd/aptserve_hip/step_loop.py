"""Synthetic single-GPU serving step loop over the hybrid cache.

A harness, not a scheduler: it produces the stream of homogeneous batches the
reference's engine would hand to its worker (every step is all-prompt or all-decode,
additional_designs/core/aptserve_scheduler.py:1613-1625) so that the GPU side — ragged
metadata construction and the decoder stack on the hybrid cache — can be run and timed
on realistic shapes.  Which requests use the hidden cache is a seeded coin flip here; the
reference's SLO-aware greedy choice is host policy and not part of this library.

Request stream (gen_client_requests.py:71-102 and sample_requests_from_datasets/
sample_from_sharegpt.py:35-41): inter-arrival times Gamma(shape=(1/cv)^2, scale=1/(rate*shape));
prompt lengths lognormal(5.5, 1.0) clipped to [4, 2048]; output lengths lognormal(5.0, 0.9)
clipped to [4, 1024]; prompt + output <= 2048.

Block numbering follows ``UncachedBlockAllocator`` and ``_allocate_sequence``
(additional_designs/core/aptserve_block_manager.py:176-199, 530-541, 744-749): private
blocks ``0..N-1``, shared blocks ``N..2N-1``; a hidden-cached sequence takes a new private
block ``p`` for every even logical block and ``p+N`` for the following odd one, plus one
shared block per logical block.
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional

import numpy as np
import torch

from . import metadata


@dataclass
class Request:
    rid: int
    arrival: float
    prompt_ids: np.ndarray
    output_len: int
    use_hidden: bool
    generated: List[int] = field(default_factory=list)
    block_table: List[int] = field(default_factory=list)
    shared_table: List[int] = field(default_factory=list)

    @property
    def seq_len(self) -> int:
        return len(self.prompt_ids) + len(self.generated)

    @property
    def token_ids(self) -> np.ndarray:
        """Prompt and everything generated so far: what a prompt step feeds the model (after a recompute
        preemption the generated tokens are part of it)."""
        if not self.generated:
            return self.prompt_ids
        return np.concatenate([self.prompt_ids, np.asarray(self.generated, dtype=np.int64)])


def synth_requests(seed: int, n: int, rate: float = 3.0, cv: float = 1.0, hidden_fraction: float = 0.5,
                   vocab: int = 50272, max_len: int = 2048, prompt_mu: float = 5.5, prompt_sigma: float = 1.0,
                   out_mu: float = 5.0, out_sigma: float = 0.9) -> List[Request]:
    rng = np.random.default_rng(seed)
    shape = (1.0 / cv) ** 2
    gaps = rng.gamma(shape, 1.0 / (rate * shape), n)
    arrivals = np.cumsum(gaps)
    reqs = []
    for i in range(n):
        p = int(np.clip(np.rint(rng.lognormal(prompt_mu, prompt_sigma)), 4, max_len))
        o = int(np.clip(np.rint(rng.lognormal(out_mu, out_sigma)), 4, 1024))
        if p + o > max_len:
            o = max(1, max_len - p)
            p = min(p, max_len - o)
        ids = rng.integers(0, vocab, p).astype(np.int64)
        reqs.append(Request(i, float(arrivals[i]), ids, o, bool(rng.random() < hidden_fraction)))
    return reqs


def fixed_step_cost(decode_s: float = 0.0125, prefill_s: float = 0.010, prefill_s_per_token: float = 2.0e-5):
    """A fixed cost model for the simulated clock: a decode step costs ``decode_s``, a prompt step
    ``prefill_s + tokens * prefill_s_per_token`` (roughly what OPT-13B takes on one MI355X)."""
    def cost(entry: Dict) -> float:
        if entry["kind"] == "decode":
            return decode_s
        return prefill_s + prefill_s_per_token * entry["tokens"]
    return cost


class BlockPool:
    def __init__(self, num_blocks: int) -> None:
        self.n = num_blocks
        self.free_private = list(range(num_blocks))
        self.free_shared = list(range(num_blocks, 2 * num_blocks))

    def blocks_needed(self, req: Request, new_len: int, block_size: int):
        have = len(req.block_table)
        need = -(-new_len // block_size)
        if not req.use_hidden:
            return need - have, 0
        new_private = sum(1 for i in range(have, need) if i % 2 == 0)
        return new_private, need - have

    def grow(self, req: Request, new_len: int, block_size: int) -> None:
        need = -(-new_len // block_size)
        while len(req.block_table) < need:
            i = len(req.block_table)
            if req.use_hidden:
                if i % 2 == 0:
                    req.block_table.append(self.free_private.pop())
                else:
                    req.block_table.append(req.block_table[-1] + self.n)
                req.shared_table.append(self.free_shared.pop())
            else:
                req.block_table.append(self.free_private.pop())

    def release(self, req: Request) -> None:
        self.free_private.extend(b for b in req.block_table if b < self.n)
        self.free_shared.extend(req.shared_table)
        req.block_table, req.shared_table = [], []


class StepLoop:
    """``forward(input_ids, positions, md) -> hidden_states`` is the GPU model step;
    ``pick(hidden_states, md) -> next token ids`` (a tensor of one id per sequence)."""

    def __init__(self, forward: Callable, pick: Callable, requests: List[Request], num_blocks: int, block_size: int,
                 device, max_prompt_tokens: int = 4096, max_seqs: int = 256,
                 on_step: Optional[Callable] = None, step_cost: Optional[Callable[[Dict], float]] = None,
                 decode_runner=None) -> None:
        """``step_cost(entry) -> seconds`` drives the simulated clock from a fixed cost model (same arrivals,
        admissions and batches whatever the measured speed, so two data flows can be compared step by step);
        ``None`` advances it by the measured wall time of every step.  ``decode_runner``
        (:class:`aptserve_hip.graph_step.DecodeGraphRunner`): decode steps are replayed from its HIP graphs
        instead of being issued through ``forward``."""
        self.forward, self.pick = forward, pick
        self.decode_runner = decode_runner
        self.waiting = sorted(requests, key=lambda r: r.arrival)
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self.pool = BlockPool(num_blocks)
        self.block_size, self.device = block_size, torch.device(device)
        self.max_prompt_tokens, self.max_seqs = max_prompt_tokens, max_seqs
        self.now = 0.0
        self.on_step = on_step
        self.step_cost = step_cost
        self.preemptions = 0
        self.log: List[Dict] = []

    def _admit(self) -> List[Request]:
        batch, tokens = [], 0
        while self.waiting and self.waiting[0].arrival <= self.now and len(self.running) + len(batch) < self.max_seqs:
            r = self.waiting[0]
            n_tok = r.seq_len                    # a preempted request comes back with its generated tokens
            p_need, s_need = self.pool.blocks_needed(r, n_tok + 1, self.block_size)
            if tokens + n_tok > self.max_prompt_tokens and batch:
                break
            if p_need > len(self.pool.free_private) - 8 or s_need > len(self.pool.free_shared) - 8:
                break
            self.pool.grow(r, n_tok, self.block_size)
            batch.append(self.waiting.pop(0))
            tokens += n_tok
        return batch

    def _make_room(self) -> None:
        """Before a decode step: if the free lists cannot take the blocks the running sequences are about to
        need, the most recently admitted sequences are preempted in recompute mode as the reference does when it
        runs out of blocks (additional_designs/core/aptserve_scheduler.py:2118-2130, `_preempt_by_recompute`):
        the blocks are released and the computed-token count starts over, but the generated tokens are kept
        (the next prompt step of the request runs over prompt + outputs), the request falls back to the K/V
        cache (`use_hidden = False`) and goes to the head of the queue."""
        while self.running:
            need_p = need_s = 0
            for r in self.running:
                p, s_ = self.pool.blocks_needed(r, r.seq_len, self.block_size)
                need_p += p
                need_s += s_
            if need_p <= len(self.pool.free_private) and need_s <= len(self.pool.free_shared):
                return
            if len(self.running) == 1:
                raise RuntimeError("the block pool cannot hold a single sequence of this length")
            victim = self.running.pop()
            self.pool.release(victim)
            victim.use_hidden = False
            self.waiting.insert(0, victim)
            self.preemptions += 1

    def step(self) -> Optional[Dict]:
        """Run one step; returns its log entry, or None when nothing is left to do."""
        batch = self._admit()
        is_prompt = bool(batch)
        if not is_prompt:
            if not self.running:
                if not self.waiting:
                    return None
                if self.waiting[0].arrival <= self.now:  # it has arrived, nothing else holds blocks, and it still
                    raise RuntimeError(                  # does not fit: waiting longer would change nothing
                        "the block pool cannot hold a single sequence of this length")
                self.now = self.waiting[0].arrival      # idle until the next arrival
                return self.step()
            self._make_room()
            batch = self.running
            for r in batch:                              # slot for the token produced by the previous step
                self.pool.grow(r, r.seq_len, self.block_size)
        seq_lens = [r.seq_len for r in batch]
        t0 = time.perf_counter()
        if is_prompt:
            ids = np.concatenate([r.token_ids for r in batch])
        else:
            ids = np.fromiter((r.generated[-1] for r in batch), dtype=np.int64, count=len(batch))
        input_ids = torch.from_numpy(ids).to(self.device, non_blocking=True)
        graphed = self.decode_runner is not None and not is_prompt
        captures = self.decode_runner.captures if graphed else 0
        if graphed:
            rec = self.decode_runner.prepare(seq_lens, [r.use_hidden for r in batch], [r.block_table for r in batch],
                                             [r.shared_table for r in batch], input_ids)
            md = rec.md
        else:
            md = metadata.build_metadata(is_prompt, seq_lens, [r.use_hidden for r in batch],
                                         [r.block_table for r in batch], [r.shared_table for r in batch],
                                         self.block_size, self.device)
        torch.cuda.synchronize(self.device)
        t1 = time.perf_counter()
        if graphed:
            hidden, md = self.decode_runner.run(rec)
        else:
            hidden = self.forward(input_ids, md.input_positions, md)
        nxt = self.pick(hidden, md)
        t_enq = time.perf_counter()              # everything is enqueued: host time of the step
        torch.cuda.synchronize(self.device)
        t2 = time.perf_counter()
        nxt_host = nxt.tolist()
        entry = dict(kind="prefill" if is_prompt else "decode", seqs=len(batch), tokens=int(len(ids)),
                     rows=md.num_tot_tokens, hidden_seqs=sum(r.use_hidden for r in batch),
                     metadata_ms=(t1 - t0) * 1e3, model_ms=(t2 - t1) * 1e3, host_enqueue_ms=(t_enq - t1) * 1e3,
                     now=self.now, graph=graphed,
                     recorded=graphed and self.decode_runner.captures != captures)  # this step recorded its graph
        if self.on_step is not None:
            self.on_step(dict(is_prompt=is_prompt, seq_lens=seq_lens, use_hidden=[r.use_hidden for r in batch],
                              block_tables=[list(r.block_table) for r in batch],
                              shared_tables=[list(r.shared_table) for r in batch], input_ids=ids.copy(),
                              hidden=hidden, next_tokens=nxt_host, md=md))
        for r, tok in zip(batch, nxt_host):
            r.generated.append(int(tok))
        if is_prompt:
            self.running.extend(batch)
        done = [r for r in self.running if len(r.generated) >= r.output_len or r.seq_len >= 2048]
        for r in done:
            self.pool.release(r)
            self.running.remove(r)
            self.finished.append(r)
        self.now += self.step_cost(entry) if self.step_cost is not None else (t2 - t0)
        self.log.append(entry)
        return entry

    def run(self, max_steps: int) -> List[Dict]:
        for _ in range(max_steps):
            if self.step() is None:
                break
        return self.log
