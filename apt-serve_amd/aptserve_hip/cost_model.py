"""Profit coefficient of the hybrid cache for the scheduler, measured on this library's kernels.

The reference derives the coefficient its greedy scheduler charges per hidden-cached block
(``hidden_profit = profit - U * coef * n_blocks``, additional_designs/core/aptserve_scheduler.py:586,634)
from a timing loop over ``F.linear`` (additional_designs/engine/aptserve_llm_engine.py:316-354): for
``num_tokens`` in ``range(1, 4101, 100)`` it times ``num_layers`` products of ``[num_tokens, Hd]`` with
the fused QKV weight, regresses the times on ``num_tokens // block_size`` (at least 1, with a (0, 0)
point added) and returns ``slope / 5``.  ``get_coef`` keeps that recipe and swaps the timed operation:

* ``mode="reprojection"``: the K/V re-projection GEMM of this library (``ops.linear_nt``), i.e. the cost
  the reference's data flow pays per cached hidden block and layer;
* ``mode="absorbed"``: the attention on the hidden rows themselves (``ops.absorbed_hidden_attention``),
  minus nothing: what a hidden-cached block costs per layer when nothing is re-projected;
* ``mode="reference_recipe"``: the reference's own timed operation, ``torch.nn.functional.linear`` (the vendor
  BLAS on this GPU) — in fp32 when ``dtype=torch.float32``, which is what the reference's ``torch.randn(...)``
  operands are — as the figure to hold the other two against.
"""

from __future__ import annotations

import time
from typing import Sequence, Tuple

import numpy as np
import torch

from . import ops


def fit_coef(num_tokens: Sequence[int], seconds: Sequence[float], block_size: int) -> float:
    """The regression of aptserve_llm_engine.py:336-347: blocks = tokens // block_size (>= 1), a (0, 0)
    point prepended, ordinary least squares with intercept, slope / 5."""
    x = np.array([0] + list(num_tokens)) // block_size
    x[1:][x[1:] == 0] = 1
    y = np.array([0.0] + list(seconds))
    slope, _ = np.polyfit(x.astype(np.float64), y, 1)
    return float(slope) / 5


def get_coef(hidden_size: int, num_heads: int, num_layers: int, block_size: int, device, dtype=torch.float16,
             mode: str = "reprojection", token_counts: Sequence[int] = tuple(range(1, 4101, 100))
             ) -> Tuple[float, list]:
    """Returns ``(coef, [(num_tokens, seconds)])``."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(0)
    w = (torch.randn(3 * hidden_size, hidden_size, generator=g, device=dev) * 0.02).to(dtype)
    stats = []
    if mode == "reference_recipe":
        for n in token_counts:
            x = torch.randn(n, hidden_size, generator=g, device=dev).to(dtype)
            torch.nn.functional.linear(x, w, None)
            torch.cuda.synchronize(dev)
            t0 = time.time()
            for _ in range(num_layers):
                torch.nn.functional.linear(x, w, None)
            torch.cuda.synchronize(dev)
            stats.append((n, time.time() - t0))
    elif mode == "reprojection":
        for n in token_counts:
            x = torch.randn(n, hidden_size, generator=g, device=dev).to(dtype)
            out = torch.empty(n, 3 * hidden_size, dtype=dtype, device=dev)
            ops.linear_nt(x, w, None, out=out)
            torch.cuda.synchronize(dev)
            t0 = time.time()
            for _ in range(num_layers):
                ops.linear_nt(x, w, None, out=out)
            torch.cuda.synchronize(dev)
            stats.append((n, time.time() - t0))
    elif mode == "absorbed":
        head = hidden_size // num_heads
        nblk = (max(token_counts) + block_size - 1) // block_size + 1
        cache = (torch.randn(2, nblk, block_size, num_heads, head, generator=g, device=dev)).to(dtype)
        q = torch.randn(1, hidden_size, generator=g, device=dev).to(dtype)
        out = torch.empty_like(q)
        rows = torch.zeros(1, dtype=torch.int64, device=dev)
        for n in token_counts:
            slots = torch.arange(n, dtype=torch.int64, device=dev)
            start = torch.tensor([0, n], dtype=torch.int64, device=dev)
            call = lambda: ops.absorbed_hidden_attention(q, cache, slots, start, rows, n, w[hidden_size:2 * hidden_size],
                                                         w[2 * hidden_size:], None, head ** -0.5, out)
            call()
            torch.cuda.synchronize(dev)
            t0 = time.time()
            for _ in range(num_layers):
                call()
            torch.cuda.synchronize(dev)
            stats.append((n, time.time() - t0))
    else:
        raise ValueError(f"unknown mode {mode!r}")
    return fit_coef([n for n, _ in stats], [t for _, t in stats], block_size), stats
