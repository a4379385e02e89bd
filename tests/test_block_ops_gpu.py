"""Block maintenance (copy / swap) aware of hidden blocks, and the scheduler's cost coefficient."""
import numpy as np
import pytest
import torch

from aptserve_hip import cost_model, ops
from util import sentinel_cache

pytestmark = pytest.mark.gpu

H, D, BS, N = 3, 8, 16, 20


def expected_copy(cache, pairs, kinds):
    ref = cache.clone()
    flat = ref.view(2 * N, BS, H, D)            # plane slabs: id < N is the K plane of a block, id >= N its V plane
    src_flat = cache.view(2 * N, BS, H, D)
    for (a, b), k in zip(pairs, kinds):
        if k:
            flat[b] = src_flat[a]
        else:
            ref[0, b], ref[1, b] = cache[0, a], cache[1, a]
    return ref


def test_copy_blocks_all_layers_kv_and_hidden(dev):
    layers = [sentinel_cache((2, N, BS, H, D), seed=i) for i in range(3)]
    pairs = [(1, 7), (2, 9), (3 + N, 11 + N), (4, 15 + N), (18 + N, 0)]      # distinct destinations
    kinds = [0, 0, 1, 1, 1]
    d_layers = [c.to(dev) for c in layers]
    ops.copy_blocks(d_layers, torch.tensor(pairs, dtype=torch.int64, device=dev),
                    torch.tensor(kinds, dtype=torch.uint8, device=dev))
    for c, d in zip(layers, d_layers):
        assert torch.equal(d.cpu().view(torch.int16), expected_copy(c, pairs, kinds).view(torch.int16))
    # reference call shape (no kinds): K/V blocks only; out-of-range ids are skipped
    d2 = [c.to(dev) for c in layers]
    ops.copy_blocks(d2, torch.tensor([(1, 7), (N + 2, 3), (5, N)], dtype=torch.int64, device=dev))
    for c, d in zip(layers, d2):
        assert torch.equal(d.cpu().view(torch.int16), expected_copy(c, [(1, 7)], [0]).view(torch.int16))
    ops.copy_blocks(d2, torch.empty(0, 2, dtype=torch.int64, device=dev))


def test_swap_blocks_out_and_back_in(dev):
    gpu = sentinel_cache((2, N, BS, H, D)).to(dev)
    orig = gpu.clone()
    NC = 12
    cpu = torch.zeros(2, NC, BS, H, D, dtype=torch.float16).pin_memory()
    out_pairs = torch.tensor([(3, 0), (5, 1), (7 + N, 2 + NC), (9, 4 + NC)], dtype=torch.int64)
    kinds = torch.tensor([0, 0, 1, 1], dtype=torch.uint8)
    ops.swap_blocks(gpu, cpu, out_pairs, kinds)
    torch.cuda.synchronize()
    assert torch.equal(cpu[:, 0], orig[:, 3].cpu()) and torch.equal(cpu[:, 1], orig[:, 5].cpu())
    assert torch.equal(cpu[1, 2], orig[1, 7].cpu()) and torch.equal(cpu[1, 4], orig[0, 9].cpu())
    assert (cpu[0, 2] == 0).all() and (cpu[0, 4] == 0).all()               # a hidden block is one slab
    gpu.zero_()
    back = torch.tensor([(0, 3), (1, 5), (2 + NC, 7 + N), (4 + NC, 9)], dtype=torch.int64)
    ops.swap_blocks(cpu, gpu, back, kinds)
    torch.cuda.synchronize()
    g = gpu.cpu()
    assert torch.equal(g[:, 3], orig[:, 3].cpu()) and torch.equal(g[:, 5], orig[:, 5].cpu())
    assert torch.equal(g[1, 7], orig[1, 7].cpu()) and torch.equal(g[0, 9], orig[0, 9].cpu())
    with pytest.raises(RuntimeError):
        ops.swap_blocks(cpu, gpu, torch.tensor([(NC, 0)], dtype=torch.int64))   # source block out of range


def test_cost_coefficient_is_measured_on_both_flows(dev):
    """The coefficient is the slope of time over blocks / 5 (aptserve_llm_engine.py:336-347).  Checked on a size
    where the product is long enough to time: the times grow with the token count, the coefficient agrees with
    a direct two-point slope, and the library's GEMM is in the same league as the recipe's F.linear."""
    counts = (1, 1025, 2049, 4097)
    layers, bs = 8, 16
    res = {}
    for mode in ("reprojection", "absorbed", "reference_recipe"):
        cost_model.get_coef(2048, 16, 2, bs, dev, mode=mode, token_counts=(1, 4097))     # warm-up (first launches)
        c, st = cost_model.get_coef(2048, 16, layers, bs, dev, mode=mode, token_counts=counts)
        t = [x for _, x in st]
        assert len(st) == 4 and all(x > 0 for x in t) and np.isfinite(c) and c > 0
        assert t[3] > t[1], (mode, t)                              # 4x the tokens take longer
        # between the marginal cost of a block (two-point slope) and its average cost (the recipe's (0, 0) point
        # pulls the fit towards the average when a call has a fixed cost, as the six launches of the absorbed
        # attention do)
        direct = (t[3] - t[1]) / ((counts[3] - counts[1]) // bs) / 5
        average = t[3] / (counts[3] // bs) / 5
        assert 0.4 * min(direct, average) < c < 2.5 * max(direct, average), (mode, c, direct, average)
        res[mode] = c
    assert 0.2 < res["reprojection"] / res["reference_recipe"] < 5.0, res


def test_promote_hidden_rows_to_kv(dev):
    from aptserve_hip import backend
    from oracle import reproject as OR
    from util import randn
    Hh, Dd, Nn = 4, 64, 12
    Hd = Hh * Dd
    cache = randn((2, Nn, BS, Hh, Dd), 0)
    w = (randn((3 * Hd, Hd), 1) * 0.05).half()
    b = (randn((3 * Hd,), 2) * 0.1).half()
    hidden_slots = torch.tensor([5, 6, 7, 2 * 16 + 3, Nn * 16 + 9], dtype=torch.int64)     # K- and V-plane slabs
    kv_slots = torch.tensor([8 * 16 + i for i in range(5)], dtype=torch.int64)
    rows = cache.view(-1, Hd)[hidden_slots]
    k_ref, v_ref = OR.kv_reproject(rows, w[Hd:], b[Hd:], keep_fp32=True)
    d = cache.to(dev)
    backend.promote_hidden_to_kv(w.to(dev), b.to(dev), d, hidden_slots.to(dev), kv_slots.to(dev))
    got = d.cpu()
    assert (got[0].view(-1, Hd)[kv_slots].float() - k_ref.view(5, Hd)).abs().max() < 2e-2
    assert (got[1].view(-1, Hd)[kv_slots].float() - v_ref.view(5, Hd)).abs().max() < 2e-2
    untouched = torch.ones(Nn * 16, dtype=torch.bool); untouched[kv_slots] = False
    assert torch.equal(got[0].view(-1, Hd)[untouched], cache[0].view(-1, Hd)[untouched])
    assert torch.equal(got[1].view(-1, Hd)[untouched], cache[1].view(-1, Hd)[untouched])

