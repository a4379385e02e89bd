"""Pins the layer-level oracle with properties that hold whatever the implementation:
a decode step after a prefill must equal the last row of a one-token-longer prefill,
for K/V-cached and for hidden-cached sequences alike, and the two cache types must
agree with each other."""
import numpy as np
import pytest
import torch

from aptserve_hip import workloads
from oracle import layer as OL
from oracle.metadata import SeqRecord, build_metadata
from util import randn


def weights(Hd, seed):
    return ((randn((3 * Hd, Hd), seed) * 0.08).half(), (randn((3 * Hd,), seed + 1) * 0.1).half(),
            (randn((Hd, Hd), seed + 2) * 0.08).half(), (randn((Hd,), seed + 3) * 0.1).half())


@pytest.mark.parametrize("frac", [0.0, 0.5, 1.0])
def test_decode_after_prefill_equals_longer_prefill(frac):
    H, D, N, BS = 2, 8, 48, 16
    Hd = H * D
    W = weights(Hd, 0)
    rng = np.random.default_rng(1)
    lens = [5, 16, 23, 40]
    hid = workloads.pick_hidden(rng, len(lens), frac)
    full = workloads.allocate_blocks(rng, [l + 1 for l in lens], hid, N, BS, is_prompt=True)
    xs = [randn((l + 1, Hd), 10 + i) for i, l in enumerate(lens)]

    def recs(is_prompt, seq_lens, ctx):
        return [SeqRecord(is_prompt, bool(h), l, c, bt, bts) for l, c, h, bt, bts in
                zip(seq_lens, ctx, hid, full.block_tables, full.block_tables_4_shared)]
    # (1) prefill of L+1 tokens: last row of each sequence is the reference answer
    kv1 = torch.zeros(2, N, BS, H, D, dtype=torch.float16); sh1 = torch.zeros(2, 2 * N, BS, H, D, dtype=torch.float16)
    md = build_metadata(recs(True, [l + 1 for l in lens], [0] * len(lens)), BS)
    out_full = OL.opt_attention(torch.cat(xs), kv1, sh1, md, *W, H)
    ends = np.cumsum([l + 1 for l in lens]) - 1
    # (2) prefill of L tokens, then one decode step with the last token
    kv2 = torch.zeros_like(kv1); sh2 = torch.zeros_like(sh1)
    md_p = build_metadata(recs(True, lens, [0] * len(lens)), BS)
    OL.opt_attention(torch.cat([x[:-1] for x in xs]), kv2, sh2, md_p, *W, H)
    md_d = build_metadata(recs(False, [l + 1 for l in lens], lens), BS)
    out_dec = OL.opt_attention(torch.stack([x[-1] for x in xs]), kv2, sh2, md_d, *W, H)
    assert torch.allclose(out_dec.float(), out_full[ends].float(), atol=3e-3, rtol=3e-3)
    # the persistent caches end up identical as well
    assert torch.equal(kv1, kv2)


def test_hidden_cached_and_kv_cached_runs_agree():
    H, D, N, BS = 2, 8, 48, 16
    Hd = H * D
    W = weights(Hd, 5)
    lens = [7, 30, 18]
    xs = [randn((l + 1, Hd), 20 + i) for i, l in enumerate(lens)]
    outs = []
    for frac in (0.0, 1.0):
        rng = np.random.default_rng(2)
        hid = workloads.pick_hidden(rng, len(lens), frac)
        b = workloads.allocate_blocks(rng, [l + 1 for l in lens], hid, N, BS, is_prompt=True)
        mk = lambda p, sl, ctx: build_metadata([SeqRecord(p, bool(h), l, c, bt, bts) for l, c, h, bt, bts in
                                                zip(sl, ctx, hid, b.block_tables, b.block_tables_4_shared)], BS)
        kv = torch.zeros(2, N, BS, H, D, dtype=torch.float16); sh = torch.zeros(2, 2 * N, BS, H, D, dtype=torch.float16)
        OL.opt_attention(torch.cat([x[:-1] for x in xs]), kv, sh, mk(True, lens, [0] * 3), *W, H)
        outs.append(OL.opt_attention(torch.stack([x[-1] for x in xs]), kv, sh,
                                     mk(False, [l + 1 for l in lens], lens), *W, H))
    assert torch.allclose(outs[0].float(), outs[1].float(), atol=3e-3, rtol=3e-3)
