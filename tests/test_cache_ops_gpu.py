"""HIP cache operators against the oracle on the same seeded inputs — bit-exact.

Every call goes through the C ABI (``aptserve_hip.ops`` hands raw pointers to
``libaptserve_hip.so``).
"""
import numpy as np
import pytest
import torch

import mixed_cache_ops
from aptserve_hip import ops, workloads
from oracle import cache_ops as O
from oracle import fp8 as O8
from util import bits_equal, oracle_metadata, randn, sentinel_cache, t64

pytestmark = pytest.mark.gpu


def idx(md, name, dev):
    return t64(md[name], dev)


def cheap_pattern(shape, dtype=torch.float16):
    n = int(np.prod(shape))
    a = (torch.arange(n, dtype=torch.int32) % 15361).to(torch.int16)  # fp16 bit patterns below 0x3C01
    return a.view(dtype).reshape(shape)


# ------------------------------------------------------------------ config 1

def test_config1_mixed_write_opt125m_bit_exact(dev):
    """8 prompts, 351 tokens, 12x64 heads, 512-block pool, 2 of 8 hidden-cached (seed 0)."""
    b = workloads.mixed_write_opt125m(0)
    assert b.seq_lens == [109, 82, 66, 35, 40, 6, 10, 3] and sum(b.use_hidden) == 2
    md = oracle_metadata(b)
    H, D, N, BS = 12, 64, 512, 16
    T = md["num_prefill_tokens"]
    assert T == 351
    key, value, hidden = randn((T, H, D), 0), randn((T, H, D), 1), randn((T, H * D), 2)
    cache = sentinel_cache((2, N, BS, H, D))
    ref = cache.clone()
    sm = t64(md["slot_mapping"])
    kv_use, h_use = t64(md["kv_cache_use_tot"]), t64(md["hidden_cache_use_input"])
    # oracle: the prefill sequence of aptserve_opt.py:108-109 and aptserve_flash_attn.py:347-355
    O.hidden_to_cache(hidden, ref, sm, h_use, t64(md["hidden_cache_store_tot"]))
    O.reshape_and_cache_flash(key[kv_use], value[kv_use], ref[0], ref[1], sm[kv_use], "auto")
    # HIP, reference call pattern (gather copies + full write)
    g = cache.to(dev)
    dk, dv, dh, dsm = key.to(dev), value.to(dev), hidden.to(dev), sm.to(dev)
    mixed_cache_ops.hidden_to_cache(dh, g, dsm, h_use.to(dev), idx(md, "hidden_cache_store_tot", dev))
    dkv = kv_use.to(dev)
    ops.reshape_and_cache_flash(dk[dkv], dv[dkv], g[0], g[1], dsm[dkv], "auto")
    assert bits_equal(g, ref)
    # HIP, subset write without the gather copies
    g2 = cache.to(dev)
    ops.hidden_to_cache(dh, g2, dsm, h_use.to(dev), idx(md, "hidden_cache_store_tot", dev))
    ops.reshape_and_cache_flash(dk, dv, g2[0], g2[1], dsm, "auto", token_idx=dkv)
    assert bits_equal(g2, ref)
    # HIP, one launch by token type, mask from the GPU metadata builder
    from aptserve_hip import metadata
    gmd = metadata.build_from_batch(b, dev)
    mask = torch.zeros(T, dtype=torch.uint8); mask[h_use] = 1
    assert torch.equal(gmd.token_is_hidden.cpu(), mask)
    g3 = cache.to(dev)
    ops.mixed_reshape_and_cache(dk, dv, dh, g3, gmd.slot_mapping, gmd.token_is_hidden)
    assert bits_equal(g3, ref)
    ref2 = cache.clone()
    O.mixed_reshape_and_cache(key, value, hidden, ref2, sm, mask)
    assert bits_equal(ref2, ref)
    # untouched slots still hold the sentinel
    touched = torch.zeros(2 * N * BS, dtype=torch.bool)
    touched[sm[h_use]] = True
    touched[sm[kv_use]] = True
    touched[sm[kv_use] + N * BS] = True
    assert bits_equal(g2.cpu().view(-1, H * D)[~touched], cache.view(-1, H * D)[~touched])


# ------------------------------------------------------- write by token type

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,D", [(2, 4), (12, 64), (1, 5)])
@pytest.mark.parametrize("seed,frac", [(0, 0.4), (1, 1.0), (2, 0.0)])
def test_mixed_reshape_and_cache_small(dev, dtype, H, D, seed, frac):
    b = workloads.small_prefill_batch(seed, 7, 60, frac, 64)
    md = oracle_metadata(b)
    T, N, BS = md["num_prefill_tokens"], 64, 16
    sm = t64(md["slot_mapping"]).clone()
    sm[::11] = -1                                          # padding tokens of either kind
    mask = torch.zeros(T, dtype=torch.uint8); mask[t64(md["hidden_cache_use_input"])] = 1
    wide = randn((T, 3 * H * D), seed, dtype)              # K and V as chunk views of a fused projection
    key, value = wide[:, :H * D].view(T, H, D), wide[:, H * D:2 * H * D].view(T, H, D)
    hidden = randn((T, H * D), seed + 9, dtype)
    cache = sentinel_cache((2, N, BS, H, D), dtype)
    ref = cache.clone()
    O.mixed_reshape_and_cache(key, value, hidden, ref, sm, mask)
    g = cache.to(dev)
    dw = wide.to(dev)
    dk, dv = dw[:, :H * D].view(T, H, D), dw[:, H * D:2 * H * D].view(T, H, D)
    ops.mixed_reshape_and_cache(dk, dv, hidden.to(dev), g, sm.to(dev), mask.to(dev))
    assert bits_equal(g, ref)
    # one kind only
    ref_h, ref_kv = cache.clone(), cache.clone()
    O.mixed_reshape_and_cache(None, None, hidden, ref_h, sm, mask)
    O.mixed_reshape_and_cache(key, value, None, ref_kv, sm, mask)
    g_h, g_kv = cache.to(dev), cache.to(dev)
    ops.mixed_reshape_and_cache(None, None, hidden.to(dev), g_h, sm.to(dev), mask.to(dev))
    ops.mixed_reshape_and_cache(dk, dv, None, g_kv, sm.to(dev), mask.to(dev))
    assert bits_equal(g_h, ref_h) and bits_equal(g_kv, ref_kv)
    # no mask: every token is a K/V token == reshape_and_cache_flash
    # (hidden sequences use block ids >= N for their odd blocks: no K/V block there, mark as padding)
    ref_all, g_all = cache.clone(), cache.to(dev)
    sm_kv = torch.where(sm < N * BS, sm, torch.full_like(sm, -1))
    O.reshape_and_cache_flash(key, value, ref_all[0], ref_all[1], sm_kv, "auto")
    ops.mixed_reshape_and_cache(dk, dv, None, g_all, sm_kv.to(dev), None)
    assert bits_equal(g_all, ref_all)


def test_mixed_reshape_and_cache_fp8_kv_rows(dev):
    """K/V rows quantised into a 1-byte cache, hidden rows unquantised into their own cache."""
    H, D, N, BS = 12, 64, 64, 16
    b = workloads.small_prefill_batch(5, 7, 60, 0.5, N)
    md = oracle_metadata(b)
    T = md["num_prefill_tokens"]
    sm = t64(md["slot_mapping"])
    mask = torch.zeros(T, dtype=torch.uint8); mask[t64(md["hidden_cache_use_input"])] = 1
    key, value, hidden = randn((T, H, D), 0) * 3, randn((T, H, D), 1) * 3, randn((T, H * D), 2)
    kv_idx = torch.nonzero(mask == 0).flatten()
    q_ref = torch.full((2, N, BS, H, D), 0x55, dtype=torch.uint8)
    O.reshape_and_cache_flash(key[kv_idx], value[kv_idx], q_ref[0], q_ref[1], sm[kv_idx], "fp8", 0.5, 0.25)
    h_ref = sentinel_cache((2, N, BS, H, D))
    h0 = h_ref.clone()
    O.mixed_reshape_and_cache(None, None, hidden, h_ref, sm, mask)
    q = torch.full((2, N, BS, H, D), 0x55, dtype=torch.uint8, device=dev)
    hc = h0.to(dev)
    ops.mixed_reshape_and_cache(key.to(dev), value.to(dev), hidden.to(dev), q, sm.to(dev), mask.to(dev), "fp8",
                                0.5, 0.25, hidden_cache=hc)
    assert torch.equal(q.cpu(), q_ref)
    assert bits_equal(hc, h_ref)
    with pytest.raises(ValueError):                        # an fp8 cache cannot hold hidden rows itself
        ops.mixed_reshape_and_cache(key.to(dev), value.to(dev), hidden.to(dev), q, sm.to(dev), mask.to(dev), "fp8")


# ------------------------------------------------------- small random batches

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32, torch.float64])
@pytest.mark.parametrize("H,D", [(2, 4), (3, 2), (1, 3), (12, 64)])
@pytest.mark.parametrize("seed", [0, 1])
def test_hidden_scatter_gather_small(dev, dtype, H, D, seed):
    N, BS = 40, 16
    b = workloads.small_decode_batch(seed, 7, 70, 0.5, N)
    md = oracle_metadata(b)
    B, T, Hd = len(b.seq_lens), md["num_tot_tokens"], H * D
    hs = randn((B, Hd), seed, dtype)
    cache = sentinel_cache((2, N, BS, H, D), dtype)
    ref = cache.clone()
    sm = t64(md["slot_mapping"])
    O.hidden_to_cache(hs, ref, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    g = cache.to(dev)
    ops.hidden_to_cache(hs.to(dev), g, sm.to(dev), idx(md, "hidden_cache_use_input", dev),
                        idx(md, "hidden_cache_store_tot", dev))
    assert bits_equal(g, ref)
    holder_ref = sentinel_cache((T, Hd), dtype, seed=9)
    holder = holder_ref.to(dev)
    O.cache_to_hidden(holder_ref, ref, sm, t64(md["hidden_cache_use_tot"]))
    ops.cache_to_hidden(holder, g, sm.to(dev), idx(md, "hidden_cache_use_tot", dev))
    assert bits_equal(holder, holder_ref)


def test_strided_hidden_rows_and_pad_slots(dev):
    """Row stride taken from .stride(0) (mixed_cache.cu:128); slot -1 is skipped."""
    H, D, N, BS = 2, 8, 8, 16
    wide = randn((10, 3 * H * D), 0)
    hidden = wide[:, H * D:2 * H * D]           # stride 48, width 16
    sm = t64([5, -1, 77, 130, -1, 9, 255, 18, 200, 31])
    cache = sentinel_cache((2, N, BS, H, D)); ref = cache.clone()
    src = t64([9, 1, 0, 3, 4, 2]); tgt = t64([0, 1, 2, 3, 4, 6])
    O.hidden_to_cache(hidden, ref, sm, src, tgt)
    g = cache.to(dev)
    ops.hidden_to_cache(wide.to(dev)[:, H * D:2 * H * D], g, sm.to(dev), src.to(dev), tgt.to(dev))
    assert bits_equal(g, ref)
    out_ref = sentinel_cache((10, 3 * H * D), seed=3)
    out = out_ref.to(dev)
    dst = t64([0, 1, 2, 3, 4, 5, 6, 7, 8, 9])
    O.cache_to_hidden(out_ref[:, :H * D], ref, sm, dst)
    ops.cache_to_hidden(out[:, :H * D], g, sm.to(dev), dst.to(dev))
    assert bits_equal(out, out_ref)


def test_out_of_range_indices_are_skipped_not_faulted(dev):
    H, D, N, BS = 1, 8, 2, 16
    cache = sentinel_cache((2, N, BS, H, D)); g = cache.to(dev)
    hidden = randn((3, 8), 0).to(dev)
    sm = t64([2 * N * BS, 1 << 40, 3], dev)              # first two beyond the cache
    ops.hidden_to_cache(hidden, g, sm, t64([0, 1, 2, 7], dev), t64([0, 1, 2, 2], dev))   # src 7 beyond hidden
    ref = cache.clone(); ref.view(-1, 8)[3] = hidden[2].cpu()
    assert bits_equal(g, ref)
    out = torch.zeros(3, 8, dtype=torch.float16, device=dev)
    ops.cache_to_hidden(out, g, sm, t64([0, 1, 2, 5, -3], dev))
    assert torch.equal(out[2].cpu(), hidden[2].cpu()) and out[:2].abs().sum() == 0


@pytest.mark.parametrize("seed,frac", [(0, 0.5), (1, 0.3), (2, 1.0), (3, 0.0)])
@pytest.mark.parametrize("H,D", [(2, 4), (12, 64)])
def test_hybrid_decode_gather_equals_reference_sequence(dev, seed, frac, H, D):
    N, BS = 64, 16
    b = workloads.small_decode_batch(seed, 9, 90, frac, N)
    md = oracle_metadata(b)
    B, T, Hd = len(b.seq_lens), md["num_tot_tokens"], H * D
    hs = randn((B, Hd), seed)
    cache = sentinel_cache((2, N, BS, H, D))
    ref = cache.clone()
    sm = t64(md["slot_mapping"])
    O.hidden_to_cache(hs, ref, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    holder_ref = O.assemble_hidden_holder(hs, ref, sm, T, t64(md["hidden_holder_upd"]),
                                          t64(md["hidden_cache_use_tot"]))
    g = cache.to(dev)
    holder = sentinel_cache((T, Hd), seed=5).to(dev)     # deliberately not zeroed
    ops.hybrid_decode_gather(holder, hs.to(dev), g, sm.to(dev), idx(md, "hidden_holder_upd", dev),
                             idx(md, "hidden_holder_pull", dev), idx(md, "hidden_cache_use_input", dev),
                             idx(md, "hidden_cache_store_tot", dev))
    assert bits_equal(holder, holder_ref)
    assert bits_equal(g, ref)


def test_hybrid_decode_gather_zero_fills_padding_rows(dev):
    H, D, N, BS = 1, 8, 4, 16
    # one hidden sequence of 3 rows whose middle slot is padding, one K/V sequence
    sm = t64([4, -1, 6, 40])
    upd, pull = t64([2, 3]), t64([0, 1])
    hs = randn((2, 8), 0)
    cache = sentinel_cache((2, N, BS, H, D)); ref = cache.clone()
    O.hidden_to_cache(hs, ref, sm, t64([0]), t64([2]))
    holder_ref = O.assemble_hidden_holder(hs, ref, sm, 4, upd, t64([0, 1, 2]))
    g = cache.to(dev)
    holder = sentinel_cache((4, 8), seed=5).to(dev)
    ops.hybrid_decode_gather(holder, hs.to(dev), g, sm.to(dev), upd.to(dev), pull.to(dev), t64([0], dev),
                             t64([2], dev))
    assert bits_equal(holder, holder_ref) and bits_equal(g, ref)
    assert holder[1].abs().sum() == 0


@pytest.mark.parametrize("seed,frac", [(0, 0.5), (1, 0.3), (2, 1.0), (3, 0.0)])
@pytest.mark.parametrize("H,D", [(2, 4), (12, 64), (40, 128)])
def test_resolved_gather_equals_reference_sequence(dev, seed, frac, H, D):
    """gather_hidden_rows driven by the metadata builder's holder_src."""
    from aptserve_hip import metadata
    N, BS = 64, 16
    b = workloads.small_decode_batch(seed, 9, 90, frac, N)
    md = oracle_metadata(b)
    gmd = metadata.build_from_batch(b, dev)
    B, T, Hd = len(b.seq_lens), md["num_tot_tokens"], H * D
    hs = randn((B, Hd), seed)
    cache = sentinel_cache((2, N, BS, H, D))
    ref = cache.clone()
    sm = t64(md["slot_mapping"])
    O.hidden_to_cache(hs, ref, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    holder_ref = O.assemble_hidden_holder(hs, ref, sm, T, t64(md["hidden_holder_upd"]),
                                          t64(md["hidden_cache_use_tot"]))
    g = cache.to(dev)
    holder = sentinel_cache((T, Hd), seed=5).to(dev)
    ops.gather_hidden_rows(holder, hs.to(dev), g, gmd.holder_src, gmd.slot_mapping, gmd.hidden_cache_use_input,
                           gmd.hidden_cache_store_tot)
    assert bits_equal(holder, holder_ref)
    assert bits_equal(g, ref)


def test_resolved_gather_zero_fills_padding_rows(dev):
    H, D, N, BS = 1, 8, 4, 16
    sm = t64([4, -1, 6, 40], dev)
    src = t64([4, -(1 << 63), -1, -2], dev)
    hs = randn((2, 8), 0)
    cache = sentinel_cache((2, N, BS, H, D))
    g = cache.to(dev)
    holder = sentinel_cache((4, 8), seed=5).to(dev)
    ops.gather_hidden_rows(holder, hs.to(dev), g, src, sm, t64([0], dev), t64([2], dev))
    h = holder.cpu()
    assert torch.equal(h[0], cache.view(-1, 8)[4]) and h[1].abs().sum() == 0
    assert torch.equal(h[2], hs[0]) and torch.equal(h[3], hs[1])
    assert torch.equal(g.cpu().view(-1, 8)[6], hs[0])


@pytest.mark.parametrize("seed,frac", [(0, 0.5), (1, 0.3), (2, 1.0), (3, 0.0)])
@pytest.mark.parametrize("H,D,dtype", [(2, 4, torch.float16), (12, 64, torch.bfloat16), (40, 128, torch.float16),
                                       (3, 8, torch.float32)])
def test_decode_step_cache_ops_one_launch(dev, seed, frac, H, D, dtype):
    """One launch for a decode layer's cache traffic: hidden stores, holder assembly and the newest K/V rows of
    the K/V-cached sequences, against the oracle's separate operators (aptserve_opt.py:108-121,
    aptserve_flash_attn.py:338-345); key / value are the chunk views of one [B, 2*Hd] projection."""
    from aptserve_hip import metadata
    N, BS = 64, 16
    b = workloads.small_decode_batch(seed, 9, 90, frac, N)
    md = oracle_metadata(b)
    gmd = metadata.build_from_batch(b, dev)
    B, T, Hd = len(b.seq_lens), md["num_tot_tokens"], H * D
    hs = randn((B, Hd), seed, dtype)
    kv = randn((B, 2 * Hd), seed + 7, dtype)
    k, v = (x.view(B, H, D) for x in kv.chunk(2, -1))
    cache = sentinel_cache((2, N, BS, H, D), dtype)
    ref = cache.clone()
    sm = t64(md["slot_mapping"])
    O.hidden_to_cache(hs, ref, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    holder_ref = O.assemble_hidden_holder(hs, ref, sm, T, t64(md["hidden_holder_upd"]),
                                          t64(md["hidden_cache_use_tot"]))
    seq_idx = torch.tensor([i for i, h in enumerate(b.use_hidden) if not h], dtype=torch.int64)
    O.reshape_and_cache_flash(k[seq_idx], v[seq_idx], ref[0], ref[1], sm[t64(md["kv_cache_use_tot"])], "auto")
    g = cache.to(dev)
    holder = sentinel_cache((T, Hd), dtype, seed=5).to(dev)
    dkv = kv.to(dev)
    dk, dv = dkv.chunk(2, -1)
    ops.decode_step_cache_ops(holder, hs.to(dev), g, gmd.holder_src, gmd.slot_mapping, gmd.hidden_cache_use_input,
                              gmd.hidden_cache_store_tot, dk, dv, gmd.kv_cache_use_input, gmd.new_token_slot)
    assert bits_equal(holder, holder_ref)
    assert bits_equal(g, ref)


def test_decode_step_cache_ops_without_a_holder_stores_only(dev):
    """No holder (the flow that attends on the cached hidden rows assembles none): the launch is the hidden-row
    stores and the K/V-row writes, the hidden rows into one cache and the K/V rows into another."""
    from aptserve_hip import metadata
    N, BS, H, D = 64, 16, 4, 32
    b = workloads.small_decode_batch(3, 9, 90, 0.5, N)
    md, gmd = oracle_metadata(b), metadata.build_from_batch(b, dev)
    B, Hd = len(b.seq_lens), H * D
    hs, kv = randn((B, Hd), 3), randn((B, 2 * Hd), 10)
    k, v = kv.chunk(2, -1)
    sm = t64(md["slot_mapping"])
    seq_idx = torch.tensor([i for i, h in enumerate(b.use_hidden) if not h], dtype=torch.int64)
    for separate in (False, True):
        hidden_cache, kv_cache = sentinel_cache((2, N, BS, H, D)), sentinel_cache((2, N, BS, H, D), seed=9)
        ref_h, ref_kv = hidden_cache.clone(), (kv_cache.clone() if separate else None)
        if not separate:
            ref_kv = ref_h
        O.hidden_to_cache(hs, ref_h, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
        O.reshape_and_cache_flash(k[seq_idx].view(-1, H, D), v[seq_idx].view(-1, H, D), ref_kv[0], ref_kv[1],
                                  sm[t64(md["kv_cache_use_tot"])], "auto")
        gh, gkv = hidden_cache.to(dev), kv_cache.to(dev)
        dk, dv = kv.to(dev).chunk(2, -1)
        ops.decode_step_cache_ops(None, hs.to(dev), gh, None, gmd.slot_mapping, gmd.hidden_cache_use_input,
                                  gmd.hidden_cache_store_tot, dk, dv, gmd.kv_cache_use_input, gmd.new_token_slot,
                                  kv_cache=gkv if separate else None)
        assert bits_equal(gh, ref_h)
        if separate:
            assert bits_equal(gkv, ref_kv)
    assert md["num_hidden_cache_tokens"] > 0 and len(seq_idx) > 0


def test_decode_step_cache_ops_skips_bad_rows(dev):
    """Padding slots, out-of-range sequence positions and slots past the cache are skipped, not written."""
    H, D, N, BS = 1, 8, 4, 16
    cache = sentinel_cache((2, N, BS, H, D))
    g = cache.to(dev)
    hs, k, v = randn((3, 8), 0), randn((3, 8), 1), randn((3, 8), 2)
    holder = sentinel_cache((2, 8), seed=5).to(dev)
    src = t64([5, -2], dev)                       # a cache slot, then row 1 of the inputs
    ops.decode_step_cache_ops(holder, hs.to(dev), g, src, t64([5, 9], dev), t64([], dev), t64([], dev), k.to(dev),
                              v.to(dev), t64([0, 2, 7, -1, 1], dev), t64([3, -1, N * BS], dev))
    ref = cache.clone()
    ref[0].view(-1, 8)[3] = k[0]
    ref[1].view(-1, 8)[3] = v[0]
    assert bits_equal(g, ref)
    h = holder.cpu()
    assert torch.equal(h[0], cache.view(-1, 8)[5]) and torch.equal(h[1], hs[1])


# ---------------------------------------------------------------- K/V writes

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,D", [(3, 8), (12, 64), (40, 128), (1, 5)])
def test_reshape_and_cache_flash(dev, dtype, H, D):
    N, BS, T = 12, 16, 100
    rng = np.random.default_rng(H * D)
    slots = rng.permutation(N * BS)[:T].astype(np.int64)
    slots[[0, 50, 99]] = -1
    qkv = randn((T, 3 * H * D), 0, dtype)
    key, value = qkv[:, H * D:2 * H * D].view(T, H, D), qkv[:, 2 * H * D:].view(T, H, D)   # chunk views
    kc, vc = sentinel_cache((N, BS, H, D), dtype), sentinel_cache((N, BS, H, D), dtype, seed=2)
    kr, vr = kc.clone(), vc.clone()
    O.reshape_and_cache_flash(key, value, kr, vr, t64(slots), "auto")
    gq = qkv.to(dev)
    gk, gv = gq[:, H * D:2 * H * D].view(T, H, D), gq[:, 2 * H * D:].view(T, H, D)
    gkc, gvc = kc.to(dev), vc.to(dev)
    ops.reshape_and_cache_flash(gk, gv, gkc, gvc, t64(slots, dev), "auto")
    assert bits_equal(gkc, kr) and bits_equal(gvc, vr)


@pytest.mark.parametrize("seed,frac,batch,max_len", [(0, 0.4, 6, 5), (1, 0.2, 6, 5), (7, 0.5, 12, 40), (3, 1.0, 4, 30)])
@pytest.mark.parametrize("H,D", [(2, 4), (12, 64)])
def test_mixed_kv_to_cache_intended(dev, seed, frac, batch, max_len, H, D):
    N, BS = 64, 16
    b = workloads.small_decode_batch(seed, batch, max_len, frac, N)
    md = oracle_metadata(b)
    T = md["num_tot_tokens"]
    kv = randn((T, 2 * H * D), seed)
    key, value = (x.view(T, H, D) for x in kv.chunk(2, dim=-1))       # stride 2*Hd like aptserve_opt.py:124
    caches = [sentinel_cache((n, BS, H, D), seed=i) for i, n in enumerate((N, N, 2 * N, 2 * N))]
    ref = [c.clone() for c in caches]
    names = ("slot_mapping", "slot_mapping_shared", "kv_cache_use_tot", "hidden_cache_use_tot")
    O.mixed_kv_to_cache(key, value, *ref, *(t64(md[n]) for n in names))
    g = [c.to(dev) for c in caches]
    gkv = kv.to(dev)
    gk, gv = (x.view(T, H, D) for x in gkv.chunk(2, dim=-1))
    mixed_cache_ops.mixed_kv_to_cache(gk, gv, *g, *(idx(md, n, dev) for n in names))
    for a, r in zip(g, ref):
        assert bits_equal(a, r)


def test_mixed_kv_to_cache_literal_modulo_and_skip_mirror(dev):
    H, D, N, BS = 2, 8, 24, 16
    b = workloads.small_decode_batch(5, 4, 30, 0.75, N)
    md = oracle_metadata(b)
    nkv, nh = len(md["kv_cache_use_tot"]), len(md["slot_mapping_shared"])
    assert nkv > 0 and nh > 2 * nkv
    T = md["num_tot_tokens"]
    key, value = randn((T, H, D), 1), randn((T, H, D), 2)
    caches = [sentinel_cache((n, BS, H, D), seed=i) for i, n in enumerate((N, N, 2 * N, 2 * N))]
    names = ("slot_mapping", "slot_mapping_shared", "kv_cache_use_tot", "hidden_cache_use_tot")
    ref = [c.clone() for c in caches]
    O.mixed_kv_to_cache(key, value, *ref, *(t64(md[n]) for n in names), literal_modulo=True)
    g = [c.to(dev) for c in caches]
    ops.mixed_kv_to_cache(key.to(dev), value.to(dev), *g, *(idx(md, n, dev) for n in names), literal_modulo=True)
    for a, r in zip(g, ref):
        assert bits_equal(a, r)
    # skip_mirror leaves the shared blocks 0..N-1 alone and writes everything else
    ref2 = [c.clone() for c in caches]
    O.mixed_kv_to_cache(key, value, *ref2, *(t64(md[n]) for n in names))
    g2 = [c.to(dev) for c in caches]
    ops.mixed_kv_to_cache(key.to(dev), value.to(dev), *g2, *(idx(md, n, dev) for n in names), skip_mirror=True)
    assert bits_equal(g2[0], ref2[0]) and bits_equal(g2[1], ref2[1])
    assert bits_equal(g2[2][N:], ref2[2][N:]) and bits_equal(g2[2][:N], caches[2][:N])


# ----------------------------------------------------------------------- fp8

@pytest.mark.parametrize("scale", [1.0, 0.5, 0.0123, 3.7])
def test_fp8_write_every_fp16_value(dev, scale):
    """All 65536 fp16 bit patterns through the quantising write, bit-exact vs the oracle."""
    H, D, BS = 4, 32, 16
    allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    T = 65536 // (H * D)
    key = allv.view(T, H, D)
    value = allv.flip(0).view(T, H, D).contiguous()
    N = T // BS
    slots = t64(np.random.default_rng(0).permutation(N * BS))
    kc = torch.zeros(N, BS, H, D, dtype=torch.uint8); vc = kc.clone()
    O.reshape_and_cache_flash(key, value, kc, vc, slots, "fp8", scale, 2 * scale)
    gk, gv = kc.clone().zero_().to(dev), vc.clone().zero_().to(dev)
    ops.reshape_and_cache_flash(key.to(dev), value.to(dev), gk, gv, slots.to(dev), "fp8", scale, 2 * scale)
    gk, gv = gk.cpu(), gv.cpu()
    finite = ~torch.isnan(key.float())
    fk = finite.view(T, -1)
    ck = kc.view(N * BS, -1)[slots]; cgk = gk.view(N * BS, -1)[slots]
    assert torch.equal(ck[fk], cgk[fk])
    # NaN inputs must produce a NaN code (either sign)
    assert ((cgk[~fk] & 0x7F) == 0x7F).all()
    fv = ~torch.isnan(value.float()).view(T, -1)
    cv = vc.view(N * BS, -1)[slots]; cgv = gv.view(N * BS, -1)[slots]
    assert torch.equal(cv[fv], cgv[fv])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,D", [(2, 16), (1, 5)])
def test_fp8_write_other_input_dtypes_and_unaligned_rows(dev, dtype, H, D):
    N, BS, T = 6, 16, 70
    key = (randn((T, H, D), 0, torch.float32) * 60).to(dtype)
    value = (randn((T, H, D), 1, torch.float32) * 0.01).to(dtype)
    slots = t64(np.random.default_rng(1).permutation(N * BS)[:T])
    kc = torch.full((N, BS, H, D), 0x55, dtype=torch.uint8); vc = kc.clone()
    gk, gv = kc.to(dev), vc.to(dev)
    O.reshape_and_cache_flash(key, value, kc, vc, slots, "fp8", 0.25, 0.001)
    ops.reshape_and_cache_flash(key.to(dev), value.to(dev), gk, gv, slots.to(dev), "fp8", 0.25, 0.001)
    assert bits_equal(gk, kc) and bits_equal(gv, vc)


# ------------------------------------------------------ config 2 at full size

def test_config2_write_and_gather_opt13b_full_size(dev):
    """256 decode sequences at OPT-13B shapes, half hidden-cached: the write of the new
    token and the gather of every hidden context row, against the oracle, bit-exact."""
    H, D, BS = 40, 128, 16
    Hd = H * D
    b = workloads.decode_batch_opt13b(0)
    md = oracle_metadata(b)
    N, B, T = b.num_blocks, len(b.seq_lens), md["num_tot_tokens"]
    assert sum(b.seq_lens) == 167121
    cache = cheap_pattern((2, N, BS, H, D))
    hs = randn((B, Hd), 0)
    sm = t64(md["slot_mapping"])
    g = cache.to(dev)
    ref = cache  # mutated in place below
    O.hidden_to_cache(hs, ref, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    holder_ref = O.assemble_hidden_holder(hs, ref, sm, T, t64(md["hidden_holder_upd"]),
                                          t64(md["hidden_cache_use_tot"]))
    dsm, dhs = sm.to(dev), hs.to(dev)
    # reference op sequence through the drop-in module
    mixed_cache_ops.hidden_to_cache(dhs, g, dsm, idx(md, "hidden_cache_use_input", dev),
                                    idx(md, "hidden_cache_store_tot", dev))
    holder = torch.zeros(T, Hd, dtype=torch.float16, device=dev)
    holder[idx(md, "hidden_holder_upd", dev)] = dhs
    mixed_cache_ops.cache_to_hidden(holder, g, dsm, idx(md, "hidden_cache_use_tot", dev))
    assert bits_equal(holder, holder_ref)
    # fused launch
    g2 = g.clone()
    holder2 = torch.empty(T, Hd, dtype=torch.float16, device=dev)
    ops.hybrid_decode_gather(holder2, dhs, g2, dsm, idx(md, "hidden_holder_upd", dev),
                             idx(md, "hidden_holder_pull", dev), idx(md, "hidden_cache_use_input", dev),
                             idx(md, "hidden_cache_store_tot", dev))
    assert torch.equal(holder2, holder)
    from aptserve_hip import metadata
    gmd = metadata.build_from_batch(b, dev)
    holder3 = torch.empty(T, Hd, dtype=torch.float16, device=dev)
    ops.gather_hidden_rows(holder3, dhs, g2, gmd.holder_src, gmd.slot_mapping, gmd.hidden_cache_use_input,
                           gmd.hidden_cache_store_tot)
    assert torch.equal(holder3, holder)
    del holder2, holder, holder3
    assert torch.equal(g2, g)
    del g2
    # checksum of the whole cache instead of shipping 4 GB back
    assert int(g.view(torch.int16).sum(dtype=torch.int64)) == int(ref.view(torch.int16).sum(dtype=torch.int64))
    # K/V write of the new token of the K/V-cached half
    kv = randn((B, 2 * Hd), 1)
    k, v = (x.view(B, H, D) for x in kv.chunk(2, -1))
    kv_seq = torch.tensor([not h for h in b.use_hidden])
    seq_idx = torch.nonzero(kv_seq).flatten()
    slots = sm[t64(md["kv_cache_use_tot"])]
    O.reshape_and_cache_flash(k[seq_idx], v[seq_idx], ref[0], ref[1], slots, "auto")
    dkv = kv.to(dev)
    dk, dv = (x.view(B, H, D) for x in dkv.chunk(2, -1))
    full_slots = torch.full((B,), -1, dtype=torch.int64)
    full_slots[seq_idx] = slots
    ops.reshape_and_cache_flash(dk, dv, g[0], g[1], full_slots.to(dev), "auto", token_idx=seq_idx.to(dev))
    rows = torch.cat([slots, slots + N * BS])
    assert bits_equal(g.view(-1, Hd)[rows.to(dev)], ref.view(-1, Hd)[rows])
    assert int(g.view(torch.int16).sum(dtype=torch.int64)) == int(ref.view(torch.int16).sum(dtype=torch.int64))
    # the whole step as one launch on a second copy of the initial cache: same cache bytes, same holder
    g3 = cheap_pattern((2, N, BS, H, D)).to(dev)
    holder4 = torch.empty(T, Hd, dtype=torch.float16, device=dev)
    ops.decode_step_cache_ops(holder4, dhs, g3, gmd.holder_src, gmd.slot_mapping, gmd.hidden_cache_use_input,
                              gmd.hidden_cache_store_tot, dk, dv, gmd.kv_cache_use_input, gmd.new_token_slot)
    assert torch.equal(g3, g)
    del g3
    assert bits_equal(holder4, holder_ref)


# --------------------------------------------------------------- error paths

def test_argument_validation_raises_before_launch(dev):
    H, D, N, BS = 2, 4, 4, 16
    cache = torch.zeros(2, N, BS, H, D, dtype=torch.float16, device=dev)
    hidden = torch.zeros(3, 8, dtype=torch.float16, device=dev)
    i64 = t64([0, 1, 2], dev)
    with pytest.raises(ValueError):
        ops.hidden_to_cache(hidden.float(), cache, i64, i64, i64)            # dtype mismatch
    with pytest.raises(ValueError):
        ops.hidden_to_cache(hidden, cache, i64.int(), i64, i64)              # int32 indices
    with pytest.raises(ValueError):
        ops.hidden_to_cache(hidden.cpu(), cache, i64, i64, i64)              # host tensor
    with pytest.raises(ValueError):
        ops.hidden_to_cache(hidden, cache[:, :, :, :1], i64, i64, i64)       # non-contiguous cache
    with pytest.raises(ValueError):
        ops.cache_to_hidden(hidden.t(), cache, i64, i64)                     # strided innermost dim
    k = torch.zeros(3, H, D, dtype=torch.float16, device=dev)
    kc = torch.zeros(N, BS, H, D, dtype=torch.float16, device=dev)
    pad = torch.zeros(N, BS + 1, H, D, dtype=torch.float16, device=dev)[:, :BS]
    with pytest.raises(RuntimeError):                                        # the reference's TORCH_CHECK
        ops.mixed_kv_to_cache(k, k, kc, pad, kc, kc, i64, i64[:0], i64, i64[:0])
    with pytest.raises(ValueError):
        ops.reshape_and_cache_flash(k, k, kc, kc, i64, "int4")


def test_empty_inputs_are_noops(dev):
    H, D, N, BS = 2, 4, 4, 16
    cache = sentinel_cache((2, N, BS, H, D)).to(dev); before = cache.clone()
    hidden = torch.zeros(0, 8, dtype=torch.float16, device=dev)
    e = t64([], dev)
    ops.hidden_to_cache(hidden, cache, e, e, e)        # the reference would launch a zero-sized grid
    ops.cache_to_hidden(hidden, cache, e, e)
    k = torch.zeros(0, H, D, dtype=torch.float16, device=dev)
    ops.reshape_and_cache_flash(k, k, cache[0], cache[1], e, "auto")
    ops.mixed_kv_to_cache(k, k, cache[0], cache[1], cache[0], cache[1], e, e, e, e)
    torch.cuda.synchronize()
    assert torch.equal(cache, before)
