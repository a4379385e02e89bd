"""Pins the cache-operator oracle with witnesses that do not share its code.

The witness is a literal walk over the reference kernels' launch grid — one
Python iteration per CUDA block and per thread step, flat offsets computed the
way the kernels compute them (mixed_cache.cu:6-116) — plus properties the
operators must have whatever their implementation.
"""
import numpy as np
import pytest
import torch

from aptserve_hip import workloads
from oracle import cache_ops
from util import oracle_metadata, randn, sentinel_cache, t64, bits_equal


def grid_walk_hidden_to_cache(hidden, cache, slot_mapping, src_idx, tgt_idx):
    flat = cache.view(-1)
    hs, stride_h, stride_s = hidden.size(1), hidden.stride(0), cache.stride(2)
    hflat = hidden.reshape(-1) if hidden.is_contiguous() else None
    for blk in range(len(src_idx)):
        tok = int(src_idx[blk]); slot = int(slot_mapping[int(tgt_idx[blk])])
        if slot < 0:
            continue
        for i in range(hs):
            flat[slot * stride_s + i % hs] = hidden[tok, i] if hflat is None else hflat[tok * stride_h + i]


def grid_walk_cache_to_hidden(hidden, cache, slot_mapping, dst_idx):
    flat = cache.view(-1)
    hs, stride_s = hidden.size(1), cache.stride(2)
    for blk in range(len(dst_idx)):
        tok = int(dst_idx[blk]); slot = int(slot_mapping[tok])
        if slot < 0:
            continue
        for i in range(hs):
            hidden[tok, i] = flat[slot * stride_s + i % hs]


def grid_walk_mixed_kv(key, value, kc, vc, skc, svc, sm, sms, kv_use, hid_use):
    nkv, nh = len(kv_use), len(sms)
    H, D, BS = key.size(1), key.size(2), kc.size(1)
    bstride = kc.stride(0)
    kcf, vcf, skcf, svcf = (c.view(-1) for c in (kc, vc, skc, svc))
    for blk in range(2 * nkv + nh):
        tok = slot = -1
        if blk < nkv:
            tok = int(kv_use[blk]); slot = int(sm[tok])
        if nkv <= blk < 2 * nkv:
            tok = int(kv_use[blk % nkv]); slot = int(sm[tok])
        if blk >= 2 * nkv:
            off = blk % (2 * nkv)          # the literal arithmetic of mixed_cache.cu:88
            tok = int(hid_use[off]); slot = int(sms[off])
        if slot < 0:
            continue
        b, o = slot // BS, slot % BS
        for i in range(H * D):
            tgt = b * bstride + o * H * D + (i // D) * D + i % D
            if blk < nkv:
                kcf[tgt] = key[tok].reshape(-1)[i]; vcf[tgt] = value[tok].reshape(-1)[i]
            else:
                skcf[tgt] = key[tok].reshape(-1)[i]; svcf[tgt] = value[tok].reshape(-1)[i]


def small_decode(seed, hidden_fraction=0.5, batch=5, max_len=37, N=24):
    b = workloads.small_decode_batch(seed, batch, max_len, hidden_fraction, N)
    return b, oracle_metadata(b)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_hidden_to_cache_matches_grid_walk(seed):
    H, D, N, BS = 2, 4, 24, 16
    b, md = small_decode(seed)
    hidden = randn((len(b.seq_lens), H * D), seed)
    c1 = sentinel_cache((2, N, BS, H, D)); c2 = c1.clone()
    args = (t64(md["slot_mapping"]), t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    cache_ops.hidden_to_cache(hidden, c1, *args)
    grid_walk_hidden_to_cache(hidden, c2, *args)
    assert bits_equal(c1, c2)
    # something was written, and only where expected
    n_rows = len(md["hidden_cache_use_input"])
    changed = (c1 != sentinel_cache((2, N, BS, H, D))).view(-1, H * D).any(1).sum().item()
    assert 0 < changed <= n_rows


def test_hidden_rows_land_in_v_plane_for_odd_logical_blocks():
    # a hidden sequence of 20 tokens uses logical blocks 0 (block p, K plane) and 1 (p+N, V plane)
    H, D, N, BS = 2, 4, 8, 16
    p = 5
    slot_mapping = t64([p * BS + j for j in range(16)] + [(p + N) * BS + j for j in range(4)])
    hidden = randn((20, H * D), 7)
    cache = torch.zeros(2, N, BS, H, D, dtype=torch.float16)
    idx = t64(range(20))
    cache_ops.hidden_to_cache(hidden, cache, slot_mapping, idx, idx)
    assert torch.equal(cache[0, p].reshape(16, -1), hidden[:16])
    assert torch.equal(cache[1, p, :4].reshape(4, -1), hidden[16:])
    assert cache[1, p, 4:].abs().sum() == 0 and cache[0, :p].abs().sum() == 0


@pytest.mark.parametrize("seed", [0, 3])
def test_cache_to_hidden_matches_grid_walk_and_inverts_the_write(seed):
    H, D, N, BS = 2, 4, 24, 16
    b, md = small_decode(seed)
    T = md["num_tot_tokens"]
    cache = sentinel_cache((2, N, BS, H, D))
    sm, use_tot = t64(md["slot_mapping"]), t64(md["hidden_cache_use_tot"])
    h1 = torch.zeros(T, H * D, dtype=torch.float16); h2 = h1.clone()
    cache_ops.cache_to_hidden(h1, cache, sm, use_tot)
    grid_walk_cache_to_hidden(h2, cache, sm, use_tot)
    assert bits_equal(h1, h2)
    # write -> gather is the identity on the rows that were written
    rows = randn((T, H * D), seed + 10)
    cache_ops.hidden_to_cache(rows, cache, sm, use_tot, use_tot)
    back = torch.zeros_like(rows)
    cache_ops.cache_to_hidden(back, cache, sm, use_tot)
    assert torch.equal(back[use_tot], rows[use_tot])
    kv = t64(md["kv_cache_use_tot"])
    assert back[kv].abs().sum() == 0


def test_padding_slots_are_skipped():
    H, D, N, BS = 1, 8, 4, 16
    cache = sentinel_cache((2, N, BS, H, D)); ref = cache.clone()
    sm = t64([-1, 3, -1])
    hidden = randn((3, 8), 0)
    cache_ops.hidden_to_cache(hidden, cache, sm, t64([0, 1, 2]), t64([0, 1, 2]))
    ref.view(-1, 8)[3] = hidden[1]
    assert bits_equal(cache, ref)
    out = torch.full((3, 8), 9.0, dtype=torch.float16)
    cache_ops.cache_to_hidden(out, cache, sm, t64([0, 1, 2]))
    assert torch.equal(out[1], hidden[1]) and (out[0] == 9).all() and (out[2] == 9).all()


@pytest.mark.parametrize("seed,frac", [(0, 0.4), (1, 0.2), (2, 0.34), (7, 0.4)])
def test_mixed_kv_matches_grid_walk_when_modulo_is_harmless(seed, frac):
    H, D, N, BS = 2, 4, 24, 16
    b, md = small_decode(seed, frac, batch=6, max_len=5)
    nkv, nh = len(md["kv_cache_use_tot"]), len(md["slot_mapping_shared"])
    assert nkv > 0 and 0 < nh <= 2 * nkv
    T = md["num_tot_tokens"]
    key, value = randn((T, H, D), seed), randn((T, H, D), seed + 50)
    mk = lambda n: sentinel_cache((n, BS, H, D), seed=n)
    a = [mk(N), mk(N + 1)[:N], mk(2 * N), mk(2 * N + 1)[:2 * N]]
    a = [x.contiguous() for x in a]
    bb = [x.clone() for x in a]
    idx = (t64(md["slot_mapping"]), t64(md["slot_mapping_shared"]), t64(md["kv_cache_use_tot"]),
           t64(md["hidden_cache_use_tot"]))
    cache_ops.mixed_kv_to_cache(key, value, *a, *idx)
    grid_walk_mixed_kv(key, value, *bb, *idx)
    for x, y in zip(a, bb):
        assert bits_equal(x, y)


def test_mixed_kv_literal_modulo_reproduces_the_reference_wrap():
    # nh > 2*nkv: the reference's offsets wrap (mixed_cache.cu:88)
    H, D, N, BS = 1, 4, 24, 16
    b, md = small_decode(5, 0.75, batch=4, max_len=30)
    nkv, nh = len(md["kv_cache_use_tot"]), len(md["slot_mapping_shared"])
    assert nkv > 0 and nh > 2 * nkv
    T = md["num_tot_tokens"]
    key, value = randn((T, H, D), 1), randn((T, H, D), 2)
    caches = [sentinel_cache((n, BS, H, D), seed=n) for n in (N, N, 2 * N, 2 * N)]
    lit = [x.clone() for x in caches]; walk = [x.clone() for x in caches]; intended = [x.clone() for x in caches]
    idx = (t64(md["slot_mapping"]), t64(md["slot_mapping_shared"]), t64(md["kv_cache_use_tot"]),
           t64(md["hidden_cache_use_tot"]))
    cache_ops.mixed_kv_to_cache(key, value, *lit, *idx, literal_modulo=True)
    grid_walk_mixed_kv(key, value, *walk, *idx)
    cache_ops.mixed_kv_to_cache(key, value, *intended, *idx)
    for x, y in zip(lit, walk):
        assert bits_equal(x, y)
    # the intended semantics writes every hidden row; the literal one does not
    assert not bits_equal(lit[2], intended[2])
    sms = idx[1]
    got = intended[2].view(-1, H * D)[sms]
    assert torch.equal(got, key[idx[3]].reshape(nh, -1))


def test_reshape_and_cache_flash_closed_form():
    H, D, N, BS = 3, 8, 10, 16
    T = 40
    g = np.random.default_rng(0)
    slots = g.permutation(N * BS)[:T].astype(np.int64)
    slots[[3, 17]] = -1
    key, value = randn((T, H, D), 0), randn((T, H, D), 1)
    kc, vc = sentinel_cache((N, BS, H, D)), sentinel_cache((N, BS, H, D), seed=2)
    kref, vref = kc.clone(), vc.clone()
    cache_ops.reshape_and_cache_flash(key, value, kc, vc, t64(slots), "auto")
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        for h in range(H):
            for d in range(D):
                kref[s // BS, s % BS, h, d] = key[t, h, d]
                vref[s // BS, s % BS, h, d] = value[t, h, d]
    assert bits_equal(kc, kref) and bits_equal(vc, vref)


def test_reshape_and_cache_flash_with_only_padding_slots_stores_nothing():
    """Every slot is the padding value -1 (a step whose tokens all belong elsewhere): the caches stay as they are."""
    key, value = randn((3, 2, 4), 0), randn((3, 2, 4), 1)
    kc, vc = sentinel_cache((2, 16, 2, 4)), sentinel_cache((2, 16, 2, 4), seed=2)
    k0, v0 = kc.clone(), vc.clone()
    cache_ops.reshape_and_cache_flash(key, value, kc, vc, t64([-1, -1, -1]), "auto")
    assert bits_equal(kc, k0) and bits_equal(vc, v0)


def test_holder_assembly_equals_rows_by_definition():
    H, D, N, BS = 2, 4, 24, 16
    b, md = small_decode(4, 0.5, batch=6, max_len=40)
    B, T = len(b.seq_lens), md["num_tot_tokens"]
    cache = sentinel_cache((2, N, BS, H, D))
    hs = randn((B, H * D), 3)
    sm = t64(md["slot_mapping"])
    cache_ops.hidden_to_cache(hs, cache, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    holder = cache_ops.assemble_hidden_holder(hs, cache, sm, T, t64(md["hidden_holder_upd"]),
                                              t64(md["hidden_cache_use_tot"]))
    # independent definition: walk the sequences
    row = 0
    flat = cache.view(-1, H * D)
    for i, (L, hid) in enumerate(zip(b.seq_lens, b.use_hidden)):
        if hid:
            for j in range(L):
                blk = b.block_tables[i][j // BS]
                exp = hs[i] if j == L - 1 else flat[blk * BS + j % BS]
                assert torch.equal(holder[row], exp)
                row += 1
        else:
            assert torch.equal(holder[row], hs[i]); row += 1
    assert row == T
