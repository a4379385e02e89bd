"""Seeded random sweeps over shapes, strides, dtypes and index patterns (valid inputs only), every case against the
oracle.  The fixed-size tests elsewhere pin the named configurations; these walk the space between them: a sweep
of this kind found reads past the end of strided activations that no fixed shape had hit."""
import numpy as np
import pytest
import torch

import mixed_cache_ops
from aptserve_hip import metadata, ops, workloads
from oracle import cache_ops as O
from oracle import fp8 as O8
from oracle import reproject as OR
import test_attention_gpu as TA
import test_prefill_attention_gpu as TP
import test_reproject_gpu as TR
from test_metadata_gpu import assert_same
from util import bits_equal, oracle_metadata, randn, sentinel_cache, t64

pytestmark = pytest.mark.gpu

DT16 = [torch.float16, torch.bfloat16]


@pytest.mark.parametrize("seed", [11, 12])
def test_projection_family_random_shapes(dev, seed):
    rng = np.random.default_rng(seed)
    rows = [1, 2, 3, 5, 8, 9, 16, 17, 31, 48, 49, 63, 64, 65, 100, 128, 129, 200, 256, 257, 300, 511, 513, 900]
    for case in range(90):
        s = int(rng.integers(0, 10000))
        M = int(rng.choice(rows)); N = 256 * int(rng.integers(1, 7)); K = 64 * int(rng.integers(1, 22))
        dtype = DT16[int(rng.integers(0, 2))]
        use_map, strided, bias, sk = (bool(rng.integers(0, 2)) for _ in range(4))
        relu = bool(rng.integers(0, 3) == 0)
        xs = randn((M, 2 * K if strided else K), s, dtype)
        x = xs[:, K:] if strided else xs
        w = (randn((N, K), s + 1) * 0.05).to(dtype)
        b = randn((N,), s + 2, dtype) if bias else None
        ref = OR._linear_fp32(x, w, b)
        if relu:     # fc1 with its activation: max(., 0) of the rounded product
            ref = torch.relu(ref)
        dx = xs.to(dev)[:, K:] if strided else xs.to(dev)
        db = None if b is None else b.to(dev)
        what = f"case {case}: M={M} N={N} K={K} {dtype} map={use_map} strided={strided} bias={bias} split_k={sk} relu={relu}"
        try:
            if use_map:
                n_out = M + 7
                perm = rng.permutation(n_out)[:M]
                out = torch.full((n_out, N), 5.0, dtype=dtype, device=dev)
                ops.linear_nt(dx, w.to(dev), db, out=out, out_row_map=torch.from_numpy(perm).to(dev), split_k=sk, relu=relu)
                TR.check(out.cpu()[perm], ref, dtype)
                assert (out.cpu()[np.setdiff1d(np.arange(n_out), perm)] == 5).all()
            else:
                TR.check(ops.linear_nt(dx, w.to(dev), db, split_k=sk, relu=relu), ref, dtype)
        except AssertionError as e:
            raise AssertionError(f"{what}: {e}") from e


@pytest.mark.parametrize("seed", [21])
def test_projection_into_cache_slots_random_shapes(dev, seed):
    rng = np.random.default_rng(seed)
    H, D, BS = 4, 64, 16
    Hd = H * D
    for case in range(40):
        s = int(rng.integers(0, 10000))
        T = int(rng.choice([1, 3, 17, 48, 50, 64, 65, 130, 300, 700]))
        dtype = DT16[int(rng.integers(0, 2))]
        nblk = T // BS + 6
        x = randn((T, Hd), s, dtype)
        w = (randn((2 * Hd, Hd), s + 1) * 0.05).to(dtype)
        b = randn((2 * Hd,), s + 2, dtype)
        dest = rng.permutation(nblk * BS)[:T].astype(np.int64)
        wk = torch.full((nblk, BS, H, D), 3.0, dtype=dtype, device=dev)
        wv = torch.full_like(wk, 3.0)
        ops.kv_reproject_to_cache(x.to(dev), w.to(dev), b.to(dev), wk, wv, None, None, torch.from_numpy(dest).to(dev))
        plain = ops.linear_nt(x.to(dev), w.to(dev), b.to(dev)).cpu()
        assert torch.equal(wk.cpu().view(-1, Hd)[dest], plain[:, :Hd]), f"case {case}: T={T} {dtype}"
        assert torch.equal(wv.cpu().view(-1, Hd)[dest], plain[:, Hd:]), f"case {case}: T={T} {dtype}"
        TR.check(plain, OR._linear_fp32(x, w, b), dtype)


@pytest.mark.parametrize("seed", [31])
def test_attention_random_shapes(dev, seed):
    rng = np.random.default_rng(seed)
    for case in range(60):
        B = int(rng.integers(1, 30)); H = int(rng.choice([1, 2, 4, 6, 8])); D = int(rng.choice([32, 64, 128, 256]))
        BS = int(rng.choice([16, 32])); dtype = DT16[int(rng.integers(0, 2))]
        mx = int(rng.choice([1, 20, 100, 600, 2100]))
        lens = [int(v) for v in rng.integers(0, mx + 1, B)]
        hybrid = bool(rng.integers(0, 2)); fp8 = bool(rng.integers(0, 2)) and D != 32
        ps = int(rng.choice([0, 16, 32, 64, 256, 512, 1024])); ps = ps if ps % BS == 0 else 0
        c = TA.make_case(B, H, D, BS, lens, int(rng.integers(0, 10000)), dtype, hybrid=hybrid)
        kw = {}
        if fp8:
            for k in ("kc", "vc", "wk", "wv"):
                if k in c:
                    c[k] = O8.quantize_e4m3(c[k], 0.05 if k in ("kc", "wk") else 0.03)
            kw = dict(k_scale=0.05, v_scale=0.03)
        out, ref = TA.run_both(c, dev, ps, **kw)
        try:
            TA.check(out, ref, dtype)
        except AssertionError as e:
            raise AssertionError(f"case {case}: B={B} H={H} D={D} BS={BS} {dtype} max={mx} hybrid={hybrid} fp8={fp8} "
                                 f"partition={ps}: {e}") from e
    for case in range(25):   # prompt attention
        ns = int(rng.integers(1, 6)); mx = int(rng.choice([3, 40, 200, 700]))
        lens = [int(v) for v in rng.integers(1, mx + 1, ns)]
        TP.run(dev, lens, int(rng.choice([1, 2, 5])), int(rng.choice([64, 128])), DT16[int(rng.integers(0, 2))],
               int(rng.integers(0, 10000)), bool(rng.integers(0, 2)))


@pytest.mark.parametrize("seed", [41])
def test_row_movers_random_shapes(dev, seed):
    rng = np.random.default_rng(seed)
    dts = [torch.float16, torch.bfloat16, torch.float32]
    for case in range(120):
        kind = int(rng.integers(0, 4)); s = int(rng.integers(0, 10000))
        H = int(rng.choice([1, 2, 3, 5, 12, 40])); D = int(rng.choice([1, 2, 3, 4, 5, 8, 24, 64, 80, 128]))
        if H * D > 5120:
            D = 64
        Hd = H * D; dtype = dts[int(rng.integers(0, 3))]; BS = int(rng.choice([16, 32]))
        what = f"case {case}: kind={kind} H={H} D={D} {dtype} BS={BS} seed={s}"
        if kind == 0:     # hidden rows out of a strided tensor into the cache and back
            B = int(rng.integers(1, 20)); mx = int(rng.choice([3, 40, 200])); frac = float(rng.choice([0.0, 0.5, 1.0]))
            N = B * (mx // BS + 2) + 4
            b = workloads.small_decode_batch(s, B, mx, frac, N, BS); md = oracle_metadata(b)
            wide = randn((len(b.seq_lens), 3 * Hd), s, dtype); col = int(rng.integers(0, 3)) * Hd
            cache = sentinel_cache((2, N, BS, H, D), dtype); ref = cache.clone(); sm = t64(md["slot_mapping"])
            O.hidden_to_cache(wide[:, col:col + Hd], ref, sm, t64(md["hidden_cache_use_input"]),
                              t64(md["hidden_cache_store_tot"]))
            g = cache.to(dev)
            ops.hidden_to_cache(wide.to(dev)[:, col:col + Hd], g, sm.to(dev), t64(md["hidden_cache_use_input"], dev),
                                t64(md["hidden_cache_store_tot"], dev))
            assert bits_equal(g, ref), what
            hold_ref = sentinel_cache((md["num_tot_tokens"], Hd), dtype, seed=9); hold = hold_ref.to(dev)
            O.cache_to_hidden(hold_ref, ref, sm, t64(md["hidden_cache_use_tot"]))
            ops.cache_to_hidden(hold, g, sm.to(dev), t64(md["hidden_cache_use_tot"], dev))
            assert bits_equal(hold, hold_ref), what
        elif kind == 1:   # K/V write from chunk views, padding slots
            N = int(rng.integers(2, 30)); T = int(rng.integers(1, N * BS + 1))
            slots = rng.permutation(N * BS)[:T].astype(np.int64); slots[rng.random(T) < 0.1] = -1
            qkv = randn((T, 3 * Hd), s, dtype)
            kc, vc = sentinel_cache((N, BS, H, D), dtype), sentinel_cache((N, BS, H, D), dtype, seed=2)
            kr, vr = kc.clone(), vc.clone()
            O.reshape_and_cache_flash(qkv[:, Hd:2 * Hd].view(T, H, D), qkv[:, 2 * Hd:].view(T, H, D), kr, vr, t64(slots),
                                      "auto")
            gq = qkv.to(dev); gkc, gvc = kc.to(dev), vc.to(dev)
            ops.reshape_and_cache_flash(gq[:, Hd:2 * Hd].view(T, H, D), gq[:, 2 * Hd:].view(T, H, D), gkc, gvc,
                                        t64(slots, dev), "auto")
            assert bits_equal(gkc, kr) and bits_equal(gvc, vr), what
        elif kind == 2:   # the three-range K/V scatter of a mixed decode batch
            B = int(rng.integers(1, 14)); mx = int(rng.choice([3, 30, 90])); frac = float(rng.choice([0.2, 0.5, 1.0]))
            N = B * (mx // BS + 2) + 4
            dt = torch.float16 if dtype == torch.float32 else dtype
            b = workloads.small_decode_batch(s, B, mx, frac, N, BS); md = oracle_metadata(b); T = md["num_tot_tokens"]
            kv = randn((T, 2 * Hd), s, dt)
            caches = [sentinel_cache((m, BS, H, D), dt, seed=i) for i, m in enumerate((N, N, 2 * N, 2 * N))]
            ref = [c.clone() for c in caches]
            names = ("slot_mapping", "slot_mapping_shared", "kv_cache_use_tot", "hidden_cache_use_tot")
            O.mixed_kv_to_cache(*(x.view(T, H, D) for x in kv.chunk(2, dim=-1)), *ref, *(t64(md[k]) for k in names))
            g = [c.to(dev) for c in caches]; gkv = kv.to(dev)
            mixed_cache_ops.mixed_kv_to_cache(*(x.view(T, H, D) for x in gkv.chunk(2, dim=-1)), *g,
                                              *(t64(md[k], dev) for k in names))
            assert all(bits_equal(a, r) for a, r in zip(g, ref)), what
        else:             # one write by token type in a prompt step
            B = int(rng.integers(1, 10)); mx = int(rng.choice([3, 40, 150])); frac = float(rng.choice([0.0, 0.4, 1.0]))
            N = B * (mx // BS + 2) + 4
            b = workloads.small_prefill_batch(s, B, mx, frac, N, BS); md = oracle_metadata(b); T = md["num_tot_tokens"]
            qkv = randn((T, 3 * Hd), s, dtype); hidden = randn((T, Hd), s + 1, dtype)
            mask = torch.zeros(T, dtype=torch.uint8); mask[torch.from_numpy(md["hidden_cache_use_tot"])] = 1
            cache = sentinel_cache((2, N, BS, H, D), dtype); ref = cache.clone(); sm = t64(md["slot_mapping"])
            O.mixed_reshape_and_cache(qkv[:, Hd:2 * Hd].view(T, H, D), qkv[:, 2 * Hd:].view(T, H, D), hidden, ref, sm, mask)
            g = cache.to(dev); gq = qkv.to(dev)
            ops.mixed_reshape_and_cache(gq[:, Hd:2 * Hd].view(T, H, D), gq[:, 2 * Hd:].view(T, H, D), hidden.to(dev), g,
                                        sm.to(dev), mask.to(dev))
            assert bits_equal(g, ref), what


@pytest.mark.parametrize("seed", [51])
def test_metadata_random_batches(dev, seed):
    rng = np.random.default_rng(seed)
    for case in range(60):
        B = int(rng.choice([1, 2, 9, 64, 300])); mx = int(rng.choice([3, 50, 400])); frac = float(rng.choice([0.0, 0.3, 1.0]))
        prompt = bool(rng.integers(0, 2)); bs = int(rng.choice([16, 32])); s = int(rng.integers(0, 10000))
        nb = B * (mx // bs + 2) + 8
        batch = (workloads.small_prefill_batch if prompt else workloads.small_decode_batch)(s, B, mx, frac, nb, bs)
        for packed in (False, True):
            md = metadata.build_from_batch(batch, dev, packed=packed, check_totals=True)
            assert_same(md, oracle_metadata(batch))


@pytest.mark.parametrize("seed", [61])
def test_attention_on_hidden_rows_random_batches(dev, seed):
    """Batches of hidden-cached sequences of random number and lengths: few rows (a chunk of tokens per workgroup of
    the weighted sum), more (the streaming kernel, token partitions), head layouts 4x64 .. 40x128."""
    import test_absorbed_attention_gpu as TAB
    rng = np.random.default_rng(seed)
    for case in range(14):
        H, D = [(4, 64), (12, 64), (8, 128), (40, 128)][int(rng.integers(0, 4))]
        n = int(rng.integers(1, 9))
        hi = int(rng.choice([30, 97, 200, 700]))
        lens = [int(x) for x in rng.integers(1, hi + 1, n)]
        dtype = DT16[int(rng.integers(0, 2))]
        N = 2 * sum(-(-l // 16) for l in lens) + 8
        try:
            TAB.run_case(dev, H, D, n, 1.0, max(lens), N, dtype=dtype, seed=int(rng.integers(0, 1000)), lens=lens)
        except AssertionError as e:
            raise AssertionError(f"case {case}: H={H} D={D} lens={lens} {dtype}: {e}") from e


@pytest.mark.parametrize("seed", [71])
def test_prefix_attention_random_batches(dev, seed):
    """Prompt chunks of random lengths behind cached prefixes of random lengths (none included), both block sizes."""
    rng = np.random.default_rng(seed)
    for case in range(12):
        H, D = [(2, 64), (5, 128), (12, 64)][int(rng.integers(0, 3))]
        B = int(rng.integers(1, 6))
        qlens = [int(x) for x in rng.integers(1, int(rng.choice([8, 70, 300])) + 1, B)]
        ctx = [int(x) for x in rng.integers(0, int(rng.choice([1, 40, 500])) + 1, B)]
        klens = [q + c for q, c in zip(qlens, ctx)]
        dtype = DT16[int(rng.integers(0, 2))]
        try:
            TP.run_prefix(dev, klens, qlens, H, D, dtype, seed=int(rng.integers(0, 1000)), BS=int(rng.choice([16, 32])))
        except AssertionError as e:
            raise AssertionError(f"case {case}: H={H} D={D} klens={klens} qlens={qlens} {dtype}: {e}") from e


@pytest.mark.parametrize("seed", [81])
def test_add_layer_norm_random_shapes(dev, seed):
    import torch.nn.functional as F
    rng = np.random.default_rng(seed)
    for case in range(30):
        rows = int(rng.integers(1, 40)); width = 8 * int(rng.integers(1, 2049))
        dtype = DT16[int(rng.integers(0, 2))]
        strided, with_res = bool(rng.integers(0, 2)), bool(rng.integers(0, 4))
        wide = randn((rows, 2 * width), case, dtype).to(dev)
        x = wide[:, :width] if strided else wide[:, :width].contiguous()
        r = (wide[:, width:] if strided else wide[:, width:].contiguous()) if with_res else None
        w, b = (1 + 0.1 * randn((width,), case + 1)).to(dtype).to(dev), (0.1 * randn((width,), case + 2)).to(dtype).to(dev)
        normed, s_ = ops.add_layer_norm(x, r, w, b)
        s_ref = (x.float() + r.float()).to(dtype) if with_res else x
        assert bits_equal(s_, s_ref), f"case {case}: rows={rows} width={width} {dtype} strided={strided}: sum differs"
        n_ref = F.layer_norm(s_ref.float(), (width,), w.float(), b.float(), 1e-5)
        ulp = 2 ** -10 if dtype == torch.float16 else 2 ** -7
        d = (normed.float() - n_ref).abs()
        assert (d <= ulp * n_ref.abs() + 2e-3).all(), f"case {case}: rows={rows} width={width} {dtype}: {d.max().item()}"


@pytest.mark.parametrize("seed", [91])
def test_decode_step_cache_ops_random_batches(dev, seed):
    """One launch for a decode layer's cache traffic (hidden stores, holder, new K/V rows) on random batches, with and
    without a holder, against the oracle's separate operators."""
    rng = np.random.default_rng(seed)
    for case in range(16):
        H, D = [(1, 8), (4, 32), (12, 64), (5, 128)][int(rng.integers(0, 4))]
        N, BS = 96, 16
        dtype = DT16[int(rng.integers(0, 2))]
        b = workloads.small_decode_batch(int(rng.integers(0, 1000)), int(rng.integers(1, 12)), int(rng.integers(1, 120)),
                                         float(rng.choice([0.0, 0.5, 1.0])), N)
        md, gmd = oracle_metadata(b), metadata.build_from_batch(b, dev)
        B, T, Hd = len(b.seq_lens), md["num_tot_tokens"], H * D
        hs, kv = randn((B, Hd), case, dtype), randn((B, 2 * Hd), case + 7, dtype)
        k, v = kv.chunk(2, -1)
        cache = sentinel_cache((2, N, BS, H, D), dtype)
        ref = cache.clone()
        sm = t64(md["slot_mapping"])
        O.hidden_to_cache(hs, ref, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
        holder_ref = O.assemble_hidden_holder(hs, ref, sm, T, t64(md["hidden_holder_upd"]), t64(md["hidden_cache_use_tot"]))
        seq_idx = torch.tensor([i for i, h in enumerate(b.use_hidden) if not h], dtype=torch.int64)
        if len(seq_idx):
            O.reshape_and_cache_flash(k[seq_idx].reshape(-1, H, D), v[seq_idx].reshape(-1, H, D), ref[0], ref[1],
                                      sm[t64(md["kv_cache_use_tot"])], "auto")
        with_holder = bool(rng.integers(0, 2)) and T > 0
        g = cache.to(dev)
        holder = sentinel_cache((T, Hd), dtype, seed=5).to(dev) if with_holder else None
        dk, dv = kv.to(dev).chunk(2, -1)
        ops.decode_step_cache_ops(holder, hs.to(dev), g, gmd.holder_src if with_holder else None, gmd.slot_mapping,
                                  gmd.hidden_cache_use_input, gmd.hidden_cache_store_tot, dk, dv,
                                  gmd.kv_cache_use_input, gmd.new_token_slot)
        what = f"case {case}: H={H} D={D} {dtype} seqs={B} holder={with_holder}"
        assert bits_equal(g, ref), what
        if with_holder:
            assert bits_equal(holder, holder_ref), what


@pytest.mark.parametrize("seed", [101, 102, 103, 104])
def test_one_call_decode_attention_random_batches(dev, seed):
    """Mixed decode batches of random size, mix and lengths: the step's stores, the paged attention of the K/V-cached
    sequences and the attention on hidden rows as ONE call (jobs riding in its launches where they fit, launched by
    themselves where they do not) against the three direct calls: caches and output bit for bit."""
    import test_hybrid_attention_gpu as TH
    rng = np.random.default_rng(seed)
    for case in range(16):
        H, D = [(4, 64), (8, 128), (40, 128), (2, 256)][int(rng.integers(0, 4))]
        B = int(rng.integers(2, 24))
        frac = float(rng.choice([0.2, 0.5, 0.8]))
        max_len = int(rng.choice([20, 150, 600, 1500]))
        dtype = DT16[int(rng.integers(0, 2))]
        what = f"case {case}: H={H} D={D} B={B} frac={frac} max_len={max_len} {dtype}"
        b, md, cache, w, b_v, q = TH._batch(dev, H, D, B, frac, max_len, 2048, dtype, int(rng.integers(0, 1000)))
        n_h = md.num_hidden_cache_tokens
        if n_h == 0 or n_h == len(b.seq_lens):
            continue
        hs, k, v = (randn((len(b.seq_lens), H * D), 40 + case + i, dtype).to(dev) for i in range(3))

        def stores(c, **kw):
            return ops.decode_step_cache_ops(None, hs, c, None, md.slot_mapping, md.hidden_cache_use_input,
                                             md.hidden_cache_store_tot, k, v, md.kv_cache_use_input,
                                             md.new_token_slot, **kw)

        cache_a, want = cache.clone(), torch.full_like(q, 7.0)
        stores(cache_a)
        TH._paged(q, cache_a, md, H, D, want)
        TH._hidden(q, cache_a, md, w, b_v, D, want)
        cache_b, got = cache.clone(), torch.full_like(q, 7.0)
        TH._hidden(q, cache_b, md, w, b_v, D, got, kv_job=TH._paged(q, cache_b, md, H, D, got, as_job=True),
                   store_job=stores(cache_b, as_job=True))
        assert torch.equal(cache_b, cache_a), what + ": caches differ"
        assert torch.equal(got, want), what + ": outputs differ"
