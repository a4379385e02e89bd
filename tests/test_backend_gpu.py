"""Decoder self-attention over the hybrid cache, HIP operators end to end, against the
layer oracle (OPT-125m shapes: 12 heads x 64, hidden 768)."""
import numpy as np
import pytest
import torch

from aptserve_hip import backend, metadata, workloads
from oracle import layer as OL
from util import oracle_metadata, randn

pytestmark = pytest.mark.gpu

H, D, BS, N = 12, 64, 16, 96
Hd = H * D


def weights(seed):
    return ((randn((3 * Hd, Hd), seed) * 0.03).half(), (randn((3 * Hd,), seed + 1) * 0.1).half(),
            (randn((Hd, Hd), seed + 2) * 0.03).half(), (randn((Hd,), seed + 3) * 0.1).half())


def torch_prefill_attention(q, k, v, cu_seqlens, max_seqlen, scale):
    """Prompt attention is not part of the library; the test supplies a plain PyTorch one."""
    out = torch.empty_like(q)
    cu = cu_seqlens.tolist()
    for a, e in zip(cu[:-1], cu[1:]):
        qq, kk, vv = (x[a:e].transpose(0, 1).float() for x in (q, k, v))
        o = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, is_causal=True, scale=scale)
        out[a:e] = o.transpose(0, 1).to(q.dtype)
    return out


def close(a, b, tol=6e-3):
    a, b = a.float().cpu(), b.float().cpu()
    assert (a - b).abs().max().item() <= 2e-2
    assert torch.allclose(a, b, atol=tol, rtol=tol), (a - b).abs().max().item()


@pytest.mark.parametrize("frac", [0.0, 0.4, 1.0])
@pytest.mark.parametrize("fused", [True, "gather-only", False, "absorbed"])
def test_decode_layer_matches_oracle(dev, frac, fused):
    W = weights(0)
    batch = workloads.small_decode_batch(3, 10, 150, frac, N)
    ref_md = oracle_metadata(batch)
    B = len(batch.seq_lens)
    hs = randn((B, Hd), 5)
    kv = randn((2, N, BS, H, D), 6)
    sh = randn((2, 2 * N, BS, H, D), 7)
    ref_kv, ref_sh = kv.clone(), sh.clone()
    ref = OL.opt_attention(hs, ref_kv, ref_sh, ref_md, *W, H)
    layer = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W), fused=bool(fused),
                                       fuse_kv_write=fused is True, absorbed=fused == "absorbed")
    md = metadata.build_from_batch(batch, dev)
    d_kv, d_sh = kv.to(dev), sh.to(dev)
    out = layer(hs.to(dev), d_kv, d_sh, md)
    close(out, ref)
    # persistent cache: bit-exact for the hidden rows (pure copies); K/V rows within GEMM tolerance
    close(d_kv, ref_kv)
    assert torch.equal(d_kv.cpu().view(-1, Hd)[torch.from_numpy(ref_md["slot_mapping"][ref_md["hidden_cache_store_tot"]])],
                       ref_kv.view(-1, Hd)[torch.from_numpy(ref_md["slot_mapping"][ref_md["hidden_cache_store_tot"]])])
    if fused == "absorbed":          # no re-projection: the shared cache is not touched at all
        assert torch.equal(d_sh.cpu(), sh)
        return
    # workspace blocks N..2N-1 hold the re-projected K/V of the hidden sequences
    close(d_sh[:, N:], ref_sh[:, N:])
    # the mirror blocks 0..N-1 are not written by the default data flow
    assert torch.equal(d_sh[:, :N].cpu(), sh[:, :N])


@pytest.mark.parametrize("fused", [True, False, "absorbed"])
def test_decode_layer_matches_oracle_at_opt13b_width(dev, fused):
    """The same check at 40 heads x 128 (hidden 5120): the fused flow, the reference's operator sequence and the
    attention on hidden rows against the layer oracle, on a small mixed batch."""
    h, d, n = 40, 128, 40
    hd = h * d
    sc = 0.03 * (768 / hd) ** 0.5
    W = ((randn((3 * hd, hd), 20) * sc).half(), (randn((3 * hd,), 21) * 0.1).half(),
         (randn((hd, hd), 22) * sc).half(), (randn((hd,), 23) * 0.1).half())
    batch = workloads.small_decode_batch(11, 6, 90, 0.5, n)
    ref_md = oracle_metadata(batch)
    B = len(batch.seq_lens)
    hs = randn((B, hd), 24)
    kv = randn((2, n, BS, h, d), 25)
    sh = randn((2, 2 * n, BS, h, d), 26)
    ref_kv, ref_sh = kv.clone(), sh.clone()
    ref = OL.opt_attention(hs, ref_kv, ref_sh, ref_md, *W, h)
    layer = backend.HybridOPTAttention(hd, h, *(w.to(dev) for w in W), fused=bool(fused),
                                       fuse_kv_write=fused is True, absorbed=fused == "absorbed")
    md = metadata.build_from_batch(batch, dev)
    d_kv, d_sh = kv.to(dev), sh.to(dev)
    out = layer(hs.to(dev), d_kv, d_sh, md)
    close(out, ref)
    close(d_kv, ref_kv)
    if fused != "absorbed":
        close(d_sh[:, n:], ref_sh[:, n:])


@pytest.mark.parametrize("frac", [0.4, 1.0])
def test_fused_kv_write_is_bit_identical_to_the_operator_sequence(dev, frac):
    """Projection with the cache write in its epilogue == projection, chunk, mixed_kv_to_cache."""
    W = weights(1)
    batch = workloads.small_decode_batch(4, 10, 150, frac, N)
    hs = randn((len(batch.seq_lens), Hd), 8)
    kv = randn((2, N, BS, H, D), 9)
    sh = randn((2, 2 * N, BS, H, D), 10)
    md = metadata.build_from_batch(batch, dev)
    res = []
    for fuse in (True, False):
        layer = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W), fuse_kv_write=fuse, holder_free=False)
        d_kv, d_sh = kv.to(dev), sh.to(dev)
        res.append((layer(hs.to(dev), d_kv, d_sh, md).cpu(), d_kv.cpu(), d_sh.cpu()))
    for a, b in zip(*res):
        assert torch.equal(a, b)


@pytest.mark.parametrize("frac", [0.4, 1.0])
@pytest.mark.parametrize("shape", [(12, 64, 150), (40, 128, 700)])
def test_holder_free_reprojection_is_bit_identical_to_the_gathered_holder(dev, frac, shape):
    """The re-projection that fetches cached hidden rows in place (no holder) against the flow that gathers them
    into a holder first: same output, same cache contents, bit for bit.  The second shape (40 x 128, ~3000 rows)
    runs the full-size tiles."""
    h, d, max_len = shape
    hd, n = h * d, 12 * max_len // 16
    sc = 0.03 * (768 / hd) ** 0.5
    W = ((randn((3 * hd, hd), 30) * sc).half(), (randn((3 * hd,), 31) * 0.1).half(),
         (randn((hd, hd), 32) * sc).half(), (randn((hd,), 33) * 0.1).half())
    batch = workloads.small_decode_batch(4, 10, max_len, frac, n)
    hs = randn((len(batch.seq_lens), hd), 34)
    kv = randn((2, n, BS, h, d), 35)
    sh = randn((2, 2 * n, BS, h, d), 36)
    md = metadata.build_from_batch(batch, dev)
    assert md.num_tot_tokens > 48
    res = []
    for holder_free in (True, False):
        layer = backend.HybridOPTAttention(hd, h, *(w.to(dev) for w in W), holder_free=holder_free)
        d_kv, d_sh = kv.to(dev), sh.to(dev)
        res.append((layer(hs.to(dev), d_kv, d_sh, md).cpu(), d_kv.cpu(), d_sh.cpu()))
    for a, b in zip(*res):
        assert torch.equal(a, b)


def test_literal_flow_agrees_where_the_reference_is_well_defined(dev):
    """All-hidden and no-hidden decode batches: the reference's own call pattern and the
    per-block select must give the same answer."""
    W = weights(1)
    for frac in (0.0, 1.0):
        batch = workloads.small_decode_batch(4, 6, 100, frac, N)
        hs = randn((len(batch.seq_lens), Hd), 8)
        kv, sh = randn((2, N, BS, H, D), 9), randn((2, 2 * N, BS, H, D), 10)
        md = metadata.build_from_batch(batch, dev)
        outs = []
        for literal in (False, True):
            layer = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W), literal=literal)
            outs.append(layer(hs.to(dev), kv.to(dev), sh.to(dev), md))
        assert torch.equal(outs[0], outs[1])
    # mixed batch, literal flow: the oracle reproduces the same (mirror-reading) pattern
    batch = workloads.small_decode_batch(4, 6, 100, 0.5, N)
    ref_md = oracle_metadata(batch)
    hs = randn((len(batch.seq_lens), Hd), 8)
    kv, sh = randn((2, N, BS, H, D), 9), randn((2, 2 * N, BS, H, D), 10)
    ref = OL.opt_attention(hs, kv.clone(), sh.clone(), ref_md, *W, H, literal=True)
    layer = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W), literal=True)
    out = layer(hs.to(dev), kv.to(dev), sh.to(dev), metadata.build_from_batch(batch, dev))
    close(out, ref)


@pytest.mark.parametrize("frac", [0.0, 0.5, 1.0])
def test_prefill_layer_cache_writes_and_output(dev, frac):
    W = weights(2)
    batch = workloads.small_prefill_batch(5, 5, 90, frac, N)
    ref_md = oracle_metadata(batch)
    T = ref_md["num_prefill_tokens"]
    hs = randn((T, Hd), 11)
    kv, sh = randn((2, N, BS, H, D), 12), randn((2, 2 * N, BS, H, D), 13)
    ref_kv, ref_sh = kv.clone(), sh.clone()
    ref = OL.opt_attention(hs, ref_kv, ref_sh, ref_md, *W, H)
    layer = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W), prefill_attention=torch_prefill_attention)
    d_kv, d_sh = kv.to(dev), sh.to(dev)
    out = layer(hs.to(dev), d_kv, d_sh, metadata.build_from_batch(batch, dev))
    close(out, ref)
    close(d_kv, ref_kv)
    assert torch.equal(d_sh.cpu(), sh)        # prompts never touch the shared cache
    # the library's own prompt attention gives the same answer as the injected one
    own = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W))
    d_kv2 = kv.to(dev)
    out2 = own(hs.to(dev), d_kv2, sh.to(dev), metadata.build_from_batch(batch, dev))
    close(out2, ref)
    assert torch.equal(d_kv2, d_kv)


def _fp8_codes(x, scale):
    return torch.clamp(x.float() / scale, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8)


@pytest.mark.parametrize("frac", [0.0, 0.4, 1.0])
@pytest.mark.parametrize("absorbed", [False, True])
def test_decode_layer_with_fp8_kv_cache_matches_oracle(dev, frac, absorbed):
    """K/V cached as e4m3 codes with per-tensor scales, hidden rows in a separate 16-bit cache: written codes
    are bit-exact, the output is within tolerance of the oracle (which quantises the same way)."""
    W = weights(3)
    ks, vs = 0.02, 0.015
    batch = workloads.small_decode_batch(6, 9, 140, frac, N)
    ref_md = oracle_metadata(batch)
    hs = randn((len(batch.seq_lens), Hd), 40)
    kv8 = _fp8_codes(randn((2, N, BS, H, D), 41), 1.0 / 60)             # codes of values around +-1/60 * 448
    sh8 = _fp8_codes(randn((2, 2 * N, BS, H, D), 42), 1.0 / 60)
    hcache = randn((2, N, BS, H, D), 43)
    ref_kv, ref_sh, ref_hc = kv8.clone(), sh8.clone(), hcache.clone()
    ref = OL.opt_attention(hs, ref_kv, ref_sh, ref_md, *W, H, kv_cache_dtype="fp8", k_scale=ks, v_scale=vs,
                           hidden_cache=ref_hc)
    layer = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W), absorbed=absorbed, kv_cache_dtype="fp8",
                                       k_scale=ks, v_scale=vs)
    md = metadata.build_from_batch(batch, dev)
    d_kv, d_sh, d_hc = kv8.to(dev), sh8.to(dev), hcache.to(dev)
    out = layer(hs.to(dev), d_kv, d_sh, md, hidden_cache=d_hc)
    close(out, ref, tol=1.5e-2)
    assert torch.equal(d_hc.cpu(), ref_hc)                       # hidden rows: pure copies
    # codes written this step: the GEMM's rounding may differ by an ulp of fp16 before quantisation, which can
    # move a code by one step; everything else must be identical
    diff = (d_kv.cpu() != ref_kv)
    assert diff.float().mean().item() < 1e-3
    if absorbed:
        assert torch.equal(d_sh.cpu(), sh8)                      # nothing is re-projected
    else:
        assert (d_sh.cpu() != ref_sh).float().mean().item() < 1e-3
    if frac > 0:
        with pytest.raises(ValueError, match="hidden_cache"):
            layer(hs.to(dev), d_kv, d_sh, md)


def test_prefill_layer_with_fp8_kv_cache(dev):
    W = weights(4)
    ks, vs = 0.03, 0.02
    batch = workloads.small_prefill_batch(7, 5, 90, 0.5, N)
    ref_md = oracle_metadata(batch)
    hs = randn((ref_md["num_prefill_tokens"], Hd), 44)
    kv8 = torch.zeros(2, N, BS, H, D, dtype=torch.uint8)
    sh8 = torch.zeros(2, 2 * N, BS, H, D, dtype=torch.uint8)
    hcache = randn((2, N, BS, H, D), 45)
    ref_kv, ref_hc = kv8.clone(), hcache.clone()
    ref = OL.opt_attention(hs, ref_kv, sh8.clone(), ref_md, *W, H, kv_cache_dtype="fp8", k_scale=ks, v_scale=vs,
                           hidden_cache=ref_hc)
    layer = backend.HybridOPTAttention(Hd, H, *(w.to(dev) for w in W), kv_cache_dtype="fp8", k_scale=ks, v_scale=vs)
    d_kv, d_hc = kv8.to(dev), hcache.to(dev)
    out = layer(hs.to(dev), d_kv, sh8.to(dev), metadata.build_from_batch(batch, dev), hidden_cache=d_hc)
    close(out, ref)
    assert torch.equal(d_hc.cpu(), ref_hc)
    assert (d_kv.cpu() != ref_kv).float().mean().item() < 1e-3


def test_decode_follows_prefill_through_the_hip_path(dev):
    """Prefill L tokens then decode token L+1 == last row of a prefill of L+1 tokens, for a
    batch mixing both cache types — the whole chain on the GPU."""
    W = weights(3)
    dW = [w.to(dev) for w in W]
    rng = np.random.default_rng(7)
    lens = [9, 33, 64, 20, 47, 5]
    hid = workloads.pick_hidden(rng, len(lens), 0.5)
    full = workloads.allocate_blocks(rng, [l + 1 for l in lens], hid, N, BS, is_prompt=True)
    xs = [randn((l + 1, Hd), 30 + i) for i, l in enumerate(lens)]
    layer = backend.HybridOPTAttention(Hd, H, *dW)      # prompt and decode attention both from the library
    kv1, sh1 = backend.allocate_caches(1, N, BS, H, D, torch.float16, dev)
    md = metadata.build_metadata(True, [l + 1 for l in lens], hid, full.block_tables, full.block_tables_4_shared, BS, dev)
    out_full = layer(torch.cat(xs).to(dev), kv1[0], sh1, md)
    ends = torch.tensor(np.cumsum([l + 1 for l in lens]) - 1, device=dev)
    kv2, sh2 = backend.allocate_caches(1, N, BS, H, D, torch.float16, dev)
    md_p = metadata.build_metadata(True, lens, hid, full.block_tables, full.block_tables_4_shared, BS, dev)
    layer(torch.cat([x[:-1] for x in xs]).to(dev), kv2[0], sh2, md_p)
    md_d = metadata.build_metadata(False, [l + 1 for l in lens], hid, full.block_tables,
                                   full.block_tables_4_shared, BS, dev)
    out_dec = layer(torch.stack([x[-1] for x in xs]).to(dev), kv2[0], sh2, md_d)
    close(out_dec, out_full[ends])
    close(kv2[0], kv1[0])


def test_backend_surface(dev):
    assert backend.HybridCacheBackend.get_kv_cache_shape(10, 16, 12, 64) == (2, 10, 16, 12, 64)
    with pytest.raises(ValueError):
        backend.HybridCacheBackend.get_kv_cache_shape(10, 8, 12, 64)
    with pytest.raises(ValueError):
        backend.HybridAttentionImpl(12, 80, 0.1)
    kv, sh = backend.allocate_caches(2, 4, 16, 2, 32, torch.float16, dev)
    assert len(kv) == 2 and kv[0].shape == (2, 4, 16, 2, 32) and sh.shape == (2, 8, 16, 2, 32)
