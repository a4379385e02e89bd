"""The decode attention of a mixed batch as one call: a paged decode attention that is planned as a job and
launched later, by itself or inside the attention on the hidden rows.  The bar is equality bit for bit with the
two direct calls (paged_decode_attention, absorbed_hidden_attention), which have oracle tests of their own: the
job runs the same kernels on the same arguments, whichever launch carries its workgroups."""
import ctypes

import numpy as np
import pytest
import torch

from aptserve_hip import metadata, ops, workloads
from util import randn

pytestmark = pytest.mark.gpu
BS = 16


def _batch(dev, H, D, batch, frac, max_len, N, dtype, seed):
    Hd = H * D
    b = workloads.small_decode_batch(seed, batch, max_len, frac, N, BS)
    md = metadata.build_from_batch(b, dev)
    cache = randn((2, N, BS, H, D), seed + 1).to(dtype).to(dev)
    w = [(randn((Hd, Hd), seed + 2 + i) / np.sqrt(Hd)).to(dtype).to(dev) for i in range(2)]
    b_v = (randn((Hd,), seed + 4) * 0.1).to(dtype).to(dev)
    q = randn((len(b.seq_lens), Hd), seed + 5, dtype).to(dev)
    return b, md, cache, w, b_v, q


def _paged(q, cache, md, H, D, out, **kw):
    return ops.paged_decode_attention(q.view(-1, H, D), cache[0], cache[1], md.private_block_tables, md.kv_seq_lens,
                                      D ** -0.5, max_seq_len=md.max_kv_seq_len or None, out=out.view(-1, H, D), **kw)


def _hidden(q, cache, md, w, b_v, D, out, **kw):
    return ops.absorbed_hidden_attention(q, cache, md.hidden_slots, md.hidden_seq_start, md.hidden_cache_use_input,
                                         md.max_hidden_seq_len, w[0], w[1], b_v, D ** -0.5, out, **kw)


# small batches at head size 128 take the combined launch, the others launch the job first
@pytest.mark.parametrize("H,D,batch,frac,max_len,dtype", [
    (40, 128, 5, 0.5, 400, torch.float16), (40, 128, 5, 0.5, 400, torch.bfloat16),
    (40, 128, 8, 0.3, 120, torch.float16),      # more K/V-cached sequences than hidden-cached ones
    (8, 128, 3, 0.4, 1000, torch.float16),      # partitions of 128 tokens, eight wavefronts busy
    (12, 64, 6, 0.5, 200, torch.float16),       # head size 64: the job is launched by itself
    (40, 128, 60, 0.5, 300, torch.float16),     # a batch too large for the chunked sum
])
def test_one_call_for_both_kinds_of_sequence_equals_the_two_calls(dev, H, D, batch, frac, max_len, dtype):
    for seed in (0, 1):
        b, md, cache, w, b_v, q = _batch(dev, H, D, batch, frac, max_len, 512, dtype, 10 * seed)
        n_h = md.num_hidden_cache_tokens
        assert 0 < n_h < len(b.seq_lens)
        want = torch.full_like(q, 7.0)
        _paged(q, cache, md, H, D, want)
        _hidden(q, cache, md, w, b_v, D, want)
        got = torch.full_like(q, 7.0)
        job = _paged(q, cache, md, H, D, got, as_job=True)
        torch.cuda.synchronize()
        assert (got == 7).all()                      # planning launches nothing
        _hidden(q, cache, md, w, b_v, D, got, kv_job=job)
        assert torch.equal(got, want) and not (got == 7).all(dim=1).any()
        # the same job again, by itself
        alone = torch.full_like(q, 7.0)
        job2 = _paged(q, cache, md, H, D, alone, as_job=True)
        job2.launch()
        kv_rows = torch.tensor([i for i, h in enumerate(b.use_hidden) if not h], device=dev)
        assert torch.equal(alone[kv_rows], want[kv_rows])
        hid_rows = torch.tensor([i for i, h in enumerate(b.use_hidden) if h], device=dev)
        assert (alone[hid_rows] == 0).all()          # length 0 in kv_seq_lens: zeros, as in the direct call


@pytest.mark.parametrize("H,D,batch,frac,max_len,dtype", [
    (40, 128, 5, 0.5, 400, torch.float16),      # stores beside the absorbed queries, attention in the chunk launch
    (40, 128, 7, 0.6, 150, torch.bfloat16),
    (12, 64, 6, 0.5, 200, torch.float16),       # stores ride, the attention job is launched behind them
    (4, 256, 4, 0.5, 100, torch.float16),       # wide heads: both jobs by themselves, stores first
    (40, 128, 60, 0.5, 300, torch.float16),     # a large batch: stores ride, nothing else does
])
def test_step_stores_and_both_attentions_as_one_call_equal_the_three_calls(dev, H, D, batch, frac, max_len, dtype):
    """The newest K/V rows and hidden rows of the step are written by the same call that then reads them: the
    caches and the attention output must equal those of store, paged attention and hidden-row attention called one
    after the other."""
    b, md, cache, w, b_v, q = _batch(dev, H, D, batch, frac, max_len, 512, dtype, 21)
    B, Hd = len(b.seq_lens), H * D
    hs, k, v = (randn((B, Hd), 30 + i, dtype).to(dev) for i in range(3))

    def stores(c, **kw):
        return ops.decode_step_cache_ops(None, hs, c, None, md.slot_mapping, md.hidden_cache_use_input,
                                         md.hidden_cache_store_tot, k, v, md.kv_cache_use_input, md.new_token_slot, **kw)

    cache_a, want = cache.clone(), torch.full_like(q, 7.0)
    stores(cache_a)
    _paged(q, cache_a, md, H, D, want)
    _hidden(q, cache_a, md, w, b_v, D, want)
    assert not torch.equal(cache_a, cache)
    cache_b, got = cache.clone(), torch.full_like(q, 7.0)
    store_job = stores(cache_b, as_job=True)
    kv_job = _paged(q, cache_b, md, H, D, got, as_job=True)
    torch.cuda.synchronize()
    assert torch.equal(cache_b, cache) and (got == 7).all()      # planning launches nothing
    _hidden(q, cache_b, md, w, b_v, D, got, kv_job=kv_job, store_job=store_job)
    assert torch.equal(cache_b, cache_a) and torch.equal(got, want)
    # the store job by itself
    cache_c = cache.clone()
    stores(cache_c, as_job=True).launch()
    assert torch.equal(cache_c, cache_a)


def test_job_of_split_sequences_and_of_an_fp8_cache_equals_the_direct_call(dev):
    """Long sequences (partial results in a workspace, the second launch that merges them) and fp8 codes."""
    H, D, N = 8, 128, 1024
    rng = np.random.default_rng(5)
    lens = [3000, 17, 1500, 4096]
    b = workloads.allocate_blocks(rng, lens, [False] * len(lens), N, BS, is_prompt=False)
    md = metadata.build_from_batch(b, dev)
    q = randn((len(lens), H, D), 1).to(dev)
    for fp8 in (False, True):
        cache = randn((2, N, BS, H, D), 2)
        cache = (cache * 0.5).to(torch.float8_e4m3fn).view(torch.uint8).to(dev) if fp8 else cache.to(dev)
        kw = dict(k_scale=0.5, v_scale=2.0) if fp8 else {}
        want = ops.paged_decode_attention(q, cache[0], cache[1], md.private_block_tables, md.kv_seq_lens, D ** -0.5,
                                          max_seq_len=max(lens), partition_size=256, **kw)
        got = torch.full_like(q, 7.0)
        job = ops.paged_decode_attention(q, cache[0], cache[1], md.private_block_tables, md.kv_seq_lens, D ** -0.5,
                                         max_seq_len=max(lens), partition_size=256, out=got, as_job=True, **kw)
        for _ in range(2):               # a job may be launched more than once
            got.fill_(7.0)
            job.launch()
            assert torch.equal(got, want)


def test_only_one_kind_of_sequence_and_bad_jobs(dev):
    H, D = 40, 128
    lib = ops._lib.load()
    # every sequence K/V-cached: the hybrid call only launches the job
    b, md, cache, w, b_v, q = _batch(dev, H, D, 4, 0.0, 100, 256, torch.float16, 3)
    assert md.num_hidden_cache_tokens == 0
    want = torch.full_like(q, 7.0)
    _paged(q, cache, md, H, D, want)
    got = torch.full_like(q, 7.0)
    job = _paged(q, cache, md, H, D, got, as_job=True)
    empty = torch.zeros(0, dtype=torch.int64, device=dev)
    ops.absorbed_hidden_attention(q, cache, empty, torch.zeros(1, dtype=torch.int64, device=dev), empty, 0, w[0], w[1],
                                  b_v, D ** -0.5, got, kv_job=job)
    assert torch.equal(got, want)
    # every sequence hidden-cached: a job over an empty batch rides along and does nothing
    b, md, cache, w, b_v, q = _batch(dev, H, D, 3, 1.0, 100, 256, torch.float16, 4)
    want = torch.full_like(q, 7.0)
    _hidden(q, cache, md, w, b_v, D, want)
    got = torch.full_like(q, 7.0)
    job = ops.paged_decode_attention(q[:0].view(-1, H, D), cache[0], cache[1], md.private_block_tables[:0],
                                     md.kv_seq_lens[:0], D ** -0.5, out=got[:0].view(-1, H, D), as_job=True)
    _hidden(q, cache, md, w, b_v, D, got, kv_job=job)
    assert torch.equal(got, want)
    # ... and its stores are the hidden rows alone (no key, no value)
    hs = randn((3, H * D), 9).to(dev)
    cache_a, cache_b = cache.clone(), cache.clone()
    ops.hidden_to_cache(hs, cache_a, md.slot_mapping, md.hidden_cache_use_input, md.hidden_cache_store_tot)
    _hidden(q, cache_a, md, w, b_v, D, want)
    sj = ops.decode_step_cache_ops(None, hs, cache_b, None, md.slot_mapping, md.hidden_cache_use_input,
                                   md.hidden_cache_store_tot, None, None, None, None, as_job=True)
    _hidden(q, cache_b, md, w, b_v, D, got, store_job=sj)
    assert torch.equal(cache_a, cache_b) and not torch.equal(cache_a, cache) and torch.equal(got, want)
    # bytes that no planning call wrote are refused, and so is a buffer that is too small
    junk = (ctypes.c_uint64 * 40)()
    assert lib.aps_attention_job_launch(ctypes.addressof(junk), None) == -1
    ws = torch.empty(lib.aps_absorbed_attention_workspace_bytes(3, 100, H, D), dtype=torch.uint8, device=dev)
    st = lib.aps_hybrid_decode_attention(
        None, ctypes.addressof(junk), q.data_ptr(), q.stride(0), md.hidden_cache_use_input.data_ptr(), q.size(0),
        cache.data_ptr(), cache.stride(2), cache.numel() // cache.stride(2), md.hidden_slots.data_ptr(),
        md.hidden_seq_start.data_ptr(), 3, int(md.max_hidden_seq_len), w[0].data_ptr(), w[1].data_ptr(),
        b_v.data_ptr(), w[0].stride(0), H, D, D ** -0.5, got.data_ptr(), got.stride(0), got.size(0), 0, ws.data_ptr(),
        ws.numel(), None)
    assert st == -1
    assert lib.aps_cache_job_launch(ctypes.addressof(junk), None) == -1
    out = torch.empty(2, H, D, dtype=torch.float16, device=dev)
    st = lib.aps_paged_decode_attention_job(
        ctypes.addressof(junk), 64, out.data_ptr(), out.data_ptr(), cache[0].data_ptr(), cache[1].data_ptr(), None,
        None, md.private_block_tables.data_ptr(), None, md.seq_lens_tensor.data_ptr(), 2, H, D, BS,
        md.private_block_tables.size(1), md.private_block_tables.stride(0), 0, H * D, H * D, cache.stride(1),
        cache.size(1), 0, 0, 100, 0, D ** -0.5, 0, 0, 1.0, 1.0, None, 0)
    torch.cuda.synchronize()
    assert st == -1
