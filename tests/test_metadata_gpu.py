"""GPU metadata builder against the list-based oracle — integer, bit-exact."""
import numpy as np
import pytest
import torch

from aptserve_hip import metadata, workloads
from util import oracle_metadata

pytestmark = pytest.mark.gpu

TENSOR_FIELDS = ["slot_mapping", "slot_mapping_shared", "hidden_cache_use_tot", "kv_cache_use_tot",
                 "hidden_cache_use_input", "hidden_cache_store_tot", "hidden_holder_upd", "hidden_holder_pull",
                 "seq_lens_tensor", "context_lens_tensor", "query_start_loc", "seq_start_loc", "block_tables",
                 "input_positions"]
SCALAR_FIELDS = ["num_prefills", "num_prefill_tokens", "num_decode_tokens", "num_tot_tokens",
                 "num_hidden_cache_tokens", "max_query_len", "max_prefill_seq_len", "max_decode_seq_len", "seq_lens"]


def assert_same(md, ref):
    for f in SCALAR_FIELDS:
        assert getattr(md, f) == ref[f], f
    for f in TENSOR_FIELDS:
        got = getattr(md, f).cpu().numpy()
        assert got.dtype == ref[f].dtype, (f, got.dtype, ref[f].dtype)
        assert got.shape == ref[f].shape, (f, got.shape, ref[f].shape)
        assert np.array_equal(got, ref[f]), f
    if md.num_decode_tokens:
        # the two resolved per-row vectors this implementation adds, restated from the reference's fields
        src = ref["slot_mapping"].copy()
        src[src < 0] = np.iinfo(np.int64).min
        src[ref["hidden_holder_upd"]] = -(np.arange(len(ref["hidden_holder_upd"])) + 1)
        assert np.array_equal(md.holder_src.cpu().numpy(), src)
        dest = np.full(ref["num_tot_tokens"], -1, dtype=np.int64)
        dest[ref["hidden_cache_use_tot"]] = ref["slot_mapping_shared"]
        private = ref["slot_mapping"][ref["kv_cache_use_tot"]]
        dest[ref["kv_cache_use_tot"]] = np.where(private >= 0, -(private + 2), -1)
        assert np.array_equal(md.kv_dest.cpu().numpy(), dest)
        hid = np.zeros(md.num_decode_tokens, dtype=bool)
        hid[ref["hidden_cache_use_input"]] = True
        assert np.array_equal(md.kv_cache_use_input.cpu().numpy(), np.nonzero(~hid)[0])
        assert np.array_equal(md.new_token_slot.cpu().numpy(), ref["slot_mapping"][ref["hidden_holder_upd"]])
        assert np.array_equal(md.kv_seq_lens.cpu().numpy(), np.where(hid, 0, ref["seq_lens_tensor"]).astype(np.int32))
        assert np.array_equal(md.hidden_slots.cpu().numpy(), ref["slot_mapping"][ref["hidden_cache_use_tot"]])
        starts = np.concatenate([[0], np.cumsum(ref["seq_lens_tensor"][hid])])
        if hid.any():
            assert np.array_equal(md.hidden_seq_start.cpu().numpy(), starts)


@pytest.mark.parametrize("seed", range(5))
@pytest.mark.parametrize("frac", [0.0, 0.3, 0.5, 1.0])
@pytest.mark.parametrize("bs", [16, 32])
def test_decode_metadata_small(dev, seed, frac, bs):
    batch = workloads.small_decode_batch(seed, 11, 300, frac, 400, bs)
    md = metadata.build_from_batch(batch, dev, check_totals=True)
    assert_same(md, oracle_metadata(batch))


@pytest.mark.parametrize("frac", [0.0, 0.5, 1.0])
@pytest.mark.parametrize("prompt", [False, True])
def test_packed_tables_give_the_same_metadata_as_lists(dev, frac, prompt):
    """Block tables handed over as 0-padded int32 arrays: every field equals the oracle's, as with lists."""
    batch = (workloads.small_prefill_batch(3, 9, 200, frac, 300) if prompt
             else workloads.small_decode_batch(3, 11, 300, frac, 400))
    md = metadata.build_from_batch(batch, dev, packed=True, check_totals=True)
    assert_same(md, oracle_metadata(batch))


def test_packed_tables_wider_than_needed_and_too_narrow(dev):
    """Packed tables may be wider than the longest sequence needs (a runner keeps them at a fixed width): the
    extra columns are ignored.  Tables narrower than ceil(seq_len / block_size) are refused, the private one
    and the shared one alike; mixing a packed private table with ragged shared lists works."""
    batch = workloads.small_decode_batch(5, 11, 300, 0.5, 400)
    ref = oracle_metadata(batch)
    bt, bts = batch.packed_tables()
    lens, hid = np.asarray(batch.seq_lens), np.asarray(batch.use_hidden, dtype=bool)
    pad = lambda a: np.concatenate([a, np.full((a.shape[0], 7), 12345, dtype=a.dtype)], axis=1)
    md = metadata.build_metadata(False, lens, hid, pad(bt), pad(bts), batch.block_size, dev, check_totals=True)
    assert_same(md, ref)
    md = metadata.build_metadata(False, lens, hid, bt, batch.block_tables_4_shared, batch.block_size, dev,
                                 check_totals=True)
    assert_same(md, ref)
    need = int(-(-lens.max() // batch.block_size))
    with pytest.raises(ValueError):
        metadata.build_metadata(False, lens, hid, bt[:, :need - 1], bts, batch.block_size, dev)
    need_h = int(-(-lens[hid].max() // batch.block_size))
    with pytest.raises(ValueError):
        metadata.build_metadata(False, lens, hid, bt, bts[:, :need_h - 1], batch.block_size, dev)


@pytest.mark.parametrize("seed", range(4))
@pytest.mark.parametrize("frac", [0.0, 0.4, 1.0])
def test_prefill_metadata_small(dev, seed, frac):
    batch = workloads.small_prefill_batch(seed, 9, 500, frac, 600)
    md = metadata.build_from_batch(batch, dev, check_totals=True)
    assert_same(md, oracle_metadata(batch))
    # the three aliases of the prompt path (aptserve_model_runner.py:658-662)
    assert md.hidden_cache_use_tot.data_ptr() == md.hidden_cache_use_input.data_ptr() == md.hidden_cache_store_tot.data_ptr()


def test_config1_and_config2_batches(dev):
    b1 = workloads.mixed_write_opt125m(0)
    assert_same(metadata.build_from_batch(b1, dev, check_totals=True), oracle_metadata(b1))
    b2 = workloads.decode_batch_opt13b(0)
    md = metadata.build_from_batch(b2, dev, check_totals=True)
    assert_same(md, oracle_metadata(b2))
    assert md.num_tot_tokens == 87719 and len(md.hidden_cache_use_tot) == 87591


def test_large_batch_many_workgroups(dev):
    """More sequences than threads in a workgroup: the prefix loop takes several strides."""
    rng = np.random.default_rng(0)
    B = 1500
    batch = workloads.allocate_blocks(rng, rng.integers(1, 60, B), rng.random(B) < 0.5, 8000, 16, is_prompt=False)
    assert_same(metadata.build_from_batch(batch, dev, check_totals=True), oracle_metadata(batch))
    batch = workloads.allocate_blocks(rng, rng.integers(1, 60, B), rng.random(B) < 0.5, 8000, 16, is_prompt=True)
    assert_same(metadata.build_from_batch(batch, dev, check_totals=True), oracle_metadata(batch))


def test_views_slice_like_the_reference(dev):
    batch = workloads.small_decode_batch(1, 6, 80, 0.5, 100)
    md = metadata.build_from_batch(batch, dev)
    assert md.prefill_metadata is None
    d = md.decode_metadata
    assert d is md.decode_metadata                      # cached
    assert d.num_prefills == 0 and d.num_decode_tokens == 6 and d.seq_lens is None and d.max_query_len is None
    assert d.slot_mapping.data_ptr() == md.slot_mapping.data_ptr()
    assert torch.equal(d.block_tables, md.block_tables) and torch.equal(d.seq_lens_tensor, md.seq_lens_tensor)
    pb = workloads.small_prefill_batch(1, 4, 30, 0.5, 100)
    pm = metadata.build_from_batch(pb, dev)
    assert pm.decode_metadata is None
    p = pm.prefill_metadata
    assert p.num_decode_tokens == 0 and p.max_decode_seq_len == 0 and p.seq_lens == pb.seq_lens
    assert p.slot_mapping.numel() == pm.num_prefill_tokens


def test_memory_profiling_run_and_bad_arguments(dev):
    md = metadata.build_metadata(True, [7, 3], [False, False], [[], []], [[], []], 16, dev)
    assert md.slot_mapping.tolist() == [-1] * 10
    with pytest.raises(ValueError):
        metadata.build_metadata(False, [40], [True], [[1, 2, 3]], [[5]], 16, dev)     # shared table too short
    with pytest.raises(ValueError):
        metadata.build_metadata(False, [40], [False], [[1]], [[]], 16, dev)           # private table too short
    with pytest.raises(ValueError):
        metadata.build_metadata(False, [], [], [], [], 16, dev)


def test_back_to_back_builds_do_not_race_on_the_staging_buffers(dev):
    batches = [workloads.small_decode_batch(s, 20, 200, 0.5, 600) for s in range(12)]
    mds = [metadata.build_from_batch(b, dev) for b in batches]     # no synchronisation in between
    for b, md in zip(batches, mds):
        assert_same(md, oracle_metadata(b))
