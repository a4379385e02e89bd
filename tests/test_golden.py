"""The oracle still reproduces the committed fixtures (CPU)."""
import hashlib

import numpy as np
import torch

from aptserve_hip import workloads
from golden_util import META_SCALARS, META_TENSORS, f16, load, tables_of
from oracle import attention as OA
from oracle import cache_ops as OC
from oracle import fp8 as O8
from oracle import reproject as OR
from oracle.metadata import SeqRecord, build_metadata
from util import oracle_metadata, randn, sentinel_cache, t64


def test_config1_mixed_write_fixture():
    z = load("config1_mixed_write.npz")
    b = workloads.mixed_write_opt125m(0)
    assert list(z["seq_lens"]) == b.seq_lens and list(z["use_hidden"]) == b.use_hidden
    md = oracle_metadata(b)
    for k in ("slot_mapping", "kv_cache_use_tot", "hidden_cache_use_input"):
        assert np.array_equal(md[k], z[k])
    H, D, N, BS = 12, 64, 512, 16
    T = md["num_prefill_tokens"]
    key, value, hidden = randn((T, H, D), 0), randn((T, H, D), 1), randn((T, H * D), 2)
    cache = sentinel_cache((2, N, BS, H, D))
    sm, kv_use = t64(md["slot_mapping"]), t64(md["kv_cache_use_tot"])
    OC.hidden_to_cache(hidden, cache, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    OC.reshape_and_cache_flash(key[kv_use], value[kv_use], cache[0], cache[1], sm[kv_use], "auto")
    assert hashlib.sha256(cache.view(torch.uint8).numpy().tobytes()).hexdigest() == str(z["cache_sha256"])
    assert np.array_equal(cache.view(-1, H * D)[t64(z["sample_rows"])].view(torch.int16).numpy(), z["sample_values"])


def test_metadata_fixture():
    z = load("metadata_small.npz")
    for name, is_prompt in (("decode", False), ("prefill", True)):
        bt, bts = tables_of(z, name)
        lens, hid = z[f"{name}_in_seq_lens"], z[f"{name}_in_use_hidden"]
        recs = [SeqRecord(is_prompt, bool(h), int(l), 0 if is_prompt else int(l) - 1, t, s)
                for l, h, t, s in zip(lens, hid, bt, bts)]
        md = build_metadata(recs, 16)
        for k in META_TENSORS:
            assert np.array_equal(md[k], z[f"{name}_{k}"]) and md[k].dtype == z[f"{name}_{k}"].dtype, (name, k)
        for k in META_SCALARS:
            assert md[k] == int(z[f"{name}_{k}"]), (name, k)


def test_attention_fixture():
    z = load("attention_small.npz")
    q, kc, vc, wk, wv = (f16(z[k]) for k in ("q", "kc", "vc", "wk", "wv"))
    out = OA.paged_decode_attention(q, kc, vc, torch.from_numpy(z["bt"]), torch.from_numpy(z["sl"]), 64 ** -0.5,
                                    block_types=torch.from_numpy(z["types"]), ws_k_cache=wk, ws_v_cache=wv)
    assert np.allclose(out.numpy(), z["out"], rtol=1e-6, atol=1e-7)
    assert np.array_equal(O8.quantize_e4m3(kc, 0.05).numpy(), z["k8"])
    out8 = OA.paged_decode_attention(q, torch.from_numpy(z["k8"]), torch.from_numpy(z["v8"]), torch.from_numpy(z["bt"]),
                                     torch.from_numpy(z["sl"]), 64 ** -0.5, k_scale=0.05, v_scale=0.03)
    assert np.allclose(out8.numpy(), z["out8"], rtol=1e-6, atol=1e-7)


def test_fp8_and_reproject_fixtures():
    z = load("fp8_e4m3.npz")
    assert np.array_equal(np.nan_to_num(O8.decode_table(), nan=-1), np.nan_to_num(z["table"], nan=-1))
    x = f16(z["x"])
    assert np.array_equal(O8.quantize_e4m3(x, 1.0).numpy(), z["codes_scale1"])
    assert np.array_equal(O8.quantize_e4m3(x, 0.37).numpy(), z["codes_scale_0p37"])
    r = load("reproject_small.npz")
    out = OR._linear_fp32(f16(r["x"]), f16(r["w"]), f16(r["b"]))
    assert np.allclose(out.numpy(), r["out"], rtol=1e-6, atol=1e-6)
