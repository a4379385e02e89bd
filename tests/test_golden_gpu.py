"""The HIP path reproduces the committed fixtures (GPU, through the C ABI)."""
import hashlib

import numpy as np
import pytest
import torch

from aptserve_hip import metadata, ops, workloads
from golden_util import META_SCALARS, META_TENSORS, f16, load, tables_of
from util import randn, sentinel_cache

pytestmark = pytest.mark.gpu


def test_config1_mixed_write_fixture(dev):
    z = load("config1_mixed_write.npz")
    b = workloads.mixed_write_opt125m(0)
    md = metadata.build_from_batch(b, dev)
    for k in ("slot_mapping", "kv_cache_use_tot", "hidden_cache_use_input"):
        assert np.array_equal(getattr(md, k).cpu().numpy(), z[k])
    H, D, N, BS = 12, 64, 512, 16
    T = md.num_prefill_tokens
    key, value, hidden = randn((T, H, D), 0).to(dev), randn((T, H, D), 1).to(dev), randn((T, H * D), 2).to(dev)
    cache = sentinel_cache((2, N, BS, H, D)).to(dev)
    ops.hidden_to_cache(hidden, cache, md.slot_mapping, md.hidden_cache_use_input, md.hidden_cache_store_tot)
    ops.reshape_and_cache_flash(key, value, cache[0], cache[1], md.slot_mapping, "auto", token_idx=md.kv_cache_use_tot)
    assert hashlib.sha256(cache.cpu().view(torch.uint8).numpy().tobytes()).hexdigest() == str(z["cache_sha256"])


def test_metadata_fixture(dev):
    z = load("metadata_small.npz")
    for name, is_prompt in (("decode", False), ("prefill", True)):
        bt, bts = tables_of(z, name)
        md = metadata.build_metadata(is_prompt, [int(x) for x in z[f"{name}_in_seq_lens"]],
                                     [bool(x) for x in z[f"{name}_in_use_hidden"]], bt, bts, 16, dev, check_totals=True)
        for k in META_TENSORS:
            got = getattr(md, k).cpu().numpy()
            assert np.array_equal(got, z[f"{name}_{k}"]) and got.dtype == z[f"{name}_{k}"].dtype, (name, k)
        for k in META_SCALARS:
            assert getattr(md, k) == int(z[f"{name}_{k}"]), (name, k)


def test_attention_fixture(dev):
    z = load("attention_small.npz")
    q, kc, vc, wk, wv = (f16(z[k]).to(dev) for k in ("q", "kc", "vc", "wk", "wv"))
    bt, sl, ty = (torch.from_numpy(z[k]).to(dev) for k in ("bt", "sl", "types"))
    out = ops.paged_decode_attention(q, kc, vc, bt, sl, 64 ** -0.5, block_types=ty, ws_k_cache=wk, ws_v_cache=wv,
                                     max_seq_len=33)
    assert np.allclose(out.float().cpu().numpy(), z["out"], atol=4e-3, rtol=4e-3)
    k8, v8 = torch.zeros_like(kc, dtype=torch.uint8), torch.zeros_like(vc, dtype=torch.uint8)
    nblk, BS = kc.shape[:2]
    slots = torch.arange(nblk * BS, device=dev)
    ops.reshape_and_cache_flash(kc.view(nblk * BS, 2, 64), vc.view(nblk * BS, 2, 64), k8, v8, slots, "fp8", 0.05, 0.03)
    assert np.array_equal(k8.cpu().numpy(), z["k8"]) and np.array_equal(v8.cpu().numpy(), z["v8"])
    out8 = ops.paged_decode_attention(q, k8, v8, bt, sl, 64 ** -0.5, k_scale=0.05, v_scale=0.03, max_seq_len=33)
    assert np.allclose(out8.float().cpu().numpy(), z["out8"], atol=4e-3, rtol=4e-3)


def test_fp8_and_reproject_fixtures(dev):
    z = load("fp8_e4m3.npz")
    x = f16(z["x"])                       # 4001 values -> pad to a [T, 1, 8] key tensor
    pad = torch.zeros(4008, dtype=torch.float16); pad[:4001] = x
    key = pad.view(501, 1, 8).to(dev)
    for scale, name in ((1.0, "codes_scale1"), (0.37, "codes_scale_0p37")):
        kc = torch.zeros(32, 16, 1, 8, dtype=torch.uint8, device=dev); vc = torch.zeros_like(kc)
        ops.reshape_and_cache_flash(key, key, kc, vc, torch.arange(501, device=dev), "fp8", scale, scale)
        assert np.array_equal(kc.cpu().numpy().reshape(-1)[:4001], z[name])
    r = load("reproject_small.npz")
    out = ops.linear_nt(f16(r["x"]).to(dev), f16(r["w"]).to(dev), f16(r["b"]).to(dev))
    assert np.allclose(out.float().cpu().numpy(), r["out"], atol=2e-3, rtol=2e-3)
