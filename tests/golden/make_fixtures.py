"""Writes the small golden fixtures under tests/golden/ from the CPU oracle.

    python tests/golden/make_fixtures.py

The reference ships no tests and no golden vectors, and its Python cannot be
imported here (it needs vllm, vllm_flash_attn and its own CUDA extension), so
these vectors come from the oracle after it has been pinned by the independent
witnesses in tests/test_oracle_*.py.  They freeze the oracle's answers: a later
edit of the oracle or of a kernel that changes any of them fails
tests/test_golden.py on the CPU and tests/test_golden_gpu.py on the GPU.
"""
import hashlib
import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
for p in (ROOT, ROOT / "apt-serve_amd", ROOT / "tests"):
    sys.path.insert(0, str(p))

from aptserve_hip import workloads  # noqa: E402
from oracle import attention as OA  # noqa: E402
from oracle import cache_ops as OC  # noqa: E402
from oracle import fp8 as O8  # noqa: E402
from oracle import reproject as OR  # noqa: E402
from util import oracle_metadata, randn, sentinel_cache, t64  # noqa: E402


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def config1():
    b = workloads.mixed_write_opt125m(0)
    md = oracle_metadata(b)
    H, D, N, BS = 12, 64, 512, 16
    T = md["num_prefill_tokens"]
    key, value, hidden = randn((T, H, D), 0), randn((T, H, D), 1), randn((T, H * D), 2)
    cache = sentinel_cache((2, N, BS, H, D))
    sm, kv_use = t64(md["slot_mapping"]), t64(md["kv_cache_use_tot"])
    OC.hidden_to_cache(hidden, cache, sm, t64(md["hidden_cache_use_input"]), t64(md["hidden_cache_store_tot"]))
    OC.reshape_and_cache_flash(key[kv_use], value[kv_use], cache[0], cache[1], sm[kv_use], "auto")
    rows = np.concatenate([md["slot_mapping"][:3], md["slot_mapping"][-3:]])
    np.savez(HERE / "config1_mixed_write.npz", seq_lens=np.array(b.seq_lens), use_hidden=np.array(b.use_hidden),
             slot_mapping=md["slot_mapping"], kv_cache_use_tot=md["kv_cache_use_tot"],
             hidden_cache_use_input=md["hidden_cache_use_input"], cache_sha256=np.array(sha(cache)),
             sample_rows=rows, sample_values=cache.view(-1, H * D)[t64(rows)].view(torch.int16).numpy())


def metadata_small():
    out = {}
    for name, batch in (("decode", workloads.small_decode_batch(11, 6, 70, 0.5, 64)),
                        ("prefill", workloads.small_prefill_batch(12, 5, 60, 0.4, 64))):
        md = oracle_metadata(batch)
        W = max(len(t) for t in batch.block_tables)
        bt = np.zeros((len(batch.seq_lens), W), dtype=np.int32); bts = np.zeros_like(bt)
        nb = np.zeros(len(batch.seq_lens), dtype=np.int32); nbs = np.zeros_like(nb)
        for i, (t, s) in enumerate(zip(batch.block_tables, batch.block_tables_4_shared)):
            bt[i, :len(t)] = t; nb[i] = len(t); bts[i, :len(s)] = s; nbs[i] = len(s)
        out.update({f"{name}_in_seq_lens": np.array(batch.seq_lens), f"{name}_in_use_hidden": np.array(batch.use_hidden),
                    f"{name}_in_tables": bt, f"{name}_in_table_lens": nb, f"{name}_in_shared": bts,
                    f"{name}_in_shared_lens": nbs})
        for k, v in md.items():
            out[f"{name}_{k}"] = np.asarray(v)
    np.savez(HERE / "metadata_small.npz", **out)


def attention_small():
    B, H, D, BS, nblk = 3, 2, 64, 16, 12
    lens = [5, 33, 17]
    rng = np.random.default_rng(3)
    bt = np.zeros((B, 3), dtype=np.int32)
    perm = rng.permutation(nblk); p = 0
    for b, l in enumerate(lens):
        n = -(-l // BS); bt[b, :n] = perm[p:p + n]; p += n
    types = rng.integers(0, 2, bt.shape).astype(np.uint8)
    q, kc, vc = randn((B, H, D), 0), randn((nblk, BS, H, D), 1), randn((nblk, BS, H, D), 2)
    wk, wv = randn((nblk, BS, H, D), 3), randn((nblk, BS, H, D), 4)
    sl = torch.tensor(lens, dtype=torch.int32)
    out = OA.paged_decode_attention(q, kc, vc, torch.from_numpy(bt), sl, D ** -0.5, block_types=torch.from_numpy(types),
                                    ws_k_cache=wk, ws_v_cache=wv)
    k8, v8 = O8.quantize_e4m3(kc, 0.05), O8.quantize_e4m3(vc, 0.03)
    out8 = OA.paged_decode_attention(q, k8, v8, torch.from_numpy(bt), sl, D ** -0.5, k_scale=0.05, v_scale=0.03)
    np.savez(HERE / "attention_small.npz", q=q.view(torch.int16).numpy(), kc=kc.view(torch.int16).numpy(),
             vc=vc.view(torch.int16).numpy(), wk=wk.view(torch.int16).numpy(), wv=wv.view(torch.int16).numpy(),
             bt=bt, types=types, sl=np.array(lens, dtype=np.int32), out=out.numpy(), k8=k8.numpy(), v8=v8.numpy(),
             out8=out8.numpy())


def fp8_and_reproject():
    x = torch.linspace(-500, 500, 4001, dtype=torch.float32).half()
    np.savez(HERE / "fp8_e4m3.npz", table=O8.decode_table(), x=x.view(torch.int16).numpy(),
             codes_scale1=O8.quantize_e4m3(x, 1.0).numpy(), codes_scale_0p37=O8.quantize_e4m3(x, 0.37).numpy())
    a, w, b = randn((5, 64), 0), (randn((256, 64), 1) * 0.1).half(), randn((256,), 2)
    np.savez(HERE / "reproject_small.npz", x=a.view(torch.int16).numpy(), w=w.view(torch.int16).numpy(),
             b=b.view(torch.int16).numpy(), out=OR._linear_fp32(a, w, b).numpy())


if __name__ == "__main__":
    config1(); metadata_small(); attention_small(); fp8_and_reproject()
    for f in sorted(HERE.glob("*.np*")):
        print(f.name, f.stat().st_size)
