"""HIP paged decode attention against the fp32-softmax oracle.

Tolerance stated by the task for an fp16 result: 2e-2 absolute.  The kernel
accumulates in fp32 like the oracle, so the tests hold it to a tighter bound
(the fp16 rounding of the result plus summation-order noise) and check the
2e-2 figure as well.
"""
import numpy as np
import pytest
import torch

from aptserve_hip import ops, workloads
from oracle import attention as OA
from oracle import fp8 as O8
from util import randn

pytestmark = pytest.mark.gpu

SPEC_ATOL = 2e-2


def make_case(B, H, D, BS, lens, seed, dtype=torch.float16, extra_blocks=5, hybrid=False):
    rng = np.random.default_rng(seed)
    need = sum(-(-max(l, 0) // BS) for l in lens)
    nblk = need + extra_blocks
    W = max(1, max(-(-max(l, 0) // BS) for l in lens))
    bt = np.zeros((B, W), dtype=np.int32)
    perm = rng.permutation(nblk)
    p = 0
    for b, l in enumerate(lens):
        n = -(-max(l, 0) // BS)
        bt[b, :n] = perm[p:p + n]; p += n
    case = dict(
        q=randn((B, H, D), seed, dtype), kc=randn((nblk, BS, H, D), seed + 1, dtype),
        vc=randn((nblk, BS, H, D), seed + 2, dtype), bt=torch.from_numpy(bt),
        sl=torch.tensor(lens, dtype=torch.int32), scale=D ** -0.5)
    if hybrid:
        case["types"] = torch.from_numpy(rng.integers(0, 2, bt.shape).astype(np.uint8))
        case["wk"] = randn((nblk, BS, H, D), seed + 3, dtype)
        case["wv"] = randn((nblk, BS, H, D), seed + 4, dtype)
    return case


def run_both(c, dev, partition_size=0, **kw):
    hyb = "types" in c
    ref = OA.paged_decode_attention(
        c["q"], c["kc"], c["vc"], c["bt"], c["sl"], c["scale"],
        block_types=c.get("types"), ws_k_cache=c.get("wk"), ws_v_cache=c.get("wv"), **kw)
    g = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = ops.paged_decode_attention(
        g["q"], g["kc"], g["vc"], g["bt"], g["sl"], g["scale"], block_types=g.get("types"),
        ws_k_cache=g.get("wk"), ws_v_cache=g.get("wv"), partition_size=partition_size,
        max_seq_len=int(max(1, c["sl"].max())), **kw)
    return out.float().cpu(), ref


def check(out, ref, dtype=torch.float16):
    err = (out - ref).abs().max().item()
    assert err <= SPEC_ATOL, f"max abs error {err} above the stated tolerance"
    tight = 4e-3 if dtype == torch.float16 else 1e-2   # bf16 keeps 8 mantissa bits
    assert torch.allclose(out, ref, atol=tight, rtol=tight), f"max abs error {err}"


@pytest.mark.parametrize("D", [32, 64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("partition_size", [0, 32])
def test_decode_attention_small(dev, D, dtype, partition_size):
    lens = [1, 15, 16, 17, 33, 64, 100, 3]
    c = make_case(len(lens), 3, D, 16, lens, D, dtype)
    out, ref = run_both(c, dev, partition_size)
    check(out, ref, dtype)


@pytest.mark.parametrize("BS", [16, 32])
def test_decode_attention_block_sizes_and_many_partitions(dev, BS):
    lens = [700, 1, 257, 512, 31]
    c = make_case(len(lens), 4, 128, BS, lens, 11)
    for ps in (0, 64, 256, 1024):
        out, ref = run_both(c, dev, ps)
        check(out, ref)


def test_zero_length_sequences_give_zero_rows(dev):
    lens = [0, 5, 0, 40]
    c = make_case(4, 2, 64, 16, lens, 5)
    for ps in (0, 16):
        out, ref = run_both(c, dev, ps)
        check(out, ref)
        assert out[0].abs().sum() == 0 and out[2].abs().sum() == 0


def test_garbage_past_the_end_of_a_block_is_ignored(dev):
    """Slots beyond seq_len hold NaN/inf: they must not leak into the result."""
    lens = [5, 18, 33]
    c = make_case(3, 2, 128, 16, lens, 6)
    for b, l in enumerate(lens):
        last = c["bt"][b, (l - 1) // 16]
        c["kc"][last, l % 16:] = float("nan")
        c["vc"][last, l % 16:] = float("inf")
    clean = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out, _ = run_both(c, dev)
    clean["kc"] = torch.nan_to_num(clean["kc"], nan=0.0)
    clean["vc"] = torch.nan_to_num(clean["vc"], posinf=0.0)
    ref = OA.paged_decode_attention(clean["q"], clean["kc"], clean["vc"], clean["bt"], clean["sl"], clean["scale"])
    assert torch.isfinite(out).all()
    check(out, ref)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("partition_size", [0, 48])
def test_hybrid_block_source_select(dev, D, partition_size):
    lens = [20, 33, 64, 200, 7]
    c = make_case(len(lens), 3, D, 16, lens, 21, hybrid=True)
    out, ref = run_both(c, dev, partition_size)
    check(out, ref)
    # all-cache and all-workspace must also agree with the plain call on the respective pool
    c2 = dict(c); c2["types"] = torch.ones_like(c["types"])
    out2, _ = run_both(c2, dev, partition_size)
    plain = OA.paged_decode_attention(c["q"], c["wk"], c["wv"], c["bt"], c["sl"], c["scale"])
    check(out2, plain)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("qdtype", [torch.float16, torch.bfloat16])
def test_fp8_cache(dev, D, qdtype):
    lens = [1, 16, 45, 130, 300]
    c = make_case(len(lens), 2, D, 16, lens, 31, qdtype, hybrid=True)
    ks, vs = 0.05, 0.02
    for k in ("kc", "vc", "wk", "wv"):
        c[k] = O8.quantize_e4m3(c[k], ks if k in ("kc", "wk") else vs)
    for ps in (0, 64):
        out, ref = run_both(c, dev, ps, k_scale=ks, v_scale=vs)
        check(out, ref, qdtype)


def test_flash_attn_with_kvcache_keywords(dev):
    lens = [9, 77]
    c = make_case(2, 12, 64, 16, lens, 41)
    g = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    o = ops.flash_attn_with_kvcache(g["q"].unsqueeze(1), g["kc"], g["vc"], block_table=g["bt"],
                                    cache_seqlens=g["sl"], softmax_scale=c["scale"], causal=True, alibi_slopes=None)
    ref = OA.flash_attn_with_kvcache(c["q"].unsqueeze(1), c["kc"], c["vc"], block_table=c["bt"],
                                     cache_seqlens=c["sl"], softmax_scale=c["scale"])
    assert o.shape == (2, 1, 12, 64)
    check(o.float().cpu(), ref.float())


def test_strided_query_and_preallocated_output(dev):
    """q is a chunk view of the fused qkv activations (row stride 3*Hd)."""
    lens = [30, 5, 64]
    H, D = 4, 64
    c = make_case(3, H, D, 16, lens, 51)
    qkv = randn((3, 3 * H * D), 7)
    c["q"] = qkv[:, :H * D].view(3, H, D)
    ref = OA.paged_decode_attention(c["q"], c["kc"], c["vc"], c["bt"], c["sl"], c["scale"])
    gq = qkv.to(dev)[:, :H * D].view(3, H, D)
    out = torch.zeros(3, H, D, dtype=torch.float16, device=dev)
    r = ops.paged_decode_attention(gq, c["kc"].to(dev), c["vc"].to(dev), c["bt"].to(dev), c["sl"].to(dev),
                                   c["scale"], out=out)
    assert r.data_ptr() == out.data_ptr()
    check(out.float().cpu(), ref)


def test_bad_block_ids_are_ignored_not_faulted(dev):
    lens = [40]
    c = make_case(1, 2, 64, 16, lens, 61)
    c["bt"][0, 1] = 10 ** 6          # far outside the pool
    g = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    out = ops.paged_decode_attention(g["q"], g["kc"], g["vc"], g["bt"], g["sl"], c["scale"]).float().cpu()
    # equivalent to attending over blocks 0 and 2 only
    k = torch.cat([c["kc"][c["bt"][0, 0]], c["kc"][c["bt"][0, 2]][:8]], 0).float()
    v = torch.cat([c["vc"][c["bt"][0, 0]], c["vc"][c["bt"][0, 2]][:8]], 0).float()
    s = torch.einsum("hd,lhd->hl", c["q"][0].float(), k) * c["scale"]
    ref = torch.einsum("hl,lhd->hd", torch.softmax(s, -1), v)
    check(out[0], ref)


def test_argument_validation(dev):
    c = make_case(2, 2, 64, 16, [5, 6], 1)
    g = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    with pytest.raises(ValueError):
        ops.paged_decode_attention(g["q"].float(), g["kc"], g["vc"], g["bt"], g["sl"])
    with pytest.raises(ValueError):
        ops.paged_decode_attention(g["q"], g["kc"], g["vc"], g["bt"].long(), g["sl"])
    with pytest.raises(ValueError):
        ops.paged_decode_attention(g["q"], g["kc"], g["vc"], g["bt"], g["sl"].long())
    with pytest.raises(ValueError):
        ops.paged_decode_attention(g["q"], g["kc"], g["vc"].float(), g["bt"], g["sl"])
    with pytest.raises(RuntimeError):       # head size the kernels are not built for
        q = torch.zeros(2, 2, 48, dtype=torch.float16, device=dev)
        kc = torch.zeros(4, 16, 2, 48, dtype=torch.float16, device=dev)
        ops.paged_decode_attention(q, kc, kc, g["bt"], g["sl"])


# --------------------------------------------------- config 4 at full size

def config4(dev, seed=0, fp8=False):
    """128 sequences, 40x128, lognormal context, 65536-block pool, every block from the
    workspace with probability 1/2."""
    H, D, BS, B, POOL = 40, 128, 16, 128, 65536
    rng = np.random.default_rng(seed)
    lens = workloads.lognormal_lengths(rng, B)
    nblk = [-(-int(l) // BS) for l in lens]
    W = max(nblk)
    ids = rng.permutation(POOL)[:sum(nblk)]
    bt = np.zeros((B, W), dtype=np.int32)
    p = 0
    for b, n in enumerate(nblk):
        bt[b, :n] = ids[p:p + n]; p += n
    types = (rng.random((B, W)) < 0.5).astype(np.uint8)
    g = torch.Generator(device=dev).manual_seed(seed)
    dt = torch.float16

    def pool():
        x = torch.empty(POOL, BS, H, D, dtype=dt, device=dev)
        for i in range(0, POOL, 8192):
            x[i:i + 8192] = torch.randn(8192, BS, H, D, generator=g, dtype=torch.float32, device=dev).to(dt)
        return x
    return dict(lens=lens, bt=bt, types=types, pool=pool, H=H, D=D, BS=BS, B=B, POOL=POOL, g=g)


@pytest.mark.parametrize("fp8", [False, True])
def test_config4_hybrid_decode_attention_full_size(dev, fp8):
    cfg = config4(dev, 0)
    H, D, BS, B = cfg["H"], cfg["D"], cfg["BS"], cfg["B"]
    assert int(cfg["lens"].sum()) == 86514
    ks, vs = (0.04, 0.03) if fp8 else (1.0, 1.0)
    pools = []
    for i in range(4):          # K cache, V cache, workspace K, workspace V
        x = cfg["pool"]()
        if fp8:
            sc = ks if i % 2 == 0 else vs
            y = torch.empty(x.shape, dtype=torch.uint8, device=dev)
            for j in range(0, x.size(0), 8192):
                y[j:j + 8192] = torch.clamp(x[j:j + 8192].float() / sc, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
            x = y
        pools.append(x)
    kc, vc, wk, wv = pools
    q = randn((B, H, D), 3)
    bt = torch.from_numpy(cfg["bt"]); types = torch.from_numpy(cfg["types"])
    sl = torch.from_numpy(cfg["lens"].astype(np.int32))
    scale = D ** -0.5
    out = ops.paged_decode_attention(q.to(dev), kc, vc, bt.to(dev), sl.to(dev), scale, block_types=types.to(dev),
                                     ws_k_cache=wk, ws_v_cache=wv, k_scale=ks, v_scale=vs,
                                     max_seq_len=int(sl.max())).float().cpu()
    # oracle on a compact copy of the blocks in use (block ids remapped; the result
    # does not depend on where a block lives)
    used = np.unique(cfg["bt"])
    remap = np.zeros(cfg["POOL"], dtype=np.int32); remap[used] = np.arange(len(used), dtype=np.int32)
    u = torch.from_numpy(used).to(dev)
    ckc, cvc, cwk, cwv = (x[u].cpu() for x in (kc, vc, wk, wv))
    ref = OA.paged_decode_attention(q, ckc, cvc, torch.from_numpy(remap[cfg["bt"]]), sl, scale, block_types=types,
                                    ws_k_cache=cwk, ws_v_cache=cwv, k_scale=ks, v_scale=vs)
    check(out, ref)
