"""MFMA q-only / kv-only projection against the oracle (exact fp32 product of the
fp16-rounded operands, rounded once).

Tolerances: 1e-3 relative on the fp32-accumulated value is the stated bar; the
kernel rounds its fp32 accumulator once to fp16, so against the oracle's fp16
result an element may differ by one fp16 ulp (2^-10 relative) plus the
accumulation-order noise — checked as |d| <= 1e-3*|ref| + 2e-3 and, for the
stated absolute bar of an fp16 output, |d| <= 2e-2.
"""
import numpy as np
import pytest
import torch

from aptserve_hip import layers, ops
from oracle import reproject as OR
from util import randn

pytestmark = pytest.mark.gpu


def check(out, ref32, dtype=torch.float16):
    out = out.float().cpu()
    d = (out - ref32).abs()
    if dtype == torch.float16:   # bf16 rounds in steps of 2^-8 relative: above |4| half a step alone exceeds 2e-2
        assert d.max().item() <= 2e-2, f"max abs error {d.max().item()}"
    ulp = 2 ** -10 if dtype == torch.float16 else 2 ** -7
    bound = (1e-3 + ulp) * ref32.abs() + 2e-3
    bad = (d > bound).sum().item()
    assert bad == 0, f"{bad} elements outside tolerance, worst {d.max().item()}"


@pytest.mark.parametrize("M", [1, 7, 49, 64, 65, 128, 129, 192, 193, 255, 256, 257, 384, 385, 700])   # 64- to 256-row tiles
@pytest.mark.parametrize("N,K", [(256, 64), (512, 192), (1536, 768)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_nt_small(dev, M, N, K, dtype):
    x = randn((M, K), M, dtype)
    w = (randn((N, K), N) * 0.05).to(dtype)
    b = randn((N,), 3, dtype)
    ref = OR._linear_fp32(x, w, b)
    out = ops.linear_nt(x.to(dev), w.to(dev), b.to(dev))
    check(out, ref, dtype)
    out2 = ops.linear_nt(x.to(dev), w.to(dev), None)
    check(out2, OR._linear_fp32(x, w, None), dtype)


@pytest.mark.parametrize("M", [3, 8, 16, 17, 32, 33, 48])
@pytest.mark.parametrize("N,K", [(256, 64), (512, 1600), (1024, 2048), (2560, 5120), (16896, 1024), (20992, 512)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_nt_few_rows_weight_stream(dev, M, N, K, dtype):
    """3..48 rows: weight rows through the row-streaming MFMA core (16-, 32- and 48-row images), K in one part
    or in parts added by the reduce kernel, with a short last chunk (K = 64, 1600) and without (2048, 5120), and
    workgroups of fewer than 128 weight rows with a short last one (N = 16896, 20992);
    the same product without a workspace goes through the single-launch kernels and must agree."""
    x = randn((M, K), M + 1, dtype)
    w = (randn((N, K), N + 1) * 0.02).to(dtype)    # outputs of magnitude ~1: the absolute bar holds for bf16 too
    b = (randn((N,), 5) * 0.2).to(dtype)
    ref = OR._linear_fp32(x, w, b)
    out = ops.linear_nt(x.to(dev), w.to(dev), b.to(dev))
    check(out, ref, dtype)
    if M <= 16:
        check(ops.linear_nt(x.to(dev), w.to(dev), b.to(dev), split_k=False), ref, dtype)
    check(ops.linear_nt(x.to(dev), w.to(dev), None), OR._linear_fp32(x, w, None), dtype)


@pytest.mark.parametrize("M", [3, 5, 8])
@pytest.mark.parametrize("N,K", [(5120, 5120), (15360, 5120), (1024, 2048), (768, 4096), (512, 6144), (8192, 2048)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_nt_k_split_inside_the_workgroups(dev, M, N, K, dtype):
    """3..8 rows with K of 2048, 4096, 5120 or 6144: 16 (or, for few weight rows, 8) weight rows per workgroup,
    the eight wavefronts an eighth of K each, all activation rows staged in LDS; no workspace is planned for these
    shapes.  Against the fp32 oracle, with a row map, a strided x, the ReLU flag and without bias."""
    assert ops._lib.load().aps_linear_nt_splits(M, N, K) == 1
    assert ops._lib.load().aps_linear_nt_workspace_bytes(M, N, K) == 0
    wide = randn((M, K + 24), M + K, dtype)
    x = wide[:, 8:8 + K]
    w = (randn((N, K), N + 1) * 0.02).to(dtype)
    b = (randn((N,), 5) * 0.2).to(dtype)
    ref = OR._linear_fp32(x, w, b)
    xd, wd, bd = wide.to(dev)[:, 8:8 + K], w.to(dev), b.to(dev)
    out = ops.linear_nt(xd, wd, bd)
    check(out, ref, dtype)
    assert torch.equal(ops.linear_nt(xd, wd, bd, relu=True), torch.relu(out))
    check(ops.linear_nt(xd, wd, None), OR._linear_fp32(x, w, None), dtype)
    perm = torch.from_numpy(np.random.default_rng(M).permutation(16)[:M].astype(np.int64)); perm[1] = -1
    dest = torch.full((16, N), 7.0, dtype=dtype, device=dev)
    ops.linear_nt(xd, wd, bd, out=dest, out_row_map=perm.to(dev))
    keep = perm >= 0
    assert torch.equal(dest[perm[keep].to(dev)], out[keep.to(dev)])
    untouched = torch.ones(16, dtype=torch.bool); untouched[perm[keep]] = False
    assert (dest[untouched.to(dev)] == 7).all()


def test_few_rows_weight_stream_strides_row_map_and_workspace(dev):
    K, N, M = 2048, 2560, 21
    wide = randn((M, 2 * K + 8), 0)
    x = wide[:, 8:8 + K]                                   # row stride 2K+8, 16-byte aligned start
    wfull = (randn((N + 256, K), 1) * 0.05).half()
    w = wfull[256:]                                        # a row slice of a larger weight
    b = randn((N,), 2).half()
    ref = OR._linear_fp32(x, w, b)
    xd, wd, bd = wide.to(dev)[:, 8:8 + K], wfull.to(dev)[256:], b.to(dev)
    assert ops._lib.load().aps_linear_nt_splits(M, N, K) > 1
    check(ops.linear_nt(xd, wd, bd), ref)
    rows = 64
    perm = torch.from_numpy(np.random.default_rng(1).permutation(rows)[:M].astype(np.int64)); perm[3] = -1
    dest = torch.full((rows, N), 7.0, dtype=torch.float16, device=dev)
    ops.linear_nt(xd, wd, bd, out=dest, out_row_map=perm.to(dev))
    dest = dest.cpu()
    keep = perm >= 0
    check(dest[perm[keep]], ref[keep])
    untouched = torch.ones(rows, dtype=torch.bool); untouched[perm[keep]] = False
    assert (dest[untouched] == 7).all()
    # through the C ABI: a workspace that is too small is an error (-3), not a silent fallback
    small = torch.empty(1024, dtype=torch.uint8, device=dev)
    out = torch.empty(M, N, dtype=torch.float16, device=dev)
    st = ops._lib.load().aps_linear_nt(xd.data_ptr(), wd.data_ptr(), bd.data_ptr(), out.data_ptr(), M, N, K,
                                       xd.stride(0), wd.stride(0), out.stride(0), None, M, 0, 0, small.data_ptr(),
                                       small.numel(), None, None)
    torch.cuda.synchronize()
    assert st == -3


@pytest.mark.parametrize("M", [1, 2, 5, 16, 30, 48, 49, 100, 300, 3328])   # every kernel family and the tail split
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_relu_epilogue_equals_relu_of_the_rounded_product(dev, M, dtype):
    """fc1 with its activation (aptserve_opt.py:204-205): negative results are stored as zero, everything else
    bit for bit as without the flag — in the epilogue of every kernel of the family and in the kernels that add
    K-split partial products."""
    N, K = (512, 192) if M < 1000 else (5120, 1024)
    x, w, b = randn((M, K), M, dtype).to(dev), (randn((N, K), 1) * 0.05).to(dtype).to(dev), randn((N,), 3, dtype).to(dev)
    for split_k in (True, False):
        plain = ops.linear_nt(x, w, b, split_k=split_k)
        act = ops.linear_nt(x, w, b, split_k=split_k, relu=True)
        assert (plain < 0).any() and torch.equal(act, torch.relu(plain))


@pytest.mark.parametrize("M,N,K", [(3, 768, 1600), (9, 5120, 5120), (5, 5120, 20480), (17, 1536, 1088), (48, 5120, 5120),
                                   (33, 7680, 5120), (9, 256, 2048)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_k_split_summed_inside_the_launch_equals_the_two_launch_sum(dev, M, N, K, dtype):
    """The K split of a decode step's few rows with tile counters (the workgroup that stores a tile's last
    partial product adds the parts, in part order) against the same split summed by the second kernel: the same
    bits, the counters zero again afterwards, call after call on the same counters."""
    lib = ops._lib.load()
    x, w, b = randn((M, K), M, dtype).to(dev), (randn((N, K), 1) * 0.05).to(dtype).to(dev), randn((N,), 3, dtype).to(dev)
    assert lib.aps_linear_nt_splits(M, N, K) > 1
    ws = torch.empty(lib.aps_linear_nt_workspace_bytes(M, N, K), dtype=torch.uint8, device=dev)
    code = 0 if dtype == torch.float16 else 1
    two = torch.empty(M, N, dtype=dtype, device=dev)
    st = lib.aps_linear_nt(x.data_ptr(), w.data_ptr(), b.data_ptr(), two.data_ptr(), M, N, K, K, K, N, None, M, code, 0,
                           ws.data_ptr(), ws.numel(), None, None)
    assert st == 0
    counters = ops._tile_counters(dev)
    for rep in range(30):          # the parts cross between workgroups inside the launch: every repetition must agree
        relu = rep % 3 == 1
        one = ops.linear_nt(x, w, b, relu=relu)
        assert torch.equal(one, torch.relu(two) if relu else two), rep
    assert int(counters.abs().sum()) == 0


def test_identity_and_one_hot_weights_are_exact(dev):
    """W = I reproduces x bit for bit; a one-hot row picks one input column."""
    K = N = 256
    x = randn((300, K), 0)
    w = torch.eye(N, K, dtype=torch.float16)
    out = ops.linear_nt(x.to(dev), w.to(dev)).cpu()
    assert torch.equal(out, x)
    for m in (2, 5, 16, 40):                               # the few-row kernels as well
        assert torch.equal(ops.linear_nt(x[:m].to(dev), w.to(dev)).cpu(), x[:m])
    w2 = torch.zeros(N, K, dtype=torch.float16); w2[:, 17] = 1
    out = ops.linear_nt(x.to(dev), w2.to(dev)).cpu()
    assert torch.equal(out, x[:, 17:18].expand(300, N))


def test_qkv_proj_q_only_and_kv_only_on_weight_slices(dev):
    """The reference slices the fused weight in place (aptserve_linear.py:115-130);
    the kernel reads the row slice through its stride, no copy."""
    Hd, T = 768, 130
    w = (randn((3 * Hd, Hd), 1) * 0.03).half()
    b = randn((3 * Hd,), 2)
    x = randn((T, Hd), 3)
    proj = layers.QKVLinear(w.to(dev), b.to(dev))
    q, none = proj(x.to(dev), q_only=True)
    assert none is None
    check(q, OR.q_only(x, w, b, keep_fp32=True))
    kv, _ = proj(x.to(dev), kv_only=True)
    check(kv, OR.kv_only(x, w, b, keep_fp32=True))
    k, v = kv.chunk(2, dim=-1)
    kr, vr = OR.kv_reproject(x, w[Hd:], b[Hd:], keep_fp32=True)
    check(k, kr); check(v, vr)
    full, _ = proj(x.to(dev))
    check(full, OR._linear_fp32(x, w, b))
    with pytest.raises(NotImplementedError):
        proj(x.to(dev), q_only=True, kv_only=True)


def test_strided_activations_and_row_scatter_epilogue(dev):
    K, N, M = 128, 256, 77
    wide = randn((M, 3 * K), 0)
    x = wide[:, K:2 * K]
    w = (randn((N, K), 1) * 0.1).half()
    ref = OR._linear_fp32(x, w, None)
    out = ops.linear_nt(wide.to(dev)[:, K:2 * K], w.to(dev))
    check(out, ref)
    # scatter: row m -> dest[perm[m]], rows mapped to -1 are dropped, untouched rows keep their content
    rng = np.random.default_rng(0)
    rows = 200
    perm = torch.from_numpy(rng.permutation(rows)[:M].astype(np.int64)); perm[5] = -1
    dest = torch.full((rows, N), 7.0, dtype=torch.float16, device=dev)
    ops.linear_nt(wide.to(dev)[:, K:2 * K], w.to(dev), out=dest, out_row_map=perm.to(dev))
    dest = dest.cpu()
    keep = perm >= 0
    check(dest[perm[keep]], ref[keep])
    untouched = torch.ones(rows, dtype=torch.bool); untouched[perm[keep]] = False
    assert (dest[untouched] == 7).all()


@pytest.mark.parametrize("T", [5, 300, 1100])          # split-K (few tiles) and the one-pass kernel
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kv_reproject_into_cache_slots(dev, T, dtype):
    """The fused epilogue puts K and V of every row into its slot: equal, bit for bit, to the
    plain projection followed by an index_put; rows with -1 or an out-of-range slot are dropped;
    every other slot keeps its content."""
    H, D, BS, nblk = 4, 64, 16, 80
    Hd = H * D
    rng = np.random.default_rng(T)
    x = randn((T, Hd), 1, dtype)
    w = (randn((2 * Hd, Hd), 2) * 0.05).to(dtype)
    b = randn((2 * Hd,), 3, dtype)
    ws_slots, priv_slots = 2 * nblk * BS, nblk * BS
    # a random third of the rows go to the private caches, the rest to the workspace; slots are distinct
    to_priv = rng.random(T) < 0.33
    dest = np.empty(T, dtype=np.int64)
    dest[to_priv] = -(rng.permutation(priv_slots)[:to_priv.sum()] + 2)
    dest[~to_priv] = rng.permutation(ws_slots)[:(~to_priv).sum()]
    dropped = rng.choice(T, size=min(3, T - 1), replace=False)
    dest[dropped[0]] = -1
    if len(dropped) > 1:
        dest[dropped[1]] = ws_slots + 5              # beyond the workspace
    if len(dropped) > 2:
        dest[dropped[2]] = -(priv_slots + 9 + 2)     # beyond the private cache
    caches = [torch.full((n, BS, H, D), 3.0, dtype=dtype, device=dev) for n in (2 * nblk, 2 * nblk, nblk, nblk)]
    ops.kv_reproject_to_cache(x.to(dev), w.to(dev), b.to(dev), *caches, torch.from_numpy(dest).to(dev))
    plain = ops.linear_nt(x.to(dev), w.to(dev), b.to(dev)).cpu()
    check(plain, OR._linear_fp32(x, w, b), dtype)
    expect = [torch.full((n * BS, Hd), 3.0, dtype=dtype) for n in (2 * nblk, 2 * nblk, nblk, nblk)]
    for t in range(T):
        d = int(dest[t])
        if 0 <= d < ws_slots:
            expect[0][d], expect[1][d] = plain[t, :Hd], plain[t, Hd:]
        elif d <= -2 and -(d + 2) < priv_slots:
            expect[2][-(d + 2)], expect[3][-(d + 2)] = plain[t, :Hd], plain[t, Hd:]
    for got, exp in zip(caches, expect):
        assert torch.equal(got.cpu().view(-1, Hd), exp)
    # one cache pair may be absent when no row goes there
    only_ws = np.where(dest >= 0, dest, -1)
    c2 = [torch.full((2 * nblk, BS, H, D), 3.0, dtype=dtype, device=dev) for _ in range(2)]
    ops.kv_reproject_to_cache(x.to(dev), w.to(dev), b.to(dev), c2[0], c2[1], None, None,
                              torch.from_numpy(only_ws).to(dev))
    assert torch.equal(c2[0].cpu(), caches[0].cpu()) and torch.equal(c2[1].cpu(), caches[1].cpu())
    with pytest.raises(ValueError):
        ops.kv_reproject_to_cache(x.to(dev), w.to(dev), b.to(dev), None, None, None, None,
                                  torch.from_numpy(dest).to(dev))


@pytest.mark.parametrize("T", [60, 300, 1100])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kv_reproject_reading_cached_rows_in_place(dev, T, dtype):
    """``kv_reproject_gathered`` takes row t of its left operand from a slot of the paged cache or from a row
    of the step's hidden states (aptserve_opt.py:112-121 assembles them in a holder first): the caches must end
    up bit-identical to the holder assembled on the host and pushed through ``kv_reproject_to_cache``, rows whose
    source does not exist (destination -1) must leave no trace, and every other slot keeps its content."""
    H, D, BS, nblk, B = 4, 64, 16, 40, 9
    Hd = H * D
    rng = np.random.default_rng(100 + T)
    paged = randn((2, nblk, BS, H, D), 5, dtype)
    hs = randn((B, Hd), 6, dtype)
    w = (randn((2 * Hd, Hd), 7) * 0.05).to(dtype)
    b = randn((2 * Hd,), 8, dtype)
    n_slots = 2 * nblk * BS
    src = rng.integers(0, n_slots, T).astype(np.int64)
    from_input = rng.random(T) < 0.15
    src[from_input] = -(rng.integers(0, B, from_input.sum()) + 1)
    ws_slots, priv_slots = 2 * nblk * BS, nblk * BS
    dest = rng.permutation(ws_slots)[:T].astype(np.int64)
    to_priv = rng.random(T) < 0.25
    dest[to_priv] = -(rng.permutation(priv_slots)[:to_priv.sum()] + 2)
    bad = rng.choice(T, size=3, replace=False)
    src[bad[0]], src[bad[1]], src[bad[2]] = n_slots + 7, -(B + 3), -(2 ** 40)      # no such slot / row
    dest[bad] = -1
    flat = paged.view(n_slots, Hd)
    holder = torch.zeros(T, Hd, dtype=dtype)
    for t in range(T):
        if t in bad:
            continue
        holder[t] = flat[src[t]] if src[t] >= 0 else hs[-(src[t] + 1)]
    shapes = (2 * nblk, 2 * nblk, nblk, nblk)
    want = [torch.full((n, BS, H, D), 3.0, dtype=dtype, device=dev) for n in shapes]
    ops.kv_reproject_to_cache(holder.to(dev), w.to(dev), b.to(dev), *want, torch.from_numpy(dest).to(dev))
    got = [torch.full((n, BS, H, D), 3.0, dtype=dtype, device=dev) for n in shapes]
    ops.kv_reproject_gathered(hs.to(dev), paged.to(dev), torch.from_numpy(src).to(dev), w.to(dev), b.to(dev), *got,
                              torch.from_numpy(dest).to(dev))
    for g_, w_ in zip(got, want):
        assert torch.equal(g_, w_)
    # against the oracle's product, not only against the other HIP flow
    ref = OR._linear_fp32(holder, w, b)
    t = int(np.nonzero(dest >= 0)[0][0])
    check(torch.cat([got[0].view(-1, Hd)[dest[t]], got[1].view(-1, Hd)[dest[t]]]).cpu()[None], ref[t][None], dtype)
    with pytest.raises(ValueError):      # one destination per source row
        ops.kv_reproject_gathered(hs.to(dev), paged.to(dev), torch.from_numpy(src).to(dev), w.to(dev), b.to(dev),
                                  *got, torch.from_numpy(dest[:-1]).to(dev))
    with pytest.raises(ValueError):      # the cache must hold the operand dtype
        ops.kv_reproject_gathered(hs.to(dev), paged.float().to(dev), torch.from_numpy(src).to(dev), w.to(dev),
                                  b.to(dev), *got, torch.from_numpy(dest).to(dev))


@pytest.mark.parametrize("M,N,K,split_k", [(5, 768, 1216, False),     # row-streaming kernel, K not a multiple of its 512-element pieces
                                          (9, 256, 256, True),       # weight streaming, K shorter than one 512-element chunk
                                          (12, 512, 192, False),     # 16-row kernel, odd number of 32-wide steps
                                          (3, 512, 256, True), (48, 1280, 1344, True), (100, 2048, 384, False)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_activations_that_end_where_their_storage_ends(dev, M, N, K, split_k, dtype):
    """x is the right half of a [M, 2K] tensor: row stride 2K, and the last row ends exactly where the storage
    ends.  No kernel may read past a row's K elements there (the loads that cover a partial piece of K, or rows
    past M, must be masked by the buffer bounds or redirected), and the product must not change."""
    xs = randn((M, 2 * K), M + K, dtype)
    w = (randn((N, K), 2) * 0.05).to(dtype)
    b = randn((N,), 3, dtype)
    ref = OR._linear_fp32(xs[:, K:], w, b)
    out = ops.linear_nt(xs.to(dev)[:, K:], w.to(dev), b.to(dev), split_k=split_k)
    check(out, ref, dtype)
    out2 = ops.linear_nt(xs[:, K:].contiguous().to(dev), w.to(dev), b.to(dev), split_k=split_k)
    assert torch.equal(out, out2)


def test_unsupported_shapes_raise(dev):
    x = torch.zeros(4, 64, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError):
        ops.linear_nt(x, torch.zeros(100, 64, dtype=torch.float16, device=dev))     # N not a multiple of 256
    with pytest.raises(RuntimeError):
        ops.linear_nt(torch.zeros(4, 40, dtype=torch.float16, device=dev),
                      torch.zeros(256, 40, dtype=torch.float16, device=dev))        # K not a multiple of 64
    with pytest.raises(ValueError):
        ops.linear_nt(x.float(), torch.zeros(256, 64, device=dev))


def test_config3_kv_reprojection_opt13b(dev):
    """[T,5120] x W_kv[10240,5120]^T, W ~ N(0,0.02), X ~ N(0,1).  T=4096 against the full
    oracle product; T=16384 on 384 sampled rows (every row is an independent product)."""
    Hd = 5120
    w = (randn((2 * Hd, Hd), 1, torch.float32) * 0.02).half()
    b = randn((2 * Hd,), 2)
    dw, db = w.to(dev), b.to(dev)
    x = randn((4096, Hd), 3)
    out = ops.kv_reproject(x.to(dev), dw, db)
    torch.set_num_threads(16)
    check(out, OR._linear_fp32(x, w, b))
    x2 = randn((16384, Hd), 4)
    out2 = ops.kv_reproject(x2.to(dev), dw, db)
    rows = torch.from_numpy(np.random.default_rng(0).choice(16384, 384, replace=False))
    check(out2[rows.to(dev)], OR._linear_fp32(x2[rows], w, b))


def test_matrix_core_probe_runs_and_adds_what_it_multiplies(dev):
    """aps_mfma_probe is a measurement aid, but its kernels are real: with all-ones operands every accumulator of a
    16x16x32 product grows by 32 per round (16 per round for 32x32x16), and a thread sums all of its accumulators."""
    from aptserve_hip import probes
    lib = probes.load()
    st = torch.cuda.current_stream().cuda_stream
    ones = torch.ones(16384, dtype=torch.float16, device=dev)
    zeros = torch.zeros(16384, dtype=torch.float16, device=dev)
    sink = torch.empty(4 * 256, dtype=torch.float32, device=dev)
    iters = 3
    for shape, per_thread in ((0, 16 * 16 * 16.0), (1, 32 * 4 * 32.0)):
        assert lib.aps_mfma_probe(shape, 0, ones.data_ptr(), sink.data_ptr(), 4, iters, st) == 0
        torch.cuda.synchronize()
        assert torch.all(sink == per_thread * iters), (shape, sink[:4])
        assert lib.aps_mfma_probe(shape, 0, zeros.data_ptr(), sink.data_ptr(), 4, iters, st) == 0
        torch.cuda.synchronize()
        assert torch.all(sink == 0)


def test_issue_mix_probe_shapes_compute_what_they_say(dev):
    """Shapes 2..6 of aps_mfma_probe interleave MFMAs with vector units (v_exp_f32 and three v_fma_f32 on eight
    register values per lane, two units per value and round).  With zero operands the products are zero and every
    value follows x -> fma(fma(fma(2^x, c0, c1), c0, c1), c0, c1) from 0, whatever the order of issue."""
    import numpy as np
    from aptserve_hip import probes
    lib = probes.load()
    st = torch.cuda.current_stream().cuda_stream
    zeros = torch.zeros(16384, dtype=torch.float16, device=dev)
    iters = 3
    x = np.float64(0.0)
    c0, c1 = np.float64(np.float32(1e-3)), np.float64(np.float32(0.5))
    for _ in range(2 * iters):
        x = np.float64(np.float32(np.exp2(x)))
        for _ in range(3):
            x = np.float64(np.float32(x * c0 + c1))
    for shape, threads in ((2, 256), (3, 256), (4, 256), (5, 512), (6, 512)):
        sink = torch.full((4 * threads,), float("nan"), dtype=torch.float32, device=dev)
        assert lib.aps_mfma_probe(shape, 0, zeros.data_ptr(), sink.data_ptr(), 4, iters, st) == 0
        torch.cuda.synchronize()
        assert torch.allclose(sink, torch.full_like(sink, 8 * float(x)), rtol=1e-5, atol=0), (shape, sink[:4])
