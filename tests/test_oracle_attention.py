"""Pins the attention / projection / fp8 oracles with independent witnesses."""
import numpy as np
import pytest
import torch

from oracle import attention as OA
from oracle import fp8 as O8
from oracle import reproject as OR
from util import randn


def build_paged(B, H, D, BS, lens, seed, nblk=None, dtype=torch.float16):
    rng = np.random.default_rng(seed)
    need = sum(-(-l // BS) for l in lens)
    nblk = nblk or need + 3
    perm = rng.permutation(nblk)
    W = max(-(-l // BS) for l in lens)
    bt = np.zeros((B, W), dtype=np.int32)
    k_dense, v_dense = [], []
    kc = randn((nblk, BS, H, D), seed + 1, dtype)
    vc = randn((nblk, BS, H, D), seed + 2, dtype)
    p = 0
    for b, l in enumerate(lens):
        n = -(-l // BS)
        bt[b, :n] = perm[p:p + n]; p += n
        k_dense.append(torch.cat([kc[i] for i in bt[b, :n]], 0)[:l])
        v_dense.append(torch.cat([vc[i] for i in bt[b, :n]], 0)[:l])
    return kc, vc, torch.from_numpy(bt), k_dense, v_dense


def softmax_f64(q, k, v, scale):
    """Textbook attention for one sequence in float64 numpy: q [H,D], k/v [L,H,D]."""
    q, k, v = (x.double().numpy() for x in (q, k, v))
    out = np.zeros_like(q)
    for h in range(q.shape[0]):
        s = k[:, h, :] @ q[h] * scale
        e = np.exp(s - s.max())
        out[h] = (e / e.sum()) @ v[:, h, :]
    return out


@pytest.mark.parametrize("seed", [0, 1])
def test_paged_attention_equals_dense_float64_softmax(seed):
    B, H, D, BS = 4, 3, 16, 16
    lens = [1, 16, 17, 45]
    kc, vc, bt, kd, vd = build_paged(B, H, D, BS, lens, seed)
    q = randn((B, H, D), seed + 9)
    scale = D ** -0.5
    out = OA.paged_decode_attention(q, kc, vc, bt, torch.tensor(lens, dtype=torch.int32), scale)
    for b in range(B):
        ref = softmax_f64(q[b], kd[b], vd[b], scale)
        np.testing.assert_allclose(out[b].numpy(), ref, rtol=1e-5, atol=1e-6)


def test_single_token_returns_its_value_row():
    B, H, D, BS = 2, 2, 8, 16
    kc, vc, bt, kd, vd = build_paged(B, H, D, BS, [1, 1], 3)
    q = randn((B, H, D), 0)
    out = OA.paged_decode_attention(q, kc, vc, bt, torch.tensor([1, 1], dtype=torch.int32), 0.3)
    for b in range(B):
        assert torch.equal(out[b], vd[b][0].float())


def test_equal_keys_give_the_mean_of_values():
    H, D, BS, L = 2, 8, 16, 37
    kc, vc, bt, kd, vd = build_paged(1, H, D, BS, [L], 4)
    kc[:] = kc[0, 0]          # every slot holds the same key
    q = randn((1, H, D), 1)
    out = OA.paged_decode_attention(q, kc, vc, bt, torch.tensor([L], dtype=torch.int32), 1.0)
    np.testing.assert_allclose(out[0].numpy(), vd[0].float().mean(0).numpy(), rtol=1e-5, atol=1e-6)


def test_block_permutation_leaves_the_result_unchanged():
    B, H, D, BS = 3, 2, 8, 16
    lens = [20, 33, 64]
    kc, vc, bt, _, _ = build_paged(B, H, D, BS, lens, 5)
    q = randn((B, H, D), 2)
    sl = torch.tensor(lens, dtype=torch.int32)
    a = OA.paged_decode_attention(q, kc, vc, bt, sl, 0.25)
    perm = torch.from_numpy(np.random.default_rng(0).permutation(kc.size(0)))
    inv = torch.empty_like(perm); inv[perm] = torch.arange(len(perm))
    b = OA.paged_decode_attention(q, kc[perm], vc[perm], inv[bt.long()].int(), sl, 0.25)
    assert torch.equal(a, b)


def test_hybrid_select_equals_moving_blocks_to_the_workspace():
    B, H, D, BS = 3, 2, 8, 16
    lens = [20, 33, 64]
    kc, vc, bt, _, _ = build_paged(B, H, D, BS, lens, 6)
    q = randn((B, H, D), 3)
    sl = torch.tensor(lens, dtype=torch.int32)
    a = OA.paged_decode_attention(q, kc, vc, bt, sl, 0.25)
    types = torch.from_numpy(np.random.default_rng(1).integers(0, 2, bt.shape).astype(np.uint8))
    # workspace holds the true data of the typed blocks; the cache copies of those blocks are poisoned
    wk, wv = kc.clone(), vc.clone()
    kc2, vc2 = kc.clone(), vc.clone()
    for b in range(B):
        for i in range(-(-lens[b] // BS)):
            if types[b, i]:
                kc2[bt[b, i]] = 77.0; vc2[bt[b, i]] = -55.0
            else:
                wk[bt[b, i]] = 77.0; wv[bt[b, i]] = -55.0
    b_ = OA.paged_decode_attention(q, kc2, vc2, bt, sl, 0.25, block_types=types, ws_k_cache=wk, ws_v_cache=wv)
    assert torch.equal(a, b_)


def test_flash_attn_with_kvcache_call_shape():
    B, H, D, BS = 2, 2, 8, 16
    kc, vc, bt, _, _ = build_paged(B, H, D, BS, [5, 30], 7)
    q = randn((B, 1, H, D), 4)
    sl = torch.tensor([5, 30], dtype=torch.int32)
    o = OA.flash_attn_with_kvcache(q, kc, vc, block_table=bt, cache_seqlens=sl, softmax_scale=0.2, causal=True)
    assert o.shape == (B, 1, H, D) and o.dtype == q.dtype
    ref = OA.paged_decode_attention(q[:, 0], kc, vc, bt, sl, 0.2).to(q.dtype)
    assert torch.equal(o[:, 0], ref)


def test_varlen_causal_attention_last_row_equals_decode():
    H, D = 2, 8
    lens = [5, 9]
    T = sum(lens)
    q, k, v = randn((T, H, D), 0), randn((T, H, D), 1), randn((T, H, D), 2)
    cu = torch.tensor([0, 5, 14], dtype=torch.int32)
    out = OA.varlen_causal_attention(q, k, v, cu, 0.3)
    for i, (a, e) in enumerate(zip(cu[:-1], cu[1:])):
        ref = softmax_f64(q[e - 1], k[a:e], v[a:e], 0.3)
        np.testing.assert_allclose(out[e - 1].numpy(), ref, rtol=1e-5, atol=1e-6)
        # first row of every sequence sees only itself
        assert torch.allclose(out[a], v[a].float())


# ------------------------------------------------------------------ projections

def test_projection_matches_float64_matmul_and_slices():
    Hd, T = 24, 7
    x = randn((T, Hd), 0); w = randn((3 * Hd, Hd), 1) * 0.1; b = randn((3 * Hd,), 2)
    w = w.half()
    kv = OR.kv_only(x, w, b, keep_fp32=True)
    ref = x.double().numpy() @ w.double().numpy()[Hd:].T + b.double().numpy()[Hd:]
    np.testing.assert_allclose(kv.numpy(), ref, rtol=1e-5, atol=1e-5)
    qq = OR.q_only(x, w, b, keep_fp32=True)
    np.testing.assert_allclose(qq.numpy(), x.double().numpy() @ w.double().numpy()[:Hd].T + b.double().numpy()[:Hd],
                               rtol=1e-5, atol=1e-5)
    k, v = OR.kv_reproject(x, w[Hd:], b[Hd:], keep_fp32=True)
    assert torch.equal(torch.cat([k, v], -1), kv)


def test_projection_special_weights():
    Hd, T = 8, 5
    x = randn((T, Hd), 3)
    w = torch.zeros(3 * Hd, Hd, dtype=torch.float16)
    w[Hd:2 * Hd] = torch.eye(Hd, dtype=torch.float16)          # K = x
    w[2 * Hd:, 0] = 1                                           # every V column = x[:, 0]
    k, v = OR.kv_only(x, w, None).chunk(2, -1)
    assert torch.equal(k, x) and torch.equal(v, x[:, :1].expand(T, Hd))


# ------------------------------------------------------------------------ fp8

def test_fp8_decode_table_from_bit_layout():
    tab = O8.decode_table()
    assert tab[0x00] == 0 and tab[0x80] == 0 and np.signbit(tab[0x80])
    assert tab[0x01] == 2.0 ** -9 and tab[0x07] == 7 * 2.0 ** -9          # subnormals
    assert tab[0x08] == 2.0 ** -6 and tab[0x38] == 1.0 and tab[0x7E] == 448.0
    assert np.isnan(tab[0x7F]) and np.isnan(tab[0xFF]) and tab[0xFE] == -448.0
    finite = tab[:0x7F]
    assert np.all(np.diff(finite) > 0)                                    # codes are ordered
    # PyTorch's own table
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(t, nan=-1), np.nan_to_num(tab, nan=-1))


def test_fp8_encode_is_nearest_with_ties_to_even():
    tab = O8.decode_table().astype(np.float64)
    pos = tab[:0x7F]                      # 127 finite non-negative values, ascending
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.uniform(0, 448, 20000), rng.uniform(0, 0.05, 20000), pos, (pos[:-1] + pos[1:]) / 2,   # exact ties
        np.nextafter(((pos[:-1] + pos[1:]) / 2).astype(np.float32), np.float32(0)).astype(np.float64),
        np.nextafter(((pos[:-1] + pos[1:]) / 2).astype(np.float32), np.float32(1e9)).astype(np.float64)])
    xs = xs.astype(np.float32)
    codes = O8.encode_e4m3(xs)
    # brute force: nearest table entry in float64, ties -> even code (even mantissa)
    d = np.abs(xs.astype(np.float64)[:, None] - pos[None, :])
    best = d.min(1)
    for x, c, row, bd in zip(xs, codes, d, best):
        cands = np.nonzero(row == bd)[0]
        want = cands[0] if len(cands) == 1 else [k for k in cands if k % 2 == 0][0]
        assert c == want, (x, c, cands)
    neg = O8.encode_e4m3(-xs)
    assert np.array_equal(neg & 0x7F, codes) and np.all((neg & 0x80) == 0x80)


def test_fp8_quantize_agrees_with_torch_cast_after_clamp():
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    x = x[~torch.isnan(x.float())]
    for scale in (1.0, 0.37, 4.0):
        ours = O8.quantize_e4m3(x, scale)
        y = torch.clamp(x.float() / scale, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
        assert torch.equal(ours, y)
        back = O8.dequantize_e4m3(ours, scale)
        assert torch.equal(back, y.view(torch.float8_e4m3fn).float() * scale)


@pytest.mark.parametrize("L", [1, 5, 33])
def test_absorbed_attention_equals_attention_over_reprojected_kv(L):
    """The absorbed form is an algebraic rearrangement: it must agree with the textbook softmax
    attention over k_t = W_k h_t + b_k, v_t = W_v h_t + b_v to float64 rounding, for any b_k."""
    H, D = 3, 8
    Hd = H * D
    g = torch.Generator().manual_seed(L)
    q = torch.randn(H, D, generator=g, dtype=torch.float64)
    x = torch.randn(L, Hd, generator=g, dtype=torch.float64)
    wk, wv = (torch.randn(Hd, Hd, generator=g, dtype=torch.float64) * 0.3 for _ in range(2))
    bk, bv = (torch.randn(Hd, generator=g, dtype=torch.float64) for _ in range(2))
    scale = 0.37
    k = (x @ wk.t() + bk).view(L, H, D)
    v = (x @ wv.t() + bv).view(L, H, D)
    ref = torch.empty(H, D, dtype=torch.float64)
    for h in range(H):
        p = torch.softmax(scale * (k[:, h] @ q[h]), dim=0)
        ref[h] = p @ v[:, h]
    got = OA.absorbed_hidden_attention(q, x, wk, wv, bv, scale)
    assert torch.allclose(got, ref, atol=1e-11, rtol=1e-11)
    # a dropped bias term or a transposed weight block would show here
    assert not torch.allclose(OA.absorbed_hidden_attention(q, x, wk, wv, None, scale), ref, atol=1e-3)
    if L > 1:
        assert not torch.allclose(OA.absorbed_hidden_attention(q, x, wk.t().contiguous(), wv, bv, scale), ref, atol=1e-3)


def test_prefix_attention_pinned_by_dense_softmax_and_its_two_limits():
    """``paged_prefix_attention`` (the prefix branch's flash_attn_varlen_func call): (a) every query row against a
    float64 softmax over the keys it may see, written from the definition; (b) with no prefix it is the plain
    causal prompt attention; (c) with one new token per sequence it is the decode attention."""
    B, H, D, BS = 3, 2, 8, 16
    klens, qlens = [37, 16, 50], [5, 16, 1]
    kc, vc, bt, k_dense, v_dense = build_paged(B, H, D, BS, klens, 11)
    q = randn((sum(qlens), H, D), 12)
    cu_q = torch.tensor([0] + list(np.cumsum(qlens)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(np.cumsum(klens)), dtype=torch.int32)
    out = OA.paged_prefix_attention(q, kc, vc, bt, cu_q, cu_k, 0.3)
    row = 0
    for b in range(B):
        for j in range(qlens[b]):
            n_vis = j + klens[b] - qlens[b] + 1                       # keys 0 .. j + klen - qlen
            for h in range(H):
                s = (k_dense[b][:n_vis, h].double() @ q[row, h].double()) * 0.3
                p = torch.softmax(s, 0)
                assert torch.allclose(out[row, h].double(), p @ v_dense[b][:n_vis, h].double(), atol=1e-5)
            row += 1
    # (b) no prefix: klen == qlen
    q2 = randn((sum(klens), H, D), 13)
    k2, v2 = torch.cat(k_dense), torch.cat(v_dense)
    full = OA.paged_prefix_attention(q2, kc, vc, bt, cu_k, cu_k, 0.3)
    assert torch.allclose(full, OA.varlen_causal_attention(q2, k2, v2, cu_k, 0.3), atol=1e-5)
    # (c) one query per sequence
    q3 = randn((B, H, D), 14)
    one = OA.paged_prefix_attention(q3, kc, vc, bt, torch.arange(B + 1, dtype=torch.int32), cu_k, 0.3)
    dec = OA.paged_decode_attention(q3, kc, vc, bt, torch.tensor(klens, dtype=torch.int32), 0.3)
    assert torch.allclose(one, dec, atol=1e-5)


def test_chunked_prompt_equals_one_shot_prompt():
    """The rows a prompt's second chunk produces through the prefix branch are the rows the whole prompt
    produces in one step."""
    H, D, BS = 2, 8, 16
    klens, ctx = [45, 20], [30, 7]
    kc, vc, bt, k_dense, v_dense = build_paged(2, H, D, BS, klens, 21)
    q_full = randn((sum(klens), H, D), 22)
    cu_k = torch.tensor([0] + list(np.cumsum(klens)), dtype=torch.int32)
    one_shot = OA.varlen_causal_attention(q_full, torch.cat(k_dense), torch.cat(v_dense), cu_k, 0.25)
    new = [torch.arange(int(cu_k[b]) + ctx[b], int(cu_k[b + 1])) for b in range(2)]
    idx = torch.cat(new)
    cu_q = torch.tensor([0] + list(np.cumsum([len(n) for n in new])), dtype=torch.int32)
    chunk = OA.paged_prefix_attention(q_full[idx], kc, vc, bt, cu_q, cu_k, 0.25)
    assert torch.allclose(chunk, one_shot[idx], atol=1e-5)
