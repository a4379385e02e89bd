"""Oracle for paged decode attention over a hybrid cache (test infrastructure only).

The attention arithmetic is third-party in the reference: it calls
``vllm_flash_attn.flash_attn_with_kvcache`` (vllm-flash-attn as pinned by vLLM
0.5.0.post1; not under the reference tree) at
additional_designs/attention/backends/aptserve_flash_attn.py:452-461 (private
K/V cache) and :464-473 (shared cache).  Its published definition for a single
query token per sequence, restated:

    for sequence b, head h, with L = cache_seqlens[b]:
        K[j], V[j] = cache[block_table[b, j // BS], j % BS, h, :]   j in [0, L)
        out[b, h] = softmax_j(softmax_scale * <q[b, h], K[j]>) @ V

``causal=True`` is a no-op for one query aligned to the end of the keys and
``alibi_slopes`` is ``None`` for OPT.  The softmax is evaluated in fp32.

Hybrid extension: ``block_types[b, i] != 0`` means logical block ``i`` of
sequence ``b`` is read from the re-projection workspace
(``ws_k_cache``/``ws_v_cache``, same ``[nblk, BS, H, D]`` layout) instead of the
persistent K/V cache.  With ``block_types is None`` this is exactly
``flash_attn_with_kvcache``.

fp8 variant: caches hold e4m3 codes (uint8); K and V are dequantised as
``float(code) * k_scale`` / ``* v_scale`` before use.
"""

from __future__ import annotations

import torch

from .fp8 import dequantize_e4m3


def materialize_kv(k_cache, v_cache, block_table_row, seq_len, *, block_types_row=None,
                   ws_k_cache=None, ws_v_cache=None, k_scale=1.0, v_scale=1.0):
    """Dense fp32 ``K, V`` of shape ``[L, H, D]`` for one sequence."""
    bs = k_cache.size(1)
    nblk = (seq_len + bs - 1) // bs
    ks, vs = [], []
    for i in range(nblk):
        blk = int(block_table_row[i])
        from_ws = block_types_row is not None and int(block_types_row[i]) != 0
        kc, vc = (ws_k_cache, ws_v_cache) if from_ws else (k_cache, v_cache)
        kb, vb = kc[blk], vc[blk]
        if kb.dtype == torch.uint8:
            kb = dequantize_e4m3(kb, k_scale)
            vb = dequantize_e4m3(vb, v_scale)
        ks.append(kb.to(torch.float32))
        vs.append(vb.to(torch.float32))
    k = torch.cat(ks, 0)[:seq_len]
    v = torch.cat(vs, 0)[:seq_len]
    return k, v


def paged_decode_attention(q, k_cache, v_cache, block_tables, seq_lens, softmax_scale, *,
                           block_types=None, ws_k_cache=None, ws_v_cache=None,
                           k_scale=1.0, v_scale=1.0):
    """fp32 result ``[B, H, D]``; ``q`` is ``[B, H, D]`` (fp16/bf16/fp32)."""
    b_sz, h, d = q.shape
    out = torch.zeros(b_sz, h, d, dtype=torch.float32)
    qf = q.to(torch.float32)
    for b in range(b_sz):
        L = int(seq_lens[b])
        if L <= 0:
            continue
        k, v = materialize_kv(
            k_cache, v_cache, block_tables[b], L,
            block_types_row=None if block_types is None else block_types[b],
            ws_k_cache=ws_k_cache, ws_v_cache=ws_v_cache, k_scale=k_scale, v_scale=v_scale)
        # [H, L]
        s = torch.einsum("hd,lhd->hl", qf[b], k) * softmax_scale
        p = torch.softmax(s, dim=-1)
        out[b] = torch.einsum("hl,lhd->hd", p, v)
    return out


def flash_attn_with_kvcache(q, k_cache, v_cache, block_table=None, cache_seqlens=None,
                            softmax_scale=None, causal=True, alibi_slopes=None):
    """Same call shape as the third-party function for the decode case:
    ``q [B,1,H,D]`` -> ``[B,1,H,D]`` in ``q.dtype``."""
    assert q.size(1) == 1 and alibi_slopes is None
    if softmax_scale is None:
        softmax_scale = q.size(-1) ** -0.5
    o = paged_decode_attention(q[:, 0], k_cache, v_cache, block_table, cache_seqlens, softmax_scale)
    return o.to(q.dtype).unsqueeze(1)


def varlen_causal_attention(q, k, v, cu_seqlens, softmax_scale):
    """Prefill attention on freshly projected q/k/v (no cache read).

    Third-party ``flash_attn_varlen_func`` with ``causal=True`` as called at
    aptserve_flash_attn.py:414-426: sequences are packed along dim 0 and
    delimited by ``cu_seqlens`` (int32, leading 0); query ``i`` of a sequence
    attends to keys ``0..i`` of the same sequence.  fp32 result ``[T, H, D]``.
    """
    t, h, d = q.shape
    out = torch.zeros(t, h, d, dtype=torch.float32)
    for i in range(len(cu_seqlens) - 1):
        a, e = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
        qf, kf, vf = (x[a:e].to(torch.float32) for x in (q, k, v))
        s = torch.einsum("qhd,khd->hqk", qf, kf) * softmax_scale
        n = e - a
        mask = torch.ones(n, n, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[a:e] = torch.einsum("hqk,khd->qhd", p, vf)
    return out


def paged_prefix_attention(q, k_cache, v_cache, block_tables, cu_seqlens_q, cu_seqlens_k, softmax_scale):
    """``flash_attn_varlen_func(q, k=key_cache, v=value_cache, cu_seqlens_q=, cu_seqlens_k=, causal=True,
    block_table=)`` as called at additional_designs/attention/backends/aptserve_flash_attn.py:431-447 (the
    prefix branch), restated from the third-party function's published definition: the queries of sequence
    ``b`` are rows ``cu_seqlens_q[b]:cu_seqlens_q[b+1]`` of ``q``, its keys and values the first
    ``klen = cu_seqlens_k[b+1] - cu_seqlens_k[b]`` tokens read through ``block_tables[b]``, and with fewer
    queries than keys the causal mask is aligned to the bottom right: query ``j`` sees keys
    ``0 .. j + klen - qlen``.  fp32 result ``[tokens, H, D]``."""
    out = torch.zeros(q.shape, dtype=torch.float32)
    for b in range(len(cu_seqlens_q) - 1):
        q0, q1 = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1])
        klen = int(cu_seqlens_k[b + 1]) - int(cu_seqlens_k[b])
        qlen = q1 - q0
        if qlen == 0:
            continue
        k, v = materialize_kv(k_cache, v_cache, block_tables[b], klen)          # [klen, H, D] fp32
        s = torch.einsum("qhd,khd->hqk", q[q0:q1].float(), k) * softmax_scale
        visible = torch.arange(klen)[None, :] <= (torch.arange(qlen)[:, None] + (klen - qlen))
        s = s.masked_fill(~visible[None], float("-inf"))
        out[q0:q1] = torch.einsum("hqk,khd->qhd", torch.softmax(s, dim=-1), v)
    return out


def absorbed_hidden_attention(q, hidden_rows, w_k, w_v, b_v, softmax_scale):
    """Decode attention of ONE hidden-cached sequence computed on its cached hidden rows,
    without materialising K and V ("absorbed" projection weights).

    The reference re-projects the whole context every layer
    (additional_designs/model_executor/models/aptserve_opt.py:118-124:
    ``k_t = W_k h_t + b_k``, ``v_t = W_v h_t + b_v``) and then attends
    (aptserve_flash_attn.py:464-473).  Per head ``h`` with ``W_k[h], W_v[h]`` the ``[D, Hd]``
    row blocks of the projection weights:

        s[h, t]  = scale * <q[h], W_k[h] h_t + b_k[h]>
                 = scale * <W_k[h]^T q[h], h_t>  +  (a term that does not depend on t)
        p[h, :]  = softmax_t(s[h, :])            (shift invariant: the b_k term drops out)
        out[h]   = sum_t p[h, t] (W_v[h] h_t + b_v[h]) = W_v[h] (sum_t p[h, t] h_t) + b_v[h]

    ``q [H, D]``, ``hidden_rows [L, Hd]``, ``w_k``/``w_v [H*D, Hd]``, ``b_v [H*D]`` or None;
    float64 result ``[H, D]``.  Pinned in tests against ``paged_decode_attention`` applied to
    the re-projected K/V of the same rows.
    """
    h_cnt, d = q.shape
    hd = hidden_rows.shape[1]
    q64 = q.to(torch.float64)
    x = hidden_rows.to(torch.float64)
    wk = w_k.to(torch.float64).view(h_cnt, d, hd)
    wv = w_v.to(torch.float64).view(h_cnt, d, hd)
    qt = torch.einsum("hd,hdn->hn", q64, wk) * softmax_scale          # [H, Hd]
    s = qt @ x.t()                                                     # [H, L]
    p = torch.softmax(s, dim=-1)
    ctx = p @ x                                                        # [H, Hd]
    out = torch.einsum("hdn,hn->hd", wv, ctx)
    if b_v is not None:
        out = out + b_v.to(torch.float64).view(h_cnt, d)
    return out
