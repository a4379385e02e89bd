"""Oracle for one decoder layer's self-attention over the hybrid cache (test
infrastructure only): the operator sequence of ``OPTAttention.forward``
(additional_designs/model_executor/models/aptserve_opt.py:99-134) followed by
``FlashAttentionImpl.forward`` (additional_designs/attention/backends/aptserve_flash_attn.py:290-478),
composed from the oracle's own operators.

Decode batches that mix cache types follow the intended data flow: a K/V-cached
sequence attends over its private cache (its own block table), a hidden-cached
sequence over the K/V re-projected into the shared cache this step.  (The
reference routes both through the shared cache, whose mirror blocks ``0..N-1``
never hold the history of K/V-cached sequences; with ``literal=True`` that call
pattern is reproduced.)  All-hidden and no-hidden batches are the same in both.

``md`` is the dict of :func:`oracle.metadata.build_metadata`.  K/V are rounded
to the cache dtype before they are stored, as a kernel chain through an fp16
cache does.
"""

from __future__ import annotations

import torch

from . import attention as A
from . import cache_ops as C
from . import reproject as R


def _t(md, k):
    return torch.from_numpy(md[k])


def opt_attention(hidden_states, kv_cache, shared_cache, md, qkv_w, qkv_b, out_w, out_b, num_heads,
                  literal: bool = False, private_tables=None, kv_cache_dtype: str = "auto", k_scale: float = 1.0,
                  v_scale: float = 1.0, hidden_cache=None):
    """Returns the layer's attention output ``[tokens, Hd]`` (in ``hidden_states.dtype``) and
    mutates ``kv_cache`` / ``shared_cache`` like the reference.  ``private_tables``
    (list of lists) gives the private block table of each K/V-cached decode sequence for
    the intended flow of a mixed batch (the metadata's ``block_tables`` already holds it).

    ``kv_cache_dtype="fp8"`` (no counterpart in the reference, which asserts ``kv_scale == 1.0``): ``kv_cache``
    and ``shared_cache`` are uint8 caches of e4m3 codes written with ``k_scale`` / ``v_scale`` and read back
    dequantised; hidden rows then live in ``hidden_cache`` (activation dtype, same shape)."""
    fp8 = kv_cache_dtype != "auto"
    assert not (fp8 and literal)
    hc = kv_cache if hidden_cache is None else hidden_cache
    kw = dict(kv_cache_dtype=kv_cache_dtype, k_scale=k_scale, v_scale=v_scale) if fp8 else {}
    akw = dict(k_scale=k_scale, v_scale=v_scale) if fp8 else {}
    T, Hd = hidden_states.shape
    D = Hd // num_heads
    scale = D ** -0.5
    dt = hidden_states.dtype
    n_hidden, n_dec, n_pre = md["num_hidden_cache_tokens"], md["num_decode_tokens"], md["num_prefill_tokens"]
    sm = _t(md, "slot_mapping")
    if n_hidden != 0:
        C.hidden_to_cache(hidden_states, hc, sm, _t(md, "hidden_cache_use_input"),
                          _t(md, "hidden_cache_store_tot"))
        if n_dec != 0:
            holder = C.assemble_hidden_holder(hidden_states, hc, sm, md["num_tot_tokens"],
                                              _t(md, "hidden_holder_upd"), _t(md, "hidden_cache_use_tot"))
            q = R.q_only(hidden_states, qkv_w, qkv_b)
            k, v = R.kv_only(holder, qkv_w, qkv_b).chunk(2, -1)
        else:
            q, k, v = R._linear_fp32(hidden_states, qkv_w, qkv_b).to(dt).chunk(3, -1)
    else:
        q, k, v = R._linear_fp32(hidden_states, qkv_w, qkv_b).to(dt).chunk(3, -1)
    H = num_heads
    q3, k3, v3 = q.reshape(-1, H, D), k.reshape(-1, H, D), v.reshape(-1, H, D)
    kc, vc = kv_cache[0], kv_cache[1]
    out = torch.zeros(T, H, D, dtype=torch.float32)
    mixed = False
    if n_hidden == 0:
        C.reshape_and_cache_flash(k3, v3, kc, vc, sm, **kw)
    elif n_pre != 0:
        use = _t(md, "kv_cache_use_tot")
        C.reshape_and_cache_flash(k3[use], v3[use], kc, vc, sm[use], **kw)
    else:
        sk, sv = shared_cache[0], shared_cache[1]
        sms = _t(md, "slot_mapping_shared")
        mixed = md["num_tot_tokens"] != len(sms)
        if fp8:      # ranges (A) and (C) of mixed_kv_to_cache as two quantising scatters
            hu, ku = _t(md, "hidden_cache_use_tot"), _t(md, "kv_cache_use_tot")
            C.reshape_and_cache_flash(k3[hu], v3[hu], sk, sv, sms, **kw)
            if mixed:
                C.reshape_and_cache_flash(k3[ku], v3[ku], kc, vc, sm[ku], **kw)
        elif mixed:
            C.mixed_kv_to_cache(k3, v3, kc, vc, sk, sv, sm, sms, _t(md, "kv_cache_use_tot"),
                                _t(md, "hidden_cache_use_tot"))
        else:
            C.reshape_and_cache_flash(k3, v3, sk, sv, sms)
    if n_pre:
        out[:n_pre] = A.varlen_causal_attention(q3[:n_pre], k3[:n_pre], v3[:n_pre],
                                                md["seq_start_loc"][:md["num_prefills"] + 1], scale)
    if n_dec:
        bt = _t(md, "block_tables")[md["num_prefills"]:]
        sl = _t(md, "seq_lens_tensor")[md["num_prefills"]:]
        dq = q3[n_pre:]
        if n_hidden == 0:
            out[n_pre:] = A.paged_decode_attention(dq, kc, vc, bt, sl, scale, **akw)
        elif literal or not mixed:
            out[n_pre:] = A.paged_decode_attention(dq, sk, sv, bt, sl, scale, **akw)
        else:
            hid_seq = torch.zeros(n_dec, dtype=torch.uint8)
            hid_seq[_t(md, "hidden_cache_use_input")] = 1
            types = hid_seq.unsqueeze(1).expand(n_dec, bt.size(1)).contiguous()
            out[n_pre:] = A.paged_decode_attention(dq, kc, vc, bt, sl, scale, block_types=types,
                                                   ws_k_cache=sk, ws_v_cache=sv, **akw)
    attn = out.to(dt).reshape(T, Hd)
    return R._linear_fp32(attn, out_w, out_b).to(dt)
