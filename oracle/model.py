"""Oracle for the decoder stack (test infrastructure only): the same layer sequence as
additional_designs/model_executor/models/aptserve_opt.py:179-212 and :266-290 with the
oracle's attention, on the CPU.  Activations are kept in the model dtype between
operators, like the GPU path; every operator computes in fp32 and rounds once."""

from __future__ import annotations

import torch
import torch.nn.functional as F

from . import layer as L
from . import reproject as R


def _ln(x, w, b):
    return F.layer_norm(x.float(), (x.size(-1),), w.float(), b.float()).to(x.dtype)


def decoder_forward(weights, num_layers, num_heads, input_ids, positions, kv_caches, shared_cache, md):
    w = weights
    h = (F.embedding(input_ids, w["embed_tokens"]).float() + F.embedding(positions + 2, w["embed_positions"]).float()
         ).to(w["embed_tokens"].dtype)
    for i in range(num_layers):
        p = f"layers.{i}."
        res = h
        x = _ln(h, w[p + "attn_ln_w"], w[p + "attn_ln_b"])
        x = L.opt_attention(x, kv_caches[i], shared_cache, md, w[p + "qkv_w"], w[p + "qkv_b"], w[p + "out_w"],
                            w[p + "out_b"], num_heads)
        h = (res.float() + x.float()).to(h.dtype)
        res = h
        x = _ln(h, w[p + "final_ln_w"], w[p + "final_ln_b"])
        x = R._linear_fp32(x, w[p + "fc1_w"], w[p + "fc1_b"]).to(h.dtype)
        x = torch.relu(x)
        x = R._linear_fp32(x, w[p + "fc2_w"], w[p + "fc2_b"]).to(h.dtype)
        h = (res.float() + x.float()).to(h.dtype)
    return _ln(h, w["final_ln_w"], w["final_ln_b"])
