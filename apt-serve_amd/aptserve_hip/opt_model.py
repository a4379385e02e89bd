"""Minimal OPT decoder stack over the hybrid cache — the GPU side of a serving step.

Mirrors ``OPTDecoderLayer.forward`` / ``OPTDecoder.forward``
(additional_designs/model_executor/models/aptserve_opt.py:179-212, 266-290) for the
pre-LayerNorm OPT variants (``do_layer_norm_before=True``: 125m, 1.3b ... 175b): the hidden
state cached for a hidden-cached sequence is the output of ``self_attn_layer_norm``, i.e.
the input of ``qkv_proj``.  Weights are random-initialised from a locally built config
(no checkpoint, no tokenizer).  Attention, the q/kv projections, the cache traffic, fc1 and
fc2 run on this library's kernels, and so does every (residual add, LayerNorm) pair
(``ops.add_layer_norm``: one launch instead of two element-wise ones; ``fused_norm=False``
keeps the plain PyTorch-ROCm ops); ReLU and the embedding lookup are PyTorch-ROCm ops.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from . import ops
from .backend import HybridOPTAttention, phase
from .metadata import HybridAttentionMetadata


@dataclass
class OPTConfig:
    hidden_size: int = 5120
    num_attention_heads: int = 40
    num_hidden_layers: int = 40
    ffn_dim: int = 20480
    vocab_size: int = 50272
    max_position_embeddings: int = 2048

    @staticmethod
    def opt_13b() -> "OPTConfig":
        return OPTConfig()

    @staticmethod
    def opt_125m() -> "OPTConfig":
        return OPTConfig(768, 12, 12, 3072, 50272, 2048)


def random_weights(cfg: OPTConfig, seed: int, device, dtype=torch.float16, layers: Optional[int] = None
                   ) -> Dict[str, torch.Tensor]:
    """N(0, 0.02) matrices, N(0, 0.02) biases, LayerNorm gains near 1 — generated on ``device``."""
    g = torch.Generator(device=device).manual_seed(seed)
    Hd, F_, L = cfg.hidden_size, cfg.ffn_dim, cfg.num_hidden_layers if layers is None else layers

    def n(*shape, std=0.02, mean=0.0):
        return (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * std + mean).to(dtype)
    w = {"embed_tokens": n(cfg.vocab_size, Hd), "embed_positions": n(cfg.max_position_embeddings + 2, Hd),
         "final_ln_w": n(Hd, std=0.02, mean=1.0), "final_ln_b": n(Hd)}
    for i in range(L):
        p = f"layers.{i}."
        w.update({p + "attn_ln_w": n(Hd, mean=1.0), p + "attn_ln_b": n(Hd),
                  p + "qkv_w": n(3 * Hd, Hd), p + "qkv_b": n(3 * Hd),
                  p + "out_w": n(Hd, Hd), p + "out_b": n(Hd),
                  p + "final_ln_w": n(Hd, mean=1.0), p + "final_ln_b": n(Hd),
                  p + "fc1_w": n(F_, Hd), p + "fc1_b": n(F_), p + "fc2_w": n(Hd, F_), p + "fc2_b": n(Hd)})
    return w


class HybridOPTDecoderLayer:
    def __init__(self, cfg: OPTConfig, w: Dict[str, torch.Tensor], prefix: str, **attn_kw) -> None:
        self.w, self.p, self.cfg = w, prefix, cfg
        self.self_attn = HybridOPTAttention(cfg.hidden_size, cfg.num_attention_heads, w[prefix + "qkv_w"],
                                            w[prefix + "qkv_b"], w[prefix + "out_w"], w[prefix + "out_b"], **attn_kw)

    def _mlp(self, x):
        """fc1 with its ReLU (stored by fc1's own epilogue), then fc2."""
        w, p = self.w, self.p
        with phase("projections"):
            x = ops.linear_nt(x, w[p + "fc1_w"], w[p + "fc1_b"], relu=True)
            return ops.linear_nt(x, w[p + "fc2_w"], w[p + "fc2_b"])

    def forward(self, hidden_states, kv_cache, shared_cache, md: HybridAttentionMetadata):
        """additional_designs/model_executor/models/aptserve_opt.py:179-212 with plain element-wise ops."""
        w, p, Hd = self.w, self.p, self.cfg.hidden_size
        residual = hidden_states
        hidden_states = F.layer_norm(hidden_states, (Hd,), w[p + "attn_ln_w"], w[p + "attn_ln_b"])
        hidden_states = self.self_attn(hidden_states, kv_cache, shared_cache, md)
        hidden_states = residual + hidden_states
        residual = hidden_states
        hidden_states = F.layer_norm(hidden_states, (Hd,), w[p + "final_ln_w"], w[p + "final_ln_b"])
        return residual + self._mlp(hidden_states)

    def forward_fused_norm(self, residual, normed, kv_cache, shared_cache, md, next_ln_w, next_ln_b):
        """The same layer with every (residual add, LayerNorm) pair in one launch.  ``normed`` is this layer's
        ``self_attn_layer_norm`` of ``residual`` (computed by the previous layer's last launch); returns the
        layer's output and the NEXT norm of it (the next layer's ``self_attn_layer_norm``, or the decoder's
        final one)."""
        w, p = self.w, self.p
        attn = self.self_attn(normed, kv_cache, shared_cache, md)
        normed, residual = ops.add_layer_norm(attn, residual, w[p + "final_ln_w"], w[p + "final_ln_b"])
        mlp = self._mlp(normed)
        normed, residual = ops.add_layer_norm(mlp, residual, next_ln_w, next_ln_b)
        return residual, normed

    __call__ = forward


class HybridOPTModel:
    def __init__(self, cfg: OPTConfig, weights: Dict[str, torch.Tensor], num_layers: Optional[int] = None,
                 fused_norm: bool = True, **attn_kw) -> None:
        self.cfg, self.w, self.fused_norm = cfg, weights, fused_norm
        n = cfg.num_hidden_layers if num_layers is None else num_layers
        self.layers = [HybridOPTDecoderLayer(cfg, weights, f"layers.{i}.", **attn_kw) for i in range(n)]

    def forward(self, input_ids, positions, kv_caches: List[torch.Tensor], shared_cache,
                md: HybridAttentionMetadata) -> torch.Tensor:
        w = self.w
        hidden_states = F.embedding(input_ids, w["embed_tokens"]) + F.embedding(positions + 2, w["embed_positions"])
        if not self.fused_norm or not self.layers:
            for layer, kv in zip(self.layers, kv_caches):
                hidden_states = layer(hidden_states, kv, shared_cache, md)
            return F.layer_norm(hidden_states, (self.cfg.hidden_size,), w["final_ln_w"], w["final_ln_b"])
        normed, _ = ops.add_layer_norm(hidden_states, None, w["layers.0.attn_ln_w"], w["layers.0.attn_ln_b"])
        for i, (layer, kv) in enumerate(zip(self.layers, kv_caches)):
            nxt = f"layers.{i + 1}.attn_ln_" if i + 1 < len(self.layers) else "final_ln_"
            hidden_states, normed = layer.forward_fused_norm(hidden_states, normed, kv, shared_cache, md,
                                                             w[nxt + "w"], w[nxt + "b"])
        return normed

    __call__ = forward

    def next_tokens(self, hidden_states, md: HybridAttentionMetadata) -> torch.Tensor:
        """Greedy next token of every sequence (last row of each prompt / every decode row)."""
        if md.num_prefills:
            last = md.seq_start_loc[1:md.num_prefills + 1].long() - 1
            hidden_states = hidden_states[last]
        logits = hidden_states @ self.w["embed_tokens"].t()
        return logits.argmax(-1)
