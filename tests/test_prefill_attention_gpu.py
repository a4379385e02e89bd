"""Prompt-step causal attention (MFMA) against the fp32 oracle; 2e-2 absolute is the stated bar
for an fp16 result, the kernel is held to 5e-3 (P is rounded to fp16 before the PV product)."""
import numpy as np
import pytest
import torch

from aptserve_hip import ops
from oracle import attention as OA
from util import randn

pytestmark = pytest.mark.gpu


def run(dev, lens, H, D, dtype=torch.float16, seed=0, strided=False):
    T = sum(lens)
    if strided:   # chunk views of a fused qkv activation, row stride 3*H*D
        qkv = randn((T, 3 * H * D), seed, dtype)
        q, k, v = (x.view(T, H, D) for x in qkv.chunk(3, -1))
        dq, dk, dv = (x.view(T, H, D) for x in qkv.to(dev).chunk(3, -1))
    else:
        q, k, v = randn((T, H, D), seed, dtype), randn((T, H, D), seed + 1, dtype), randn((T, H, D), seed + 2, dtype)
        dq, dk, dv = q.to(dev), k.to(dev), v.to(dev)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    ref = OA.varlen_causal_attention(q, k, v, cu, D ** -0.5)
    out = ops.flash_attn_varlen_func(q=dq, k=dk, v=dv, cu_seqlens_q=cu.to(dev), cu_seqlens_k=None,
                                     max_seqlen_q=max(lens), max_seqlen_k=max(lens), softmax_scale=D ** -0.5,
                                     causal=True)
    out = out.float().cpu()
    err = (out - ref).abs().max().item()
    assert err <= 2e-2, err
    tol = 5e-3 if dtype == torch.float16 else 2e-2
    assert torch.allclose(out, ref, atol=tol, rtol=tol), err
    return out, ref


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_prefill_attention_ragged_lengths(dev, D, dtype):
    run(dev, [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 257], 3, D, dtype)


def test_prefill_attention_long_sequence_and_strided_inputs(dev):
    run(dev, [700, 5, 1025], 2, 128, strided=True)
    run(dev, [2048], 1, 64, seed=7)


def test_first_token_sees_only_itself_and_last_matches_decode_definition(dev):
    lens = [40, 90]
    out, ref = run(dev, lens, 4, 64, seed=3)
    v = randn((sum(lens), 4, 64), 5)       # seed + 2
    assert torch.allclose(out[0], v[0].float(), atol=1e-3)
    assert torch.allclose(out[40], v[40].float(), atol=1e-3)


def test_opt13b_prompt_shape(dev):
    """40 heads x 128, three prompts (the widest rows the path sees)."""
    run(dev, [384, 17, 600], 40, 128, seed=11, strided=True)


def test_argument_validation(dev):
    q = torch.zeros(8, 2, 48, dtype=torch.float16, device=dev)
    cu = torch.tensor([0, 8], dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        ops.flash_attn_varlen_func(q, q, q, cu_seqlens_q=cu, max_seqlen_q=8)          # head size 48
    q = torch.zeros(8, 2, 64, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        ops.flash_attn_varlen_func(q, q, q, cu_seqlens_q=cu, max_seqlen_q=8, causal=False)
    with pytest.raises(ValueError):
        ops.flash_attn_varlen_func(q, q, q, cu_seqlens_q=cu.long(), max_seqlen_q=8)
    for bad in (0.0, -0.125, float("nan"), float("inf")):     # the kernel's running maximum assumes a positive scale
        with pytest.raises(ValueError):
            ops.flash_attn_varlen_func(q, q, q, cu_seqlens_q=cu, max_seqlen_q=8, softmax_scale=bad)
    e = torch.zeros(0, 2, 64, dtype=torch.float16, device=dev)
    assert ops.flash_attn_varlen_func(e, e, e, cu_seqlens_q=cu[:1], max_seqlen_q=0).shape == (0, 2, 64)
