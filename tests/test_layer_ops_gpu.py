"""Residual add + LayerNorm in one launch against the two-operator definition (add in the activation dtype, then
LayerNorm with fp32 statistics): the pair ``hidden_states = residual + hidden_states`` / ``nn.LayerNorm`` of
additional_designs/model_executor/models/aptserve_opt.py:186-211.  The sum must be bit-exact (one rounding of an
exact fp32 sum); the normalised rows may differ from the fp32 oracle by the final rounding."""
import pytest
import torch
import torch.nn.functional as F

from aptserve_hip import ops
from util import randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 8), (5, 768), (7, 5120), (256, 5120), (3, 16384), (2, 1000)])
def test_add_layer_norm_matches_the_two_operator_definition(dev, dtype, rows, width):
    x, r = randn((rows, width), 1, dtype), (randn((rows, width), 2) * 3).to(dtype)
    w, b = (1 + 0.1 * randn((width,), 3)).to(dtype), (0.1 * randn((width,), 4)).to(dtype)
    s_ref = (x.float() + r.float()).to(dtype)
    n_ref = F.layer_norm(s_ref.float(), (width,), w.float(), b.float(), 1e-5)
    normed, s = ops.add_layer_norm(x.to(dev), r.to(dev), w.to(dev), b.to(dev))
    assert torch.equal(s.cpu().view(torch.int16), s_ref.view(torch.int16))
    ulp = 2 ** -10 if dtype == torch.float16 else 2 ** -7
    d = (normed.float().cpu() - n_ref).abs()
    assert (d <= ulp * n_ref.abs() + 1e-3).all(), d.max().item()
    # without a residual: the norm of x, and x itself comes back as the sum
    n2, s2 = ops.add_layer_norm(x.to(dev), None, w.to(dev), None)
    assert s2.data_ptr() == s2.data_ptr() and torch.equal(s2.cpu(), x)
    d2 = (n2.float().cpu() - F.layer_norm(x.float(), (width,), w.float(), None, 1e-5)).abs()
    assert d2.max().item() <= 4 * ulp + 1e-3


def test_add_layer_norm_strided_rows_and_errors(dev):
    wide = randn((6, 2 * 768), 5).to(dev)
    x, r = wide[:, :768], wide[:, 768:]                     # column slices: row stride twice the width
    w, b = torch.ones(768, dtype=torch.float16, device=dev), torch.zeros(768, dtype=torch.float16, device=dev)
    normed, s = ops.add_layer_norm(x, r, w, b)
    s_ref = (x.float() + r.float()).half()
    assert torch.equal(s, s_ref)
    assert torch.allclose(normed.float(), F.layer_norm(s_ref.float(), (768,)), atol=2e-3, rtol=2e-3)
    with pytest.raises(RuntimeError):
        ops.add_layer_norm(randn((2, 12), 1).to(dev), None, torch.ones(12, dtype=torch.float16, device=dev), None)
    with pytest.raises(ValueError):
        ops.add_layer_norm(x, r.float(), w, b)
    assert ops.add_layer_norm(x[:0], r[:0], w, b)[0].shape == (0, 768)


def test_decoder_with_fused_norms_equals_plain_ops(dev):
    """Two decoder layers with the (add, LayerNorm) pairs fused against the same model on plain element-wise ops:
    same kernels everywhere else, so the hidden states agree to the norms' last-bit differences."""
    from aptserve_hip import backend, metadata, opt_model, workloads
    cfg = opt_model.OPTConfig(hidden_size=768, num_attention_heads=12, num_hidden_layers=2, ffn_dim=1024,
                              vocab_size=500, max_position_embeddings=2048)
    w = opt_model.random_weights(cfg, 0, dev)
    N, BS = 96, 16
    batch = workloads.small_decode_batch(5, 9, 100, 0.5, N)
    md = metadata.build_from_batch(batch, dev)
    ids = torch.arange(len(batch.seq_lens), device=dev) % 500
    outs = []
    for fused in (True, False):
        kv, shared = backend.allocate_caches(2, N, BS, 12, 64, torch.float16, dev)
        for c in kv:
            c.copy_(randn(tuple(c.shape), 9).to(dev))
        model = opt_model.HybridOPTModel(cfg, w, fused_norm=fused)
        outs.append(model(ids, md.input_positions, kv, shared, md).float())
    assert (outs[0] - outs[1]).abs().max().item() < 2e-2
