"""The serving step loop (BASELINE configs[4] scaled down): every step the GPU builds the ragged
metadata and runs the decoder stack on the hybrid cache; the same steps are replayed through the
CPU oracle (teacher-forced with the GPU's token ids) and compared step by step."""
import numpy as np
import pytest
import torch

from aptserve_hip import backend, opt_model, step_loop
from oracle import model as OM
from oracle.metadata import SeqRecord, build_metadata

pytestmark = pytest.mark.gpu

META = ["slot_mapping", "slot_mapping_shared", "hidden_cache_use_tot", "kv_cache_use_tot", "hidden_cache_use_input",
        "hidden_cache_store_tot", "hidden_holder_upd", "hidden_holder_pull", "seq_lens_tensor", "seq_start_loc",
        "query_start_loc", "context_lens_tensor", "block_tables", "input_positions"]


@pytest.mark.parametrize("absorbed", [False, True])
def test_step_loop_matches_oracle_replay(dev, absorbed):
    cfg = opt_model.OPTConfig(hidden_size=768, num_attention_heads=12, num_hidden_layers=2, ffn_dim=1024,
                              vocab_size=1000, max_position_embeddings=2048)
    N, BS = 96, 16
    w = opt_model.random_weights(cfg, 0, dev)
    model = opt_model.HybridOPTModel(cfg, w, absorbed=absorbed)
    kv, shared = backend.allocate_caches(cfg.num_hidden_layers, N, BS, 12, 64, torch.float16, dev)
    reqs = step_loop.synth_requests(3, 7, rate=2000.0, hidden_fraction=0.5, vocab=1000, prompt_mu=3.3,
                                    prompt_sigma=0.6, out_mu=1.6, out_sigma=0.3)
    assert any(r.use_hidden for r in reqs) and not all(r.use_hidden for r in reqs)
    steps = []
    loop = step_loop.StepLoop(lambda ids, pos, md: model(ids, pos, kv, shared, md), model.next_tokens, reqs, N, BS,
                              dev, max_prompt_tokens=120, on_step=lambda s: steps.append(
                                  {k: (v.float().cpu() if k == "hidden" else v) for k, v in s.items()}))
    log = loop.run(40)
    kinds = [e["kind"] for e in log]
    assert "prefill" in kinds and "decode" in kinds and len(loop.finished) >= 3
    assert any(e["kind"] == "decode" and 0 < e["hidden_seqs"] < e["seqs"] for e in log), "no mixed decode batch"

    # ---- replay on the CPU
    cw = {k: v.cpu() for k, v in w.items()}
    ckv = [torch.zeros(2, N, BS, 12, 64, dtype=torch.float16) for _ in range(cfg.num_hidden_layers)]
    csh = torch.zeros(2, 2 * N, BS, 12, 64, dtype=torch.float16)
    worst = 0.0
    for s in steps:
        recs = [SeqRecord(s["is_prompt"], h, l, 0 if s["is_prompt"] else l - 1, bt, bts)
                for l, h, bt, bts in zip(s["seq_lens"], s["use_hidden"], s["block_tables"], s["shared_tables"])]
        md = build_metadata(recs, BS)
        for f in META:       # metadata built on the GPU for this step, bit-exact
            assert np.array_equal(getattr(s["md"], f).cpu().numpy(), md[f]), f
        ref = OM.decoder_forward(cw, cfg.num_hidden_layers, 12, torch.from_numpy(s["input_ids"]),
                                 torch.from_numpy(md["input_positions"]), ckv, csh, md).float()
        err = (s["hidden"] - ref).abs()
        worst = max(worst, err.max().item())
        assert err.max().item() < 4e-2 and err.mean().item() < 4e-3, (err.max().item(), err.mean().item())
    # persistent caches agree after the whole run
    for a, b in zip(kv, ckv):
        assert torch.allclose(a.float().cpu(), b.float(), atol=2e-2, rtol=2e-2)
    print(f"{len(steps)} steps replayed, worst abs error {worst:.3e}")
