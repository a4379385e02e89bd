"""The operators allocate nothing of their own, synchronise nothing and launch on the caller's stream, so a decode
layer on fixed metadata can be recorded into a HIP graph.  A graph is replayed several times on new inputs, with
eager work and synchronisations between the replays, and every replay must equal the eager layer on the same
inputs bit for bit (same kernels, same launch parameters)."""
import pytest
import torch

from aptserve_hip import backend, metadata, ops, workloads
from util import randn

pytestmark = pytest.mark.gpu

H, D, BS, N = 12, 64, 16, 96
Hd = H * D


def _weights(seed, dev):
    return [w.to(dev) for w in ((randn((3 * Hd, Hd), seed) * 0.03).half(), (randn((3 * Hd,), seed + 1) * 0.1).half(),
                                (randn((Hd, Hd), seed + 2) * 0.03).half(), (randn((Hd,), seed + 3) * 0.1).half())]


@pytest.mark.parametrize("flow", ["reprojection", "absorbed"])
def test_decode_layer_replays_from_a_graph(dev, flow):
    batch = workloads.small_decode_batch(7, 10, 150, 0.5, N)
    B = len(batch.seq_lens)
    md = metadata.build_from_batch(batch, dev)              # built outside the graph: it uploads host data
    layer = backend.HybridOPTAttention(Hd, H, *_weights(30, dev), absorbed=flow == "absorbed")
    kv0, sh0 = randn((2, N, BS, H, D), 31).to(dev), randn((2, 2 * N, BS, H, D), 32).to(dev)
    inputs = [randn((B, Hd), 40 + i).to(dev) for i in range(4)]

    # eager: the same four steps on caches of its own
    e_kv, e_sh = kv0.clone(), sh0.clone()
    eager = [layer(x, e_kv, e_sh, md).clone() for x in inputs]
    torch.cuda.synchronize()

    g_kv, g_sh = kv0.clone(), sh0.clone()
    static_in = inputs[0].clone()
    side = torch.cuda.Stream()                               # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                            # warm-up on the capture stream: one-time set-up
        layer(static_in, g_kv.clone(), g_sh.clone(), md)     # (kernel attributes, workspaces) happens here
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        static_out = layer(static_in, g_kv, g_sh, md)
    for i, x in enumerate(inputs):
        static_in.copy_(x)
        graph.replay()
        got = static_out.clone()
        # eager work of the program and a synchronisation between the replays
        scratch = ops.linear_nt(x, layer.out_weight, layer.out_bias)
        torch.cuda.synchronize()
        assert torch.equal(got, eager[i]), f"replay {i} differs from the eager layer"
        assert scratch.shape == eager[i].shape
    assert torch.equal(g_kv, e_kv) and torch.equal(g_sh, e_sh)


def test_gather_write_and_attention_replay_from_a_graph(dev):
    """The movers and the paged attention at operator level, the attention through the entry point that takes no
    workspace (its partial results go to the library's static array)."""
    batch = workloads.small_decode_batch(9, 12, 400, 0.5, 4 * N)
    md = metadata.build_from_batch(batch, dev)
    B = len(batch.seq_lens)
    kv = randn((2, 4 * N, BS, H, D), 50).to(dev)
    holder = torch.empty(md.num_tot_tokens, Hd, dtype=torch.float16, device=dev)
    hs = randn((B, Hd), 51).to(dev)
    q = randn((B, H, D), 52).to(dev)
    out = torch.empty_like(q)
    tables = md.private_block_tables
    lens = md.seq_lens_tensor

    def step():
        ops.gather_hidden_rows(holder, hs, kv, md.holder_src, md.slot_mapping, md.hidden_cache_use_input,
                               md.hidden_cache_store_tot)
        ops.paged_decode_attention(q, kv[0], kv[1], tables, lens, D ** -0.5, partition_size=32, out=out,
                                   max_seq_len=max(batch.seq_lens), static_scratch=True)

    step()
    torch.cuda.synchronize()
    want_holder, want_out = holder.clone(), out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    for _ in range(3):
        holder.fill_(7.0)
        out.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(holder, want_holder) and torch.equal(out, want_out)


def test_whole_decode_steps_replay_from_graphs_of_their_shape_class(dev):
    """A two-layer decoder in the serving loop, once issued launch by launch and once with every decode step
    replayed from the HIP graph of its shape class (batch size, hidden-cached sequences, bucketed length): the
    same requests, the same schedule, and hidden states, chosen tokens and caches that are equal bit for bit.
    Graphs are recorded when a shape class first appears and replayed for the steps that follow (new metadata in
    the same buffers, eager prompt steps and synchronisations in between)."""
    from aptserve_hip import graph_step, opt_model, step_loop
    cfg = opt_model.OPTConfig(hidden_size=768, num_attention_heads=12, num_hidden_layers=2, ffn_dim=1024,
                              vocab_size=1000, max_position_embeddings=2048)
    N2, w = 96, opt_model.random_weights(cfg, 0, dev)

    def run(graphed):
        model = opt_model.HybridOPTModel(cfg, w, absorbed=True)
        kv, shared = backend.allocate_caches(cfg.num_hidden_layers, N2, BS, 12, 64, torch.float16, dev)
        reqs = step_loop.synth_requests(3, 7, rate=2000.0, hidden_fraction=0.5, vocab=1000, prompt_mu=3.3,
                                        prompt_sigma=0.6, out_mu=1.6, out_sigma=0.3)
        steps = []
        runner = graph_step.DecodeGraphRunner(model, kv, shared, BS, dev, len_bucket=64) if graphed else None
        loop = step_loop.StepLoop(lambda ids, pos, md: model(ids, pos, kv, shared, md), model.next_tokens, reqs, N2,
                                  BS, dev, max_prompt_tokens=120, decode_runner=runner,
                                  step_cost=step_loop.fixed_step_cost(),   # same schedule in both runs
                                  on_step=lambda s: steps.append((s["is_prompt"], s["hidden"].clone(),
                                                                  list(s["next_tokens"]))))
        loop.run(40)
        torch.cuda.synchronize()
        return steps, kv, runner

    eager, e_kv, _ = run(False)
    graph, g_kv, runner = run(True)
    assert len(eager) == len(graph) and any(not p for p, _, _ in eager)
    for i, ((p0, h0, t0), (p1, h1, t1)) in enumerate(zip(eager, graph)):
        assert p0 == p1 and t0 == t1, f"step {i}: schedule or tokens differ"
        assert torch.equal(h0, h1), f"step {i} ({'prompt' if p0 else 'decode'}) differs from the eager loop"
    for a, b in zip(e_kv, g_kv):
        assert torch.equal(a, b)
    n_decode = sum(1 for p, _, _ in eager if not p)
    replays = sum(r.replays for r in runner.recorded.values())
    assert replays == n_decode and 1 <= runner.captures < n_decode, (runner.captures, n_decode)
