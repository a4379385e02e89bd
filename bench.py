#!/usr/bin/env python3
"""Benchmark of the hybrid-cache hot path on one MI355X.

A "step" is one pass of the per-layer cache traffic of a decode step at OPT-13B
shapes (256 sequences, half of them hidden-cached, lognormal context lengths):
store the new hidden rows, write the new K/V rows, and gather every hidden
context row into the contiguous holder that feeds the K/V re-projection.
``value`` is the algorithmic GB/s of that step with all inputs resident in HBM.
The line also reports decode-attention tokens/s (fp16 and fp8 caches) and, when
built, the re-projection TFLOP/s, each with its own roofline fraction, plus a
CPU baseline of the same step timed on this host's cores with the oracle.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (ROOT, ROOT / "apt-serve_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (seed 0 workloads), scaled by what the
# same counters read for the 1 GiB copy kernel (x2.000 and x1.000); summary in profiles/bench_step_hbm_counters.txt
PMC_TRAFFIC_BYTES = {"step": 1815.1e6, "attention_f16": 1793.3e6, "attention_fp8": 898.3e6,
                     "gemm_T4096": 868.0e6, "gemm_T16384": 2883.0e6}
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16, published


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip attention / re-projection figures")
    ap.add_argument("--extras", default="literal,attention,prefill,metadata,write,ceilings,reproject,layer,step_loop,cost,cpu",
                    help="comma-separated subset of the extra figures to run (step_replay: not in the default list)")
    ap.add_argument("--pmc-calibrate", action="store_true",
                    help="first run the plain copy kernel on 1 GiB three times (known traffic for counter scaling)")
    return ap.parse_args()


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def event_times(torch, fn, n, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in evs]


def attention_figures(torch, ops, workloads, np, dev, seed, fp8):
    """Config 4: 128 sequences, 40x128, 65536-block pool, each block from the workspace with p=0.5."""
    H, D, BS, B, POOL = 40, 128, 16, 128, 65536
    rng = np.random.default_rng(seed)
    lens = workloads.lognormal_lengths(rng, B)
    nblk = [-(-int(l) // BS) for l in lens]
    W = max(nblk)
    ids = rng.permutation(POOL)[:sum(nblk)]
    bt = np.zeros((B, W), dtype=np.int32)
    p = 0
    for b, n in enumerate(nblk):
        bt[b, :n] = ids[p:p + n]
        p += n
    types = (rng.random((B, W)) < 0.5).astype(np.uint8)
    g = torch.Generator(device=dev).manual_seed(seed)

    def pool():
        x = torch.empty(POOL, BS, H, D, dtype=torch.uint8 if fp8 else torch.float16, device=dev)
        for i in range(0, POOL, 8192):
            r = torch.randn(8192, BS, H, D, generator=g, dtype=torch.float32, device=dev)
            x[i:i + 8192] = (torch.clamp(r / 0.04, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
                             if fp8 else r.to(torch.float16))
        return x
    kc, vc, wk, wv = pool(), pool(), pool(), pool()
    q = torch.randn(B, H, D, generator=g, dtype=torch.float32, device=dev).half()
    d_bt, d_ty = torch.from_numpy(bt).to(dev), torch.from_numpy(types).to(dev)
    d_sl = torch.from_numpy(lens.astype(np.int32)).to(dev)
    out = torch.empty_like(q)
    max_len = int(lens.max())
    fn = lambda: ops.paged_decode_attention(q, kc, vc, d_bt, d_sl, D ** -0.5, block_types=d_ty, ws_k_cache=wk,
                                            ws_v_cache=wv, k_scale=0.04, v_scale=0.04, max_seq_len=max_len, out=out)
    ms = median(event_times(torch, fn, 30))
    total = int(lens.sum())
    nbytes = total * 2 * H * D * (1 if fp8 else 2)
    gbs = nbytes / ms / 1e6
    return {"workload": "config4 paged hybrid decode attention, B=128, 40x128, sum(L)=%d, %s cache" %
                        (total, "fp8-e4m3" if fp8 else "fp16"),
            "tokens_per_s": B / (ms * 1e-3), "ms": ms, "algorithmic_bytes": nbytes,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gbs / HBM_PEAK_GBS,
                         "traffic": PMC_TRAFFIC_BYTES["attention_fp8" if fp8 else "attention_f16"] if seed == 0 else None}}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    from aptserve_hip import metadata, ops, workloads

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    H, D, BS = 40, 128, 16
    Hd = H * D

    # ---- workload: BASELINE.json configs[1]
    batch = workloads.decode_batch_opt13b(args.seed)
    md = metadata.build_from_batch(batch, dev, check_totals=True)
    N, B, T = batch.num_blocks, len(batch.seq_lens), md.num_tot_tokens
    n_hidden_rows = md.hidden_cache_use_tot.numel()
    n_hidden_seqs = md.num_hidden_cache_tokens
    n_kv_seqs = B - n_hidden_seqs
    g = torch.Generator(device=dev).manual_seed(args.seed)
    cache = torch.empty(2, N, BS, H, D, dtype=torch.float16, device=dev)
    for i in range(0, N, 4096):
        cache[:, i:i + 4096] = torch.randn(2, min(4096, N - i), BS, H, D, generator=g, device=dev).half()
    hs = torch.randn(B, Hd, generator=g, device=dev).half()
    kv = torch.randn(B, 2 * Hd, generator=g, device=dev).half()
    key, value = (x.view(B, H, D) for x in kv.chunk(2, -1))
    holder = torch.empty(T, Hd, dtype=torch.float16, device=dev)
    kv_seq_idx, new_slots = md.kv_cache_use_input, md.new_token_slot

    write_bytes = n_kv_seqs * 2 * (2 * Hd * 2) + n_hidden_seqs * 2 * (Hd * 2)   # read + write of each new row
    gather_bytes = n_hidden_rows * 2 * (Hd * 2)                                 # read + write of each context row
    step_bytes = write_bytes + gather_bytes

    def step():
        # one launch: new hidden rows -> hidden blocks, new K/V rows of the K/V-cached sequences -> private
        # cache, and the holder of every row that is re-projected
        ops.decode_step_cache_ops(holder, hs, cache, md.holder_src, md.slot_mapping, md.hidden_cache_use_input,
                                  md.hidden_cache_store_tot, key, value, md.kv_cache_use_input, md.new_token_slot)

    if args.pmc_calibrate:
        from aptserve_hip import probes
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            probes.copy_bytes(dst, src)
        torch.cuda.synchronize()
        del src, dst

    # events are created and recorded once before the timed region: creating one costs a runtime call
    span = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    n_launch_timed = max(args.steps, 200)
    launch_events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                     for _ in range(n_launch_timed)]
    for e in (*span, *launch_events[0]):
        e.record()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # ---- the timed region: exactly `steps` steps, nothing but their launches between the two synchronisations
    t0 = time.perf_counter()
    span[0].record()
    for _ in range(args.steps):
        step()
    span[1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    ms_per_step_events = span[0].elapsed_time(span[1]) / args.steps
    step_gbs = step_bytes / (ms_per_step * 1e-3) / 1e9
    # ---- second pass, outside the timed region: every launch between its own pair of HIP events (on the stream
    # the kernel is launched on: torch's current stream is the one ops hands to the library)
    for a, b in launch_events:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    launch_ms = [a.elapsed_time(b) for a, b in launch_events]
    avg_launch_ms = sum(launch_ms) / len(launch_ms)
    # algorithmic bytes of the launch = the step's: every gathered row, stored hidden row and new K/V row read
    # once and written once (the B newest rows that also enter the holder are not counted)
    achieved = step_bytes / avg_launch_ms / 1e6

    result = {
        "metric": "hybrid-cache write/gather GB/s + decode attn tokens/s, OPT-13B shapes, 1 MI355X",
        "value": step_gbs, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: hybrid cache write + hidden-block gather, OPT-13B 40x128, "
                               "decode batch 256 (128 K/V + 128 hidden), lognormal(6.2,0.8) contexts in [16,2048]",
                   "seed": args.seed, "hidden_rows_gathered": n_hidden_rows, "rows_total": T,
                   "step_bytes": step_bytes, "write_bytes": write_bytes, "gather_bytes": gather_bytes,
                   "launches_per_step": 1},
        "ms_per_step_hip_events": ms_per_step_events,
        "timing": "ms_per_step: host clock around the %d steps between two synchronisations; "
                  "ms_per_step_hip_events: one HIP event pair around the same steps on the stream" % args.steps,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": PMC_TRAFFIC_BYTES["step"] if args.seed == 0 else None,
                     "kernel": "row_mover<16,1,DecodeStepOp>",
                     "algorithmic_bytes_per_launch": step_bytes, "avg_launch_ms": avg_launch_ms,
                     "median_launch_ms": median(launch_ms), "launches_timed": len(launch_ms)},
    }

    want = set() if args.no_extras else set(x for x in args.extras.split(",") if x)
    if want:
        extras = {}
        if "literal" in want:
            gather_alg = gather_bytes + n_hidden_seqs * 2 * (Hd * 2)   # without the K/V rows, which it does not move
            # the reference's own operator sequence through the drop-in module (no caller change): hidden_to_cache,
            # torch.zeros holder, index_put of the newest rows, cache_to_hidden over every cached row
            # (additional_designs/model_executor/models/aptserve_opt.py:108-121)
            import mixed_cache_ops

            def literal():
                mixed_cache_ops.hidden_to_cache(hs, cache, md.slot_mapping, md.hidden_cache_use_input,
                                                md.hidden_cache_store_tot)
                h = torch.zeros(T, Hd, dtype=torch.float16, device=dev)
                h[md.hidden_holder_upd] = hs
                mixed_cache_ops.cache_to_hidden(h, cache, md.slot_mapping, md.hidden_cache_use_tot)
            ms_lit = median(event_times(torch, literal, 20))
            extras["gather_literal_dropin_sequence"] = {
                "workload": "same batch: mixed_cache_ops.hidden_to_cache + torch.zeros + index_put + "
                            "mixed_cache_ops.cache_to_hidden (the reference's calls, unchanged)",
                "ms": ms_lit, "algorithmic_bytes": gather_alg,
                "roofline": {"bound": "hbm", "achieved": gather_alg / ms_lit / 1e6, "peak": HBM_PEAK_GBS,
                             "unit": "GB/s", "frac": gather_alg / ms_lit / 1e6 / HBM_PEAK_GBS, "traffic": None},
                "note": "the zero fill writes the holder a second time: 1.5x the HBM traffic of the fused launch"}
        del holder
        for fp8 in ((False, True) if "attention" in want else ()):
            torch.cuda.empty_cache()
            extras["decode_attention_fp8" if fp8 else "decode_attention_f16"] = attention_figures(
                torch, ops, workloads, np, dev, args.seed, fp8)
        # metadata build, GPU vs the list-based host algorithm
        # from packed 0-padded int32 tables (kept up to date by the caller) and from the lists of lists the
        # reference's scheduler hands over; both include the kernel and a final synchronize
        for md_key, packed in (("metadata_build_us", True), ("metadata_build_us_from_lists", False)):
            t = []
            batch.packed_tables()
            for _ in range(20 if "metadata" in want else 0):
                torch.cuda.synchronize()
                a = time.perf_counter()
                metadata.build_from_batch(batch, dev, packed=packed)
                torch.cuda.synchronize()
                t.append((time.perf_counter() - a) * 1e6)
            if t:
                extras[md_key] = median(t)
        if not args.no_cpu and "metadata" in want:
            # the reference's approach to the same metadata: Python lists per cached token, then tensors
            from oracle.metadata import SeqRecord, build_metadata as list_build
            recs = [SeqRecord(False, h, l, l - 1, bt, bts) for l, h, bt, bts in
                    zip(batch.seq_lens, batch.use_hidden, batch.block_tables, batch.block_tables_4_shared)]
            t = []
            for _ in range(3):
                a = time.perf_counter()
                list_build(recs, batch.block_size)
                t.append((time.perf_counter() - a) * 1e6)
            extras["metadata_build_us_cpu_list_algorithm"] = median(t)
        if "write" in want:
            extras["kv_write_prefill_16384"] = write_figures(torch, ops, dev, args.seed)
            extras["kv_write_prefill_16384_block_contiguous"] = write_figures(torch, ops, dev, args.seed, True)
        if "ceilings" in want:
            extras["stream_ceilings"] = stream_ceiling_figures(torch, dev)
            torch.cuda.empty_cache()
        if "prefill" in want:
            extras["prompt_attention_4x2048"] = prompt_attention_figures(torch, ops, dev, args.seed)
        if "reproject" in want:
            extras.update(reproject_figures(torch, ops, dev, args.seed))
            extras["mfma_ceilings"] = mfma_ceiling_figures(torch, dev)   # after the products: it heats the part
        torch.cuda.empty_cache()
        if "layer" in want:
            extras["decode_layer_config2"] = decode_layer_figures(torch, ops, workloads, metadata, dev, args.seed)
            torch.cuda.empty_cache()
        if "step_loop" in want:
            from aptserve_hip import opt_model
            w13 = opt_model.random_weights(opt_model.OPTConfig.opt_13b(), args.seed, dev)
            extras["opt13b_step_loop"] = step_loop_figures(torch, dev, args.seed, weights=w13)
            torch.cuda.empty_cache()
            extras["opt13b_step_loop_absorbed"] = step_loop_figures(torch, dev, args.seed, absorbed=True, weights=w13)
            torch.cuda.empty_cache()
            extras["opt13b_step_loop_reference_sequence"] = step_loop_figures(
                torch, dev, args.seed, weights=w13, reference_sequence=True, profile_steps=0)
            torch.cuda.empty_cache()
            extras["opt13b_step_loop_absorbed_graphs"] = step_loop_figures(
                torch, dev, args.seed, absorbed=True, weights=w13, graph=True, profile_steps=0)
            d_ = extras["opt13b_step_loop_absorbed_graphs"].pop("schedule")
            del w13
            # all flows ran the same schedule (fixed-cost clock): keep no copy, only the comparison
            a_, b_ = extras["opt13b_step_loop"].pop("schedule"), extras["opt13b_step_loop_absorbed"].pop("schedule")
            c_ = extras["opt13b_step_loop_reference_sequence"].pop("schedule")
            extras["opt13b_step_loop_same_schedule"] = a_ == b_ == c_ == d_
        if "step_replay" in want:   # (not in the default list: the kernel split of one decode step, for a profiler)
            extras["opt13b_step_replay"] = step_replay_figures(torch, dev, args.seed)
            torch.cuda.empty_cache()
        if "cost" in want:
            extras["cost_coef"] = cost_coef_figures(torch, dev)
        if not args.no_cpu and "cpu" in want:
            extras["cpu_baselines"] = {
                "config3_kv_reproject_T4096": cpu_baseline_reproject(torch),
                "config4_decode_attention": cpu_baseline_attention(torch, np, workloads, args.seed)}
        result["extras"] = extras

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, np, batch, md, cache, hs, key, value, kv_seq_idx, new_slots,
                                              step_bytes, T, Hd)
    print(json.dumps(result))


def prompt_attention_figures(torch, ops, dev, seed):
    """Causal attention of a prompt step (the flash_attn_varlen_func call of the reference's prompt path) at
    OPT-13B width: 4 prompts of 2048 tokens, packed.  FLOPs counted as the causal half of QK^T and PV."""
    H, D, lens = 40, 128, [2048] * 4
    T = sum(lens)
    g = torch.Generator(device=dev).manual_seed(seed)
    q, k, v = (torch.randn(T, H, D, generator=g, device=dev).half() for _ in range(3))
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    ms = median(event_times(torch, lambda: ops.flash_attn_varlen_func(q, k, v, cu, cu, max(lens), max(lens),
                                                                      causal=True, out=out), 10))
    flops = sum(2 * 2 * L * L * H * D / 2 for L in lens)
    tf = flops / ms / 1e9
    # the same launch on all-zero inputs: the part keeps its clock there, so the difference is what the power the
    # real operands draw costs, and the zero-input time is what the instruction schedule alone would allow
    q.zero_(); k.zero_(); v.zero_()
    for _ in range(20):
        ops.flash_attn_varlen_func(q, k, v, cu, cu, max(lens), max(lens), causal=True, out=out)
    ms0 = median(event_times(torch, lambda: ops.flash_attn_varlen_func(q, k, v, cu, cu, max(lens), max(lens),
                                                                       causal=True, out=out), 10))
    return {"workload": "causal varlen attention, 4 prompts x 2048 tokens, 40 heads x 128, fp16", "ms": ms,
            "tokens_per_s": T / ms * 1e3, "algorithmic_flops": flops,
            "roofline": {"bound": "mfma", "achieved": tf, "peak": 2500.0, "unit": "TFLOP/s", "frac": tf / 2500.0,
                         "traffic": None},
            "ms_on_zero_inputs": ms0, "issue_mix": issue_mix_figures(torch, dev)}


def issue_mix_figures(torch, dev):
    """How a SIMD issues matrix and vector instructions side by side (aps_mfma_probe shapes 2..6, zero operands so
    that the clock stays up; 256 workgroups, a round = 16 v_mfma_f32_32x32x16 and / or 16 x [v_exp_f32 + 3
    v_fma_f32]).  The prompt attention's softmax is vector work of about the size of its matrix work: the two
    overlap when they alternate inside a wavefront's instruction stream and hardly when wavefronts issue them in
    runs, which is how a compiler-scheduled attention loop issues them."""
    from aptserve_hip import probes
    lib = probes.load()
    st = torch.cuda.current_stream().cuda_stream
    sink = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    zeros = torch.zeros(16384, dtype=torch.float16, device=dev)
    iters = 2000
    out = {"workgroups": 256, "iters": iters}
    for shape, name in ((0, "mfma_only_16_accumulators_1_wave_per_simd"), (4, "vector_only_1_wave_per_simd"),
                        (3, "mfma_run_then_vector_run_1_wave_per_simd"), (2, "alternating_1_wave_per_simd"),
                        (6, "mfma_run_then_vector_run_2_waves_per_simd"), (5, "alternating_2_waves_per_simd")):
        out[name + "_ms"] = median(event_times(torch, lambda: lib.aps_mfma_probe(
            shape, 0, zeros.data_ptr(), sink.data_ptr(), 256, iters, st), 8))
    return out


def write_figures(torch, ops, dev, seed, block_contiguous=False):
    """The cache write at a shape that can saturate HBM: a 16 384-token prompt batch at OPT-13B width,
    K and V rows scattered by slot_mapping (the decode-step write of configs[1] moves 7.9 MB and is
    bounded by launch latency, not bandwidth).  Slots: a random permutation of all slots (every 10 KiB row lands
    somewhere else: the worst case), or, `block_contiguous`, what a prompt step produces: consecutive tokens fill
    the 16 slots of a block, blocks in random order."""
    H, D, BS, T = 40, 128, 16, 16384
    N = T // BS + 64
    g = torch.Generator(device=dev).manual_seed(seed)
    kv = torch.randn(T, 2 * H * D, generator=g, device=dev).half()
    key, value = (x.view(T, H, D) for x in kv.chunk(2, -1))
    cache = torch.zeros(2, N, BS, H, D, dtype=torch.float16, device=dev)
    if block_contiguous:
        blocks = torch.randperm(N, generator=g, device=dev)[:T // BS]
        slots = (blocks[:, None] * BS + torch.arange(BS, device=dev)[None, :]).reshape(-1).contiguous()
    else:
        slots = torch.randperm(N * BS, generator=g, device=dev)[:T].contiguous()
    ms = median(event_times(torch, lambda: ops.reshape_and_cache_flash(key, value, cache[0], cache[1], slots, "auto"), 30))
    nbytes = T * 2 * (2 * H * D * 2)
    gbs = nbytes / ms / 1e6
    return {"workload": "K/V cache write of 16384 tokens, 40x128 f16, " +
                        ("slots block by block (a prompt step), blocks in random order" if block_contiguous
                         else "random slots"), "ms": ms,
            "algorithmic_bytes": nbytes,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gbs / HBM_PEAK_GBS, "traffic": None}}


def stream_ceiling_figures(torch, dev):
    """What plain streams sustain on this GPU (aps_stream_probe, 2 GiB of random fp16, one 16-byte chunk per
    thread, workgroups in address order): the ceilings the row movers and the attention are held against."""
    from aptserve_hip import probes
    lib = probes.load()
    nb = 2 << 30
    a = torch.empty(nb // 2, dtype=torch.float16, device=dev)
    for i in range(0, nb // 2, 1 << 28):
        a[i:i + (1 << 28)] = torch.randn(1 << 28, device=dev).half()
    b = torch.empty_like(a)
    st = torch.cuda.current_stream().cuda_stream
    out = {"bytes": nb, "data": "random fp16 N(0,1)"}
    for mode, name, mult in ((0, "copy", 2), (1, "read", 1), (2, "fill", 1)):
        ms = median(event_times(torch, lambda: lib.aps_stream_probe(mode, 1, b.data_ptr(), a.data_ptr(), nb, st), 20))
        out[name] = {"ms": ms, "GB/s": mult * nb / ms / 1e6, "frac_of_hbm_peak": mult * nb / ms / 1e6 / HBM_PEAK_GBS}
    # the same probes at the sizes of the smaller workloads: a launch's ramp-up and tail weigh more there
    small = 16384 * 2 * 5120 * 2       # the K/V write of 16384 tokens: this many bytes read, as many written
    ms = median(event_times(torch, lambda: lib.aps_stream_probe(0, 1, b.data_ptr(), a.data_ptr(), small, st), 20))
    out["copy_of_kv_write_size"] = {"bytes_each_way": small, "ms": ms, "GB/s": 2 * small / ms / 1e6,
                                    "frac_of_hbm_peak": 2 * small / ms / 1e6 / HBM_PEAK_GBS}
    half = 885903360                   # the fp8 cache of config 4 (what its attention reads)
    for name, n in (("read_of_fp8_attention_size", half), ("read_of_f16_attention_size", 2 * half)):
        ms = median(event_times(torch, lambda: lib.aps_stream_probe(1, 1, b.data_ptr(), a.data_ptr(), n, st), 20))
        out[name] = {"bytes": n, "ms": ms, "GB/s": n / ms / 1e6, "frac_of_hbm_peak": n / ms / 1e6 / HBM_PEAK_GBS}
    # the same buffer read again and again: sizes that stay in the 256 MB memory-side cache stream no faster than
    # 2 GiB from HBM, i.e. a second pass over rows that a first pass left in that cache is not a faster pass
    for mib in (64, 128, 256):
        n = mib << 20
        for _ in range(5):
            lib.aps_stream_probe(1, 1, b.data_ptr(), a.data_ptr(), n, st)
        ms = median(event_times(torch, lambda: lib.aps_stream_probe(1, 1, b.data_ptr(), a.data_ptr(), n, st), 20))
        out[f"read_of_{mib}MiB_repeated"] = {"bytes": n, "ms": ms, "GB/s": n / ms / 1e6,
                                             "frac_of_hbm_peak": n / ms / 1e6 / HBM_PEAK_GBS}
    return out


def mfma_ceiling_figures(torch, dev):
    """What the matrix cores sustain with nothing else running (aps_mfma_probe: 256 workgroups of 4 wavefronts,
    operands in registers): under N(0,1) operands the part lowers its clock to stay inside its power limit, and how
    far depends on the instruction shape.  The re-projection GEMM is held against the figure of its own shape."""
    from aptserve_hip import probes
    lib = probes.load()
    st = torch.cuda.current_stream().cuda_stream
    sink = torch.empty(256 * 256, dtype=torch.float32, device=dev)
    iters = 3200
    flops = 256 * 4 * iters * 2 * 16 * 32 * 32 * 16
    out = {"workgroups": 256, "iters": iters, "flops": flops}
    g = torch.Generator(device=dev).manual_seed(0)
    for data, ops_ in (("random_N01", torch.randn(16384, generator=g, device=dev).half()),
                       ("zeros", torch.zeros(16384, dtype=torch.float16, device=dev))):
        for shape, name in ((0, "32x32x16"), (1, "16x16x32")):
            ms = median(event_times(torch, lambda: lib.aps_mfma_probe(shape, 0, ops_.data_ptr(), sink.data_ptr(), 256,
                                                                        iters, st), 12))
            out[f"f16_{name}_{data}"] = {"ms": ms, "tflops": flops / ms / 1e9,
                                          "frac_of_mfma_peak": flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS}
    return out


def step_replay_figures(torch, dev, seed, seq_lens=(310, 120, 200, 260, 130), use_hidden=(1, 0, 1, 0, 1), reps=26):
    """One OPT-13B decode step of a fixed small batch (absorbed flow), recorded into a HIP graph once and replayed:
    under ``rocprofv3 --kernel-trace`` the kernels of the replays run back to back, so their durations add up to the
    step and give its split by kernel."""
    from aptserve_hip import backend, graph_step, opt_model
    cfg = opt_model.OPTConfig.opt_13b()
    model = opt_model.HybridOPTModel(cfg, opt_model.random_weights(cfg, seed, dev), absorbed=True)
    BS = 16
    kv, shared = backend.allocate_caches(cfg.num_hidden_layers, 2048, BS, cfg.num_attention_heads,
                                         cfg.hidden_size // cfg.num_attention_heads, torch.float16, dev)
    for c in kv:
        c.normal_(0, 0.3)
    tables, shared_tables, nxt = [], [], 0
    for n, h in zip([-(-l // BS) for l in seq_lens], use_hidden):
        tables.append(list(range(nxt, nxt + n))); nxt += n
        shared_tables.append(list(range(nxt, nxt + n)) if h else []); nxt += n if h else 0
    runner = graph_step.DecodeGraphRunner(model, kv, shared, BS, dev)
    ids = torch.randint(0, cfg.vocab_size, (len(seq_lens),), device=dev)
    rec = runner.prepare(list(seq_lens), [bool(h) for h in use_hidden], tables, shared_tables, ids)
    torch.cuda.synchronize()
    for _ in range(5):
        runner.run(rec)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        runner.run(rec)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / reps * 1e3
    # the same step eagerly with GPU event timers around the phases of every layer (their synchronisations serialise
    # the step: a split, not a step time)
    per = {}
    for _ in range(3):
        with backend.PhaseTimes() as pt:
            model(rec.ids, rec.md.input_positions, kv, shared, rec.md)
        for k_, v_ in pt.totals().items():
            per[k_] = per.get(k_, 0.0) + v_ / 3
    L = cfg.num_hidden_layers
    return {"workload": f"OPT-13B 40 layers fp16 random-init, decode batch of {len(seq_lens)} sequences "
                        f"({sum(bool(h) for h in use_hidden)} hidden-cached with "
                        f"{sum(l for l, h in zip(seq_lens, use_hidden) if h)} cached rows), one HIP graph replayed",
            "replays": reps, "ms_per_step": ms,
            "eager_phase_us_per_layer": {k_: v_ * 1e3 / L for k_, v_ in per.items()},
            "note": "attention_on_hidden_rows = the one call for both kinds of sequence (stores, K/V attention, "
                    "attention on hidden rows with its value projection); projections = qkv, out, fc1, fc2"}


def step_loop_figures(torch, dev, seed, warm_steps=240, timed_steps=320, profile_steps=12, absorbed=False,
                      weights=None, reference_sequence=False, graph=False):
    """BASELINE configs[4]: OPT-13B (random-init fp16, 40 layers) serving steps on the hybrid cache with
    synthetic arrivals (3 req/s, CV 1) and lognormal prompt/output lengths; half of the requests hidden-cached.
    The simulated clock runs on a fixed cost per step, so every data flow sees the same arrivals, admissions and
    batches; the first `warm_steps` steps (the start-up transient: ~3 s of simulated time) are not counted.
    Afterwards `profile_steps` decode steps run with per-phase GPU timers for the split of a step."""
    from aptserve_hip import backend, opt_model, step_loop
    cfg = opt_model.OPTConfig.opt_13b()
    N, BS = 6144, 16
    Hd, L = cfg.hidden_size, cfg.num_hidden_layers
    w = weights if weights is not None else opt_model.random_weights(cfg, seed, dev)
    # reference_sequence: the reference's own operator calls, one for one (hidden_to_cache, zero-filled holder,
    # index_put, cache_to_hidden, kv-only projection, chunk, mixed_kv_to_cache with the mirror writes, attention of
    # every sequence over the shared cache: aptserve_opt.py:108-124, aptserve_flash_attn.py:359-373,464-473)
    flow_kw = dict(literal=True, fused=False) if reference_sequence else dict(absorbed=absorbed)
    model = opt_model.HybridOPTModel(cfg, w, **flow_kw)
    kv, shared = backend.allocate_caches(cfg.num_hidden_layers, N, BS, cfg.num_attention_heads,
                                         cfg.hidden_size // cfg.num_attention_heads, torch.float16, dev)
    reqs = step_loop.synth_requests(seed, 96, rate=3.0, cv=1.0, hidden_fraction=0.5)
    seq_len_sum = []

    def on_step(info):
        seq_len_sum.append((sum(info["seq_lens"]), sum(l for l, h in zip(info["seq_lens"], info["use_hidden"]) if h)))
    runner = None
    if graph:      # decode steps replayed from one HIP graph per shape class (absorbed flow only)
        from aptserve_hip import graph_step
        runner = graph_step.DecodeGraphRunner(model, kv, shared, BS, dev, max_graphs=96)
    loop = step_loop.StepLoop(lambda ids, pos, md: model(ids, pos, kv, shared, md), model.next_tokens, reqs, N, BS, dev,
                              step_cost=step_loop.fixed_step_cost(), on_step=on_step, decode_runner=runner)
    loop.run(warm_steps)
    log = loop.run(warm_steps + timed_steps)[warm_steps:]
    dec_all = [e for e in log if e["kind"] == "decode"]
    dec = [e for e in dec_all if not e.get("recorded")]      # steps that recorded a graph ran twice: counted apart
    pre = [e for e in log if e["kind"] == "prefill"]
    mean = lambda xs: sum(xs) / len(xs) if xs else None
    # ---- split of a decode step: per-phase GPU time and what each phase achieves
    phases, host = {}, {"metadata_ms": 0.0, "model_ms": 0.0}
    work = {"gather_bytes": 0.0, "gemm_flops": 0.0, "attention_bytes": 0.0, "hidden_attention_bytes": 0.0}
    n_prof = 0
    while n_prof < profile_steps:
        n_before = len(seq_len_sum)
        with backend.PhaseTimes() as pt:
            e = loop.step()
        if e is None:
            break
        if e["kind"] != "decode":
            continue
        tot = pt.totals()
        for k_, v_ in tot.items():
            phases[k_] = phases.get(k_, 0.0) + v_
        host["metadata_ms"] += e["metadata_ms"]
        host["model_ms"] += e["model_ms"]
        all_len, hidden_len = seq_len_sum[n_before]
        kv_len = all_len - hidden_len
        if absorbed:
            work["attention_bytes"] += L * kv_len * 2 * Hd * 2
            work["hidden_attention_bytes"] += L * 2 * hidden_len * Hd * 2
        else:
            work["gather_bytes"] += L * hidden_len * 2 * Hd * 2
            work["gemm_flops"] += L * 2.0 * e["rows"] * Hd * 2 * Hd
            work["attention_bytes"] += L * all_len * 2 * Hd * 2
        n_prof += 1
    split = None
    if n_prof:
        per = {k_: v_ / n_prof for k_, v_ in phases.items()}
        model_ms = host["model_ms"] / n_prof
        split = {"steps_profiled": n_prof, "metadata_ms": host["metadata_ms"] / n_prof, "model_ms": model_ms,
                 "gpu_ms": per, "rest_ms": model_ms - sum(per.values()),
                 "note": "projections = q / out / MLP products (weight streaming); rest = layer norms, residual "
                         "adds, embedding, logits, launch gaps"}
        frac = {}
        if per.get("gather"):
            frac["gather_hbm"] = work["gather_bytes"] / n_prof / per["gather"] / 1e6 / HBM_PEAK_GBS
        if per.get("kv_gemm"):
            frac["kv_gemm_mfma"] = work["gemm_flops"] / n_prof / per["kv_gemm"] / 1e9 / MFMA_F16_PEAK_TFLOPS
        if per.get("attention"):
            frac["attention_hbm"] = work["attention_bytes"] / n_prof / per["attention"] / 1e6 / HBM_PEAK_GBS
        if per.get("attention_on_hidden_rows"):
            # (one call attends both kinds of sequence: the K/V rows of the K/V-cached ones count here when
            # no phase of their own was timed)
            both = work["hidden_attention_bytes"] + (0 if per.get("attention") else work["attention_bytes"])
            frac["attention_on_hidden_rows_hbm"] = (both / n_prof / per["attention_on_hidden_rows"] / 1e6 /
                                                    HBM_PEAK_GBS)
        if per.get("projections"):
            stream = L * (10 if not absorbed else 12) * Hd * Hd * 2      # q, out, fc1, fc2 (and k, v when projected whole)
            frac["projections_hbm"] = stream / per["projections"] / 1e6 / HBM_PEAK_GBS
        split["achieved_fraction_of_peak"] = frac
    return {"workload": "OPT-13B 40 layers fp16 random-init, eager; gamma arrivals 3 req/s cv 1; prompts "
                        "lognormal(5.5,1.0) in [4,2048]; outputs lognormal(5.0,0.9) in [4,1024]; 50% hidden-cached; "
                        "simulated clock on a fixed cost per step (12.5 ms decode, 10 ms + 20 us/token prompt); "
                        + ("decode steps replayed from one HIP graph per shape class; " if graph else "")
                        + ("the reference's operator sequence, call for call, on this library's kernels"
                           if reference_sequence else
                           "hidden-cached sequences attend on their hidden rows (absorbed projections)" if absorbed
                           else "hidden-cached sequences are re-projected every layer (the reference's data flow, "
                                "fused: in-place A rows, cache write in the GEMM epilogue, per-block source select)"),
            "warm_steps": warm_steps, "steps": len(log), "decode_steps": len(dec), "prefill_steps": len(pre),
            "schedule": [(e["kind"][0], e["seqs"], e["rows"]) for e in log],
            "preemptions": loop.preemptions,
            "decode_steps_that_recorded_a_graph": len(dec_all) - len(dec),
            "decode_ms_per_recording_step": mean([e["model_ms"] + e["metadata_ms"] for e in dec_all if e.get("recorded")]),
            "decode_ms_per_step": mean([e["model_ms"] for e in dec]),
            "decode_seqs_per_step": mean([e["seqs"] for e in dec]),
            "decode_rows_per_step": mean([e["rows"] for e in dec]),
            "prefill_ms_per_step": mean([e["model_ms"] for e in pre]),
            "prefill_tokens_per_step": mean([e["tokens"] for e in pre]),
            "metadata_ms_per_step": mean([e["metadata_ms"] for e in log]),
            "decode_host_enqueue_ms_per_step": mean([e["host_enqueue_ms"] for e in dec]),
            "decode_tokens_per_s": (sum(e["seqs"] for e in dec) / (sum(e["model_ms"] + e["metadata_ms"] for e in dec) * 1e-3)
                                    if dec else None),
            "decode_step_split": split}


def decode_layer_figures(torch, ops, workloads, metadata, dev, seed):
    """One decoder self-attention layer of the configs[1] decode batch (256 sequences, half of them
    hidden-cached, ~87.6 k cached hidden rows) in the two data flows: re-projection of every cached row
    (gather, K/V GEMM into the workspace, attention) and attention on the hidden rows themselves."""
    from aptserve_hip import backend
    H, D, BS = 40, 128, 16
    Hd = H * D
    batch = workloads.decode_batch_opt13b(seed)
    N = batch.num_blocks
    md = metadata.build_from_batch(batch, dev)
    g = torch.Generator(device=dev).manual_seed(seed)
    kv = torch.empty(2, N, BS, H, D, dtype=torch.float16, device=dev)
    for i in range(0, N, 4096):
        kv[:, i:i + 4096] = torch.randn(2, min(4096, N - i), BS, H, D, generator=g, device=dev).half()
    shared = torch.zeros(2, 2 * N, BS, H, D, dtype=torch.float16, device=dev)
    qkv_w = (torch.randn(3 * Hd, Hd, generator=g, device=dev) * 0.02).half()
    qkv_b = (torch.randn(3 * Hd, generator=g, device=dev) * 0.02).half()
    out_w = (torch.randn(Hd, Hd, generator=g, device=dev) * 0.02).half()
    out_b = (torch.randn(Hd, generator=g, device=dev) * 0.02).half()
    hs = torch.randn(len(batch.seq_lens), Hd, generator=g, device=dev).half()
    res = {"workload": "decoder self-attention layer, OPT-13B 40x128, decode batch 256 (128 K/V + 128 hidden), "
                       "%d cached hidden rows" % int(md.hidden_slots.numel())}
    outs = {}
    # reference_sequence: the reference's operator calls one for one on this library's kernels (zero-filled
    # holder, index_put, cache_to_hidden, kv-only projection, chunk, mixed_kv_to_cache with the mirror writes)
    for name, kw in (("reprojection_ms", dict()), ("absorbed_ms", dict(absorbed=True)),
                     ("reference_sequence_ms", dict(literal=True, fused=False))):
        layer = backend.HybridOPTAttention(Hd, H, qkv_w, qkv_b, out_w, out_b, **kw)
        outs[name] = layer(hs, kv, shared, md)
        res[name] = median(event_times(torch, lambda: layer(hs, kv, shared, md), 10))
        if name == "reference_sequence_ms":
            del outs[name]
            torch.cuda.empty_cache()
    res["max_abs_difference"] = (outs["reprojection_ms"].float() - outs["absorbed_ms"].float()).abs().max().item()
    res["speedup"] = res["reprojection_ms"] / res["absorbed_ms"]
    res["reference_sequence_over_reprojection"] = res["reference_sequence_ms"] / res["reprojection_ms"]
    # the attention on hidden rows alone (query image, scores, softmax, weighted sum, value projection)
    q = torch.randn(len(batch.seq_lens), Hd, generator=g, device=dev).half()
    out = torch.empty_like(q)
    w_k, w_v, b_v = qkv_w[Hd:2 * Hd], qkv_w[2 * Hd:], qkv_b[2 * Hd:]
    ws = torch.empty(ops._lib.load().aps_absorbed_attention_workspace_bytes(
        int(md.hidden_cache_use_input.numel()), md.max_hidden_seq_len, H, D), dtype=torch.uint8, device=dev)
    ms = median(event_times(torch, lambda: ops.absorbed_hidden_attention(
        q, kv, md.hidden_slots, md.hidden_seq_start, md.hidden_cache_use_input, md.max_hidden_seq_len, w_k, w_v, b_v,
        D ** -0.5, out, workspace=ws), 10))
    rows = int(md.hidden_slots.numel())
    alg = 2 * rows * Hd * 2          # every cached hidden row is read twice (scores, weighted sum)
    res["absorbed_attention"] = {
        "ms": ms, "hidden_rows": rows, "algorithmic_bytes": alg,
        "roofline": {"bound": "hbm", "achieved": alg / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg / ms / 1e6 / HBM_PEAK_GBS, "traffic": None}}
    return res


def reproject_figures(torch, ops, dev, seed):
    out = {}
    Hd = 5120
    g = torch.Generator(device=dev).manual_seed(seed)
    w = (torch.randn(2 * Hd, Hd, generator=g, device=dev) * 0.02).half()
    bias = torch.randn(2 * Hd, generator=g, device=dev).half()
    for T in (4096, 16384):
        x = torch.randn(T, Hd, generator=g, device=dev).half()
        y = torch.empty(T, 2 * Hd, dtype=torch.float16, device=dev)
        # ~25 ms of the product itself before the timed launches: coming from lighter work the part needs that
        # long to settle at the clock it sustains under matrix load (T=4096 timed cold reads 15 % slower)
        warm = 64 if T == 4096 else 20
        ms = median(event_times(torch, lambda: ops.kv_reproject(x, w, bias, out=y), 20, warm=warm))
        flops = 2.0 * T * Hd * 2 * Hd
        tf = flops / ms / 1e9
        out["kv_reproject_T%d" % T] = {
            "workload": "config3 [T,5120]x[5120,10240] f16, f32 accumulate, T=%d, %d warm-up launches" % (T, warm),
            "ms": ms, "tflops": tf,
            "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": tf / MFMA_F16_PEAK_TFLOPS,
                         "traffic": PMC_TRAFFIC_BYTES["gemm_T%d" % T] if seed == 0 else None}}
        # the vendor BLAS on the same product (what the reference's F.linear call runs on this GPU), as a
        # stated comparison: same operands, same event timing
        ms_blas = median(event_times(torch, lambda: torch.nn.functional.linear(x, w, bias), 20, warm=warm))
        out["kv_reproject_T%d" % T]["vendor_blas_F_linear"] = {
            "ms": ms_blas, "tflops": flops / ms_blas / 1e9, "frac_of_mfma_peak": flops / ms_blas / 1e9 / MFMA_F16_PEAK_TFLOPS,
            "kernel_over_vendor": ms_blas / ms}
        # the same launch as a serving step meets it: after ~10 ms of lighter, memory-bound work (a stream of copies)
        # instead of after itself; one launch timed per repetition, both kernels
        light_src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        light_dst = torch.empty_like(light_src)

        def after_light_work(fn):
            ts = []
            for _ in range(7):
                for _ in range(100):
                    light_dst.copy_(light_src)
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                fn()
                b.record()
                torch.cuda.synchronize()
                ts.append(a.elapsed_time(b))
            return median(ts)
        cold = after_light_work(lambda: ops.kv_reproject(x, w, bias, out=y))
        cold_blas = after_light_work(lambda: torch.nn.functional.linear(x, w, bias))
        del light_src, light_dst
        out["kv_reproject_T%d" % T]["after_light_work"] = {
            "note": "one launch timed right after ~10 ms of copy kernels (no warm-up launches of the product), median of 7",
            "ms": cold, "frac_of_mfma_peak": flops / cold / 1e9 / MFMA_F16_PEAK_TFLOPS,
            "vendor_ms": cold_blas, "kernel_over_vendor": cold_blas / cold}
        if T == 16384 and hasattr(ops, "kv_reproject_to_cache"):
            # same product, rows written straight to random slots of [blocks,16,40,128] K and V caches
            nblk = 2 * T // 16
            caches = [torch.empty(nblk, 16, 40, 128, dtype=torch.float16, device=dev) for _ in range(2)]
            dest = torch.randperm(nblk * 16, generator=g, device=dev)[:T].contiguous()
            ms2 = median(event_times(
                torch, lambda: ops.kv_reproject_to_cache(x, w, bias, caches[0], caches[1], None, None, dest), 20))
            out["kv_reproject_to_cache_T%d" % T] = {
                "workload": "config3 with the cache write in the epilogue (random slots), T=%d" % T, "ms": ms2,
                "tflops": flops / ms2 / 1e9,
                "roofline": {"bound": "mfma", "achieved": flops / ms2 / 1e9, "peak": MFMA_F16_PEAK_TFLOPS,
                             "unit": "TFLOP/s", "frac": flops / ms2 / 1e9 / MFMA_F16_PEAK_TFLOPS, "traffic": None}}
            del caches
    return out


def cost_coef_figures(torch, dev):
    """The scheduler's profit coefficient (additional_designs/engine/aptserve_llm_engine.py:316-354: 40 layers of
    the QKV product timed over growing token counts, slope over 16-token blocks / 5) at OPT-13B shape, measured
    on this library's two data flows and with the reference's own recipe (F.linear, whose operands the reference
    creates in fp32; fp16 beside it), on the reference's own sampling range(1, 4101, 100)."""
    from aptserve_hip import cost_model
    counts = tuple(range(1, 4101, 100))
    out = {"token_counts": list(counts), "layers": 40, "block_size": 16, "unit": "seconds per block / 5"}
    for name, kw in (("reprojection", dict(mode="reprojection")), ("absorbed", dict(mode="absorbed")),
                     ("reference_recipe_F_linear_fp16", dict(mode="reference_recipe")),
                     ("reference_recipe_F_linear_fp32", dict(mode="reference_recipe", dtype=torch.float32))):
        c, st = cost_model.get_coef(5120, 40, 40, 16, dev, token_counts=counts, **kw)
        out[name] = c
        out[name + "_seconds_at_%d_tokens" % counts[-1]] = st[-1][1]
    out["reprojection_over_recipe_fp16"] = out["reprojection"] / out["reference_recipe_F_linear_fp16"]
    out["reprojection_over_recipe_fp32"] = out["reprojection"] / out["reference_recipe_F_linear_fp32"]
    return out


def cpu_baseline_reproject(torch):
    """BASELINE configs[2] on the host cores: F.linear in fp32 on fp16-rounded operands, T = 4096."""
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    Hd, T = 5120, 4096
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, Hd, generator=g).half().float()
    w = (torch.randn(2 * Hd, Hd, generator=g) * 0.02).half().float()
    b = torch.randn(2 * Hd, generator=g).half().float()
    ts = []
    for i in range(4):
        a = time.perf_counter()
        torch.nn.functional.linear(x, w, b)
        if i >= 1:
            ts.append(time.perf_counter() - a)
    s = median(ts)
    return {"value": 2.0 * T * Hd * 2 * Hd / s / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": threads,
            "sample": "the whole T=4096 product in fp32 (torch CPU F.linear), 1 warm-up, median of 3, %.3f s" % s}


def cpu_baseline_attention(torch, np, workloads, seed, n_seqs=16):
    """BASELINE configs[3] on the host cores with the oracle (per-sequence fp32 softmax over K/V materialised
    through the block table), on the first `n_seqs` sequences of the batch and a pool that holds only their
    blocks."""
    from oracle import attention as OA
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    H, D, BS, B = 40, 128, 16, 128
    rng = np.random.default_rng(seed)
    lens = workloads.lognormal_lengths(rng, B)[:n_seqs]
    nblk = [-(-int(l) // BS) for l in lens]
    W, total = max(nblk), sum(nblk)
    bt = np.zeros((n_seqs, W), dtype=np.int32)
    p = 0
    for b_, n in enumerate(nblk):
        bt[b_, :n] = np.arange(p, p + n)
        p += n
    types = (rng.random((n_seqs, W)) < 0.5).astype(np.uint8)
    g = torch.Generator().manual_seed(seed)
    kc, vc, wk, wv = (torch.randn(total, BS, H, D, generator=g).half() for _ in range(4))
    q = torch.randn(n_seqs, H, D, generator=g).half()
    sl = torch.from_numpy(lens.astype(np.int32))
    ts = []
    for i in range(3):
        a = time.perf_counter()
        OA.paged_decode_attention(q, kc, vc, torch.from_numpy(bt), sl, D ** -0.5, block_types=torch.from_numpy(types),
                                  ws_k_cache=wk, ws_v_cache=wv)
        if i >= 1:
            ts.append(time.perf_counter() - a)
    s = median(ts)
    return {"value": n_seqs / s, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "host_cpus": threads,
            "sample": "first %d of the 128 sequences (sum of lengths %d), fp16 cache, hybrid block types, 1 warm-up, "
                      "median of 2, %.3f s" % (n_seqs, int(lens.sum()), s)}


def cpu_baseline(torch, np, batch, md, cache, hs, key, value, kv_seq_idx, new_slots, step_bytes, T, Hd):
    """The same step with the oracle (PyTorch-CPU index_put_/index_select) on this host's cores."""
    from oracle import cache_ops as OC
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    c_cache, c_hs = cache.cpu(), hs.cpu()
    c_key, c_val = key.cpu(), value.cpu()
    idx = {k: getattr(md, k).cpu() for k in ("slot_mapping", "hidden_holder_upd", "hidden_cache_use_tot",
                                             "hidden_cache_use_input", "hidden_cache_store_tot")}
    c_seq, c_slots = kv_seq_idx.cpu(), new_slots.cpu()[kv_seq_idx.cpu()]

    def step():
        OC.reshape_and_cache_flash(c_key[c_seq], c_val[c_seq], c_cache[0], c_cache[1], c_slots, "auto")
        OC.hidden_to_cache(c_hs, c_cache, idx["slot_mapping"], idx["hidden_cache_use_input"],
                           idx["hidden_cache_store_tot"])
        return OC.assemble_hidden_holder(c_hs, c_cache, idx["slot_mapping"], T, idx["hidden_holder_upd"],
                                         idx["hidden_cache_use_tot"])
    ts = []
    for i in range(7):
        a = time.perf_counter()
        step()
        if i >= 2:
            ts.append(time.perf_counter() - a)
    s = median(ts)
    return {"value": step_bytes / s / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "host_cpus": threads,
            "sample": "the full configs[1] step (same batch, seed and bytes as the GPU leg), 2 warm-ups, "
                      "median of 5 runs, %.3f s per step" % s}


if __name__ == "__main__":
    main()
