"""Host-side pieces of the step-loop harness (CPU)."""
import numpy as np

from aptserve_hip import step_loop


def test_request_stream_and_block_pool():
    reqs = step_loop.synth_requests(0, 200)
    gaps = np.diff([0.0] + [r.arrival for r in reqs])
    assert 0.25 < gaps.mean() < 0.42            # 3 requests per second
    assert all(4 <= len(r.prompt_ids) <= 2048 and len(r.prompt_ids) + r.output_len <= 2048 for r in reqs)
    pool = step_loop.BlockPool(8)
    r = step_loop.Request(0, 0.0, np.zeros(40, dtype=np.int64), 4, True)
    pool.grow(r, 40, 16)
    assert len(r.block_table) == 3 and r.block_table[1] == r.block_table[0] + 8 and r.block_table[2] < 8
    assert len(r.shared_table) == 3 and all(8 <= b < 16 for b in r.shared_table)
    assert pool.blocks_needed(r, 65, 16) == (1, 2)
    pool.release(r)
    assert len(pool.free_private) == 8 and len(pool.free_shared) == 8


def test_cost_coefficient_regression_follows_the_reference_recipe():
    """Times linear in the block count with slope s give s/5; the (0, 0) point and the floor at one block
    are part of the recipe (aptserve_llm_engine.py:336-347)."""
    from aptserve_hip.cost_model import fit_coef
    tokens = list(range(1, 4101, 100))
    blocks = [max(1, t // 16) for t in tokens]
    slope = 3.5e-4
    secs = [slope * b for b in blocks]
    assert abs(fit_coef(tokens, secs, 16) - slope / 5) < 1e-4 * slope
    # an intercept does not change the slope much (ordinary least squares with intercept)
    assert abs(fit_coef(tokens, [s + 1e-3 for s in secs], 16) - slope / 5) < 0.05 * slope / 5


def test_decode_growth_preempts_instead_of_running_out_of_blocks():
    """Before a decode step the loop checks the free lists; when the running sequences need more blocks than are
    free, the most recently admitted ones go back to the queue in recompute mode."""
    reqs = [step_loop.Request(i, 0.0, np.zeros(16, dtype=np.int64), 64, bool(i % 2)) for i in range(4)]
    loop = step_loop.StepLoop(None, None, [], 6, 16, "cpu")
    for r in reqs:                      # 16 prompt tokens: one private (+ one shared) block each
        loop.pool.grow(r, 16, 16)
        r.generated = [1]               # the next step needs token slot 16: a second block for everybody
        loop.running.append(r)
    assert len(loop.pool.free_private) == 2
    loop._make_room()
    # K/V sequences need a private block each, hidden ones a V-plane slab (no new private block) and a shared block
    assert [r.rid for r in loop.running] == [0, 1, 2, 3][:len(loop.running)] and loop.preemptions >= 0
    need = sum(loop.pool.blocks_needed(r, r.seq_len, 16)[0] for r in loop.running)
    assert need <= len(loop.pool.free_private)
    small = step_loop.StepLoop(None, None, [], 5, 16, "cpu")
    kv = [step_loop.Request(i, 0.0, np.zeros(16, dtype=np.int64), 64, False) for i in range(4)]
    for r in kv:
        small.pool.grow(r, 16, 16)
        r.generated = [1]
        small.running.append(r)
    small._make_room()                  # 4 sequences want 4 blocks, 1 is free: the newest ones are preempted
    assert small.preemptions == 2 and [r.rid for r in small.running] == [0, 1]
    assert [r.rid for r in small.waiting] == [2, 3] and all(not r.block_table for r in small.waiting)
    # recompute preemption keeps what was generated (it is re-prefilled with the prompt) and drops the hidden cache
    assert all(r.generated == [1] and r.seq_len == 17 and len(r.token_ids) == 17 for r in small.waiting)


def test_preempted_request_keeps_its_tokens_and_falls_back_to_the_kv_cache():
    """additional_designs/core/aptserve_scheduler.py:2118-2130: the victim of a recompute preemption keeps its
    output tokens, restarts its computed-token count and has use_hidden cleared; its next prompt step covers
    prompt + outputs, so no token is generated (or counted) twice."""
    reqs = [step_loop.Request(i, 0.0, np.arange(16, dtype=np.int64), 64, True) for i in range(3)]
    loop = step_loop.StepLoop(None, None, [], 2, 16, "cpu")     # 2 private + 2 shared blocks
    for r in reqs[:2]:
        loop.pool.grow(r, 16, 16)
        r.generated = [100 + r.rid]
        loop.running.append(r)
    # each hidden sequence now needs a second shared block: none is free, so the newer one is preempted
    loop._make_room()
    assert loop.preemptions == 1 and [r.rid for r in loop.running] == [0]
    v = loop.waiting[0]
    assert v.rid == 1 and v.generated == [101] and v.use_hidden is False and not v.block_table and not v.shared_table
    assert list(v.token_ids) == list(range(16)) + [101]
    # when it is admitted again it is sized on prompt + outputs, as a K/V sequence
    loop.running.clear()
    loop.pool.release(reqs[0])
    loop.pool = step_loop.BlockPool(16)
    batch = loop._admit()
    assert batch == [v] and len(v.block_table) == 2 and not v.shared_table


def test_virtual_clock_is_independent_of_measured_time():
    cost = step_loop.fixed_step_cost()
    assert cost(dict(kind="decode", seqs=5, tokens=5)) == cost(dict(kind="decode", seqs=9, tokens=9))
    assert cost(dict(kind="prefill", seqs=1, tokens=2000)) > cost(dict(kind="prefill", seqs=1, tokens=20))


def test_a_prompt_that_can_never_fit_raises_instead_of_waiting_forever():
    """Nothing runs, the head of the queue has arrived and the empty pool still cannot take it: the loop says so
    (it used to call itself again, with an unchanged clock, until the interpreter's recursion limit)."""
    import pytest
    big = step_loop.Request(0, 0.0, np.zeros(16 * 40, dtype=np.int64), 8, False)
    loop = step_loop.StepLoop(None, None, [big], 24, 16, "cpu")
    with pytest.raises(RuntimeError, match="cannot hold a single sequence"):
        loop.step()
