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
