"""The decode-attention entry point that allocates nothing (static device scratch) against the one that takes a
caller workspace: same kernels, so the results must be bit-identical.  Two calls in a row share the scratch
array, the second on a smaller problem."""
import numpy as np
import pytest
import torch

from aptserve_hip import _lib, ops
from test_attention_gpu import make_case

pytestmark = pytest.mark.gpu


def _both(c, dev, partition_size, **kw):
    g = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in c.items()}
    args = (g["q"], g["kc"], g["vc"], g["bt"], g["sl"], g["scale"])
    common = dict(block_types=g.get("types"), ws_k_cache=g.get("wk"), ws_v_cache=g.get("wv"),
                  partition_size=partition_size, max_seq_len=int(c["sl"].max()), **kw)
    ref = ops.paged_decode_attention(*args, **common)
    out = torch.full_like(ref, float("nan"))
    # the first static call of a process on a device looks the scratch array's address up (and may make the
    # runtime load the library's code object, which holds the array): allocation is measured around a later one
    ops.paged_decode_attention(*args, out=out, static_scratch=True, **common)
    torch.cuda.synchronize()
    out.fill_(float("nan"))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
    ops.paged_decode_attention(*args, out=out, static_scratch=True, **common)
    torch.cuda.synchronize()
    # torch's allocator did not grow, and neither did anything else on the device (hipMemGetInfo's free bytes
    # would show a hipMalloc made inside the library)
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    return out, ref


def test_static_scratch_matches_workspace_entry_on_two_calls_in_a_row(dev):
    big = make_case(6, 8, 128, 16, [2048, 700, 1, 257, 1500, 31], 21, hybrid=True)
    small = make_case(3, 8, 128, 16, [300, 40, 129], 22, hybrid=True)
    # partition sizes that split a sequence into more partitions than a workgroup has wavefronts: the partial
    # results go through the scratch; (big, 256) merges in LDS and touches no scratch
    for case, ps in ((big, 64), (small, 16), (big, 256), (big, 32)):
        out, ref = _both(case, dev, ps)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_static_scratch_holds_the_sequence_order_of_a_large_batch(dev):
    """More than 512 sequences: the longest-first order of the workgroups is computed by a kernel into the
    scratch.  Second call: fewer sequences (ranked inside the attention kernel, no scratch)."""
    rng = np.random.default_rng(5)
    lib = _lib.load()
    for B in (600, 40):
        lens = [int(x) for x in rng.integers(1, 65, B)]
        c = make_case(B, 8, 64, 16, lens, 24)
        assert (lib.aps_decode_attention_workspace_bytes(B, 8, 64, max(lens), 256) > 0) == (B > 512)
        out, ref = _both(c, dev, 256)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_static_scratch_fp8_and_single_partition(dev):
    c = make_case(4, 4, 64, 16, [100, 7, 64, 33], 23)
    # fp8 codes of the same values, one partition (no scratch is touched) and several
    for name in ("kc", "vc"):
        c[name] = torch.clamp(c[name].float() / 0.05, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    for ps in (128, 32):
        out, ref = _both(c, dev, ps, k_scale=0.05, v_scale=0.05)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_static_scratch_rejects_a_problem_beyond_its_limit(dev):
    lib = _lib.load()
    B, H, D, BS, W = 512, 40, 128, 16, 128
    need = lib.aps_decode_attention_workspace_bytes(B, H, D, W * BS, 64)
    assert need > 32 * 1024 * 1024
    q = torch.zeros(B, H, D, dtype=torch.float16, device=dev)
    kc = torch.zeros(4, BS, H, D, dtype=torch.float16, device=dev)
    bt = torch.zeros(B, W, dtype=torch.int32, device=dev)
    sl = torch.ones(B, dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    with pytest.raises(RuntimeError, match="static array"):
        ops.paged_decode_attention(q, kc, kc, bt, sl, partition_size=64, out=out, static_scratch=True)
    # the same problem with a caller workspace is fine
    ops.paged_decode_attention(q, kc, kc, bt, sl, partition_size=64, out=out)
    torch.cuda.synchronize()
