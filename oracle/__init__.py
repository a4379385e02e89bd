"""CPU oracle for the hybrid-cache hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the product:
only the test-suite, the smoke check and the benchmark's CPU-baseline leg may
import it, and there only as the checker.  The product path (the HIP library
and its Python host code) never imports this package and never falls back to
it.

Every function here restates, in plain PyTorch-CPU / numpy, what the reference
does on the hot path and cites the reference lines it follows.  The reference
ships no tests and no golden vectors, so each function is pinned by an
independent witness in ``tests/test_oracle_*.py``:

======================  =====================================================
function                pinned by
======================  =====================================================
hidden_to_cache         per-thread simulation of the reference kernel's grid
cache_to_hidden         (block/thread loops, element by element) on small
mixed_kv_to_cache       inputs; write->gather identity; sentinel check of
                        untouched slots; V-plane addressing; pad-slot skip
reshape_and_cache_flash element-by-element loop; 4-D indexing closed form
fp8_e4m3 quant/dequant  exhaustive 256-code table computed from the OCP bit
                        layout; brute-force nearest-value search in float64
                        with ties-to-even; PyTorch's float8_e4m3fn cast
kv_reproject / q_only   float64 numpy matmul; identity / one-hot weights
paged decode attention  float64 textbook softmax on dense K/V; L=1; equal
                        keys -> mean of V; block permutation invariance;
                        all-K/V vs all-hidden equivalence
absorbed hidden attn.   float64 textbook attention over K = W_k h + b_k, V = W_v h
                        + b_v of the same rows (any b_k); dropping b_v or
                        transposing W_k must break the agreement
mixed_reshape_and_cache composition of hidden_to_cache and
                        reshape_and_cache_flash (both pinned above)
layer.opt_attention     composition of the functions above; all-hidden vs
                        all-K/V caches built from the same hidden states agree;
                        decode after prefill equals the last row of a longer
                        prefill
build_metadata          the invariants the reference's own commented checks
                        list; brute force from an independent per-row
                        definition on tiny batches
======================  =====================================================

No function is "parity unpinned" in the sense of lacking such a check.  What
*is* unpinned is the exact fp16 bit pattern a cuBLAS GEMM or a flash-attn
kernel would produce: those libraries are not part of the reference tree, and
their outputs are covered by the stated tolerances instead (1e-3 relative with
fp32 accumulation, 2e-2 absolute for fp16 outputs).
"""

from . import cache_ops, fp8, reproject, attention, metadata, layer, model  # noqa: F401
