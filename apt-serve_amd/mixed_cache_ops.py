"""Drop-in for the reference's ``mixed_cache_ops`` extension module.

The reference builds this module from one CUDA file
(additional_designs/mixed_cache_kernels/mixed_cache_setup.py:4-13) and imports it
at additional_designs/attention/backends/aptserve_flash_attn.py:8 and
additional_designs/model_executor/models/aptserve_opt.py:44.  With the directory
holding this file on ``sys.path``, ``import mixed_cache_ops`` resolves here and
the three operators keep their names and positional signatures
(mixed_cache.cu:233-237); the work is done by the gfx950 HIP library.
"""

from aptserve_hip.ops import cache_to_hidden, hidden_to_cache, mixed_kv_to_cache

__all__ = ["hidden_to_cache", "cache_to_hidden", "mixed_kv_to_cache"]
