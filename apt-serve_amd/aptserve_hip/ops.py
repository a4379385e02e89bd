"""Tensor-level entry points of the hybrid-cache operators.

Each function validates its tensors on the host (device, dtype, innermost
contiguity, index dtype), then hands raw device pointers, sizes, strides and
the caller's current stream to the C ABI.  Nothing here computes: without the
HIP library these functions raise.
"""

from __future__ import annotations

import contextlib
import ctypes
from typing import Optional

import torch

from . import _lib

APS_F16, APS_BF16, APS_F32, APS_F64, APS_FP8_E4M3 = 0, 1, 2, 3, 4
MIXED_LITERAL_MODULO = 1
MIXED_SKIP_MIRROR = 2

_DTYPE_CODE = {
    torch.float16: APS_F16,
    torch.bfloat16: APS_BF16,
    torch.float32: APS_F32,
    torch.float64: APS_F64,
    torch.uint8: APS_FP8_E4M3,
}
if hasattr(torch, "float8_e4m3fn"):
    _DTYPE_CODE[torch.float8_e4m3fn] = APS_FP8_E4M3


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """Raw handle of torch's current stream on the tensor's device."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


_NO_SWITCH = contextlib.nullcontext()


def _on(dev):
    """Context that makes ``dev`` the current device for a launch; free when it already is."""
    return _NO_SWITCH if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


# The two checks below run several times per operator call: the conditions are tested first and the message
# (device and dtype names are slow to format) is only built for the one that failed.
def _check_data(name: str, t: torch.Tensor, dev) -> None:
    if (isinstance(t, torch.Tensor) and t.is_cuda and t.device == dev
            and (t.dim() == 0 or t.stride(-1) == 1 or t.size(-1) <= 1)):
        return
    _need(isinstance(t, torch.Tensor), f"{name} must be a tensor")
    _need(t.is_cuda, f"{name} must live on the GPU")
    _need(t.device == dev, f"{name} is on {t.device}, expected {dev}")
    raise ValueError(f"{name}: innermost dimension must be contiguous")


def _check_index(name: str, t: torch.Tensor, dev, dtype=torch.int64) -> None:
    if (isinstance(t, torch.Tensor) and t.dtype == dtype and t.is_cuda and t.device == dev and t.dim() == 1
            and (t.numel() <= 1 or t.stride(0) == 1)):
        return
    _need(isinstance(t, torch.Tensor), f"{name} must be a tensor")
    _need(t.dtype == dtype, f"{name} must be {dtype}, got {t.dtype}")
    _need(t.is_cuda and t.device == dev, f"{name} must live on {dev}")
    raise ValueError(f"{name} must be a contiguous vector")


def _check_paged(paged_cache: torch.Tensor, width: int) -> None:
    _need(paged_cache.dim() == 5, "paged_cache must be (2, num_blocks, block_size, heads, head_dim)")
    _need(paged_cache.is_contiguous(), "paged_cache must be contiguous")
    _need(paged_cache.stride(2) >= width, "row is wider than a cache slot")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None or t.numel() == 0 else t.data_ptr()


# --------------------------------------------------------------------- a1 / a2

def hidden_to_cache(hidden, paged_cache, slot_mapping, src_idx, target_slot_idx) -> None:
    """Drop-in for ``mixed_cache_ops.hidden_to_cache``
    (additional_designs/mixed_cache_kernels/mixed_cache.cu:119-147)."""
    dev = hidden.device
    _check_data("hidden", hidden, dev)
    _check_data("paged_cache", paged_cache, dev)
    _need(hidden.dim() == 2, "hidden must be [rows, hidden_size]")
    _need(hidden.dtype == paged_cache.dtype, "hidden and paged_cache dtypes differ")
    _check_paged(paged_cache, hidden.size(1))
    for n, t in (("slot_mapping", slot_mapping), ("src_idx", src_idx), ("target_slot_idx", target_slot_idx)):
        _check_index(n, t, dev)
    _need(src_idx.numel() == target_slot_idx.numel(), "src_idx and target_slot_idx lengths differ")
    slot_stride = paged_cache.stride(2)
    with _on(dev):
        st = _lib.load().aps_hidden_to_cache(
            hidden.data_ptr(), paged_cache.data_ptr(), _ptr(slot_mapping), _ptr(src_idx), _ptr(target_slot_idx),
            src_idx.numel(), hidden.size(1), hidden.stride(0), slot_stride, paged_cache.numel() // slot_stride,
            hidden.size(0), slot_mapping.numel(), hidden.element_size(), _stream(hidden))
    _lib.check(st, "hidden_to_cache")


def cache_to_hidden(hidden, paged_cache, slot_mapping, dst_idx) -> None:
    """Drop-in for ``mixed_cache_ops.cache_to_hidden`` (mixed_cache.cu:150-176)."""
    dev = hidden.device
    _check_data("hidden", hidden, dev)
    _check_data("paged_cache", paged_cache, dev)
    _need(hidden.dim() == 2, "hidden must be [rows, hidden_size]")
    _need(hidden.dtype == paged_cache.dtype, "hidden and paged_cache dtypes differ")
    _check_paged(paged_cache, hidden.size(1))
    _check_index("slot_mapping", slot_mapping, dev)
    _check_index("dst_idx", dst_idx, dev)
    slot_stride = paged_cache.stride(2)
    with _on(dev):
        st = _lib.load().aps_cache_to_hidden(
            hidden.data_ptr(), paged_cache.data_ptr(), _ptr(slot_mapping), _ptr(dst_idx), dst_idx.numel(),
            hidden.size(1), hidden.stride(0), slot_stride, paged_cache.numel() // slot_stride, hidden.size(0),
            slot_mapping.numel(), hidden.element_size(), _stream(hidden))
    _lib.check(st, "cache_to_hidden")


def hybrid_decode_gather(holder, hidden_states, paged_cache, slot_mapping, hidden_holder_upd,
                         hidden_holder_pull, hidden_cache_use_input, hidden_cache_store_tot) -> None:
    """One launch for the decode-side store + holder assembly of
    additional_designs/model_executor/models/aptserve_opt.py:108-121.  ``holder``
    may be uninitialised memory (``torch.empty``): every row is written."""
    dev = holder.device
    for n, t in (("holder", holder), ("hidden_states", hidden_states), ("paged_cache", paged_cache)):
        _check_data(n, t, dev)
    _need(holder.dim() == 2 and hidden_states.dim() == 2, "holder and hidden_states must be 2-D")
    _need(holder.size(1) == hidden_states.size(1), "holder and hidden_states widths differ")
    _need(holder.dtype == hidden_states.dtype == paged_cache.dtype, "dtypes differ")
    _check_paged(paged_cache, holder.size(1))
    for n, t in (("slot_mapping", slot_mapping), ("hidden_holder_upd", hidden_holder_upd),
                 ("hidden_holder_pull", hidden_holder_pull), ("hidden_cache_use_input", hidden_cache_use_input),
                 ("hidden_cache_store_tot", hidden_cache_store_tot)):
        _check_index(n, t, dev)
    _need(hidden_holder_upd.numel() == hidden_states.size(0), "one upd row per sequence expected")
    _need(hidden_holder_upd.numel() + hidden_holder_pull.numel() == holder.size(0),
          "upd and pull must partition the holder rows")
    _need(slot_mapping.numel() == holder.size(0), "slot_mapping must have one entry per holder row")
    _need(hidden_cache_use_input.numel() == hidden_cache_store_tot.numel(), "store index lengths differ")
    slot_stride = paged_cache.stride(2)
    with _on(dev):
        st = _lib.load().aps_hybrid_decode_gather(
            holder.data_ptr(), hidden_states.data_ptr(), paged_cache.data_ptr(), _ptr(slot_mapping),
            _ptr(hidden_holder_upd), hidden_holder_upd.numel(), _ptr(hidden_holder_pull),
            hidden_holder_pull.numel(), _ptr(hidden_cache_use_input), _ptr(hidden_cache_store_tot),
            hidden_cache_store_tot.numel(), holder.size(1), holder.stride(0), hidden_states.stride(0), slot_stride,
            paged_cache.numel() // slot_stride, holder.size(0), holder.element_size(), _stream(holder))
    _lib.check(st, "hybrid_decode_gather")


def gather_hidden_rows(holder, hidden_states, paged_cache, holder_src, slot_mapping, hidden_cache_use_input,
                       hidden_cache_store_tot) -> None:
    """``hybrid_decode_gather`` with the row sources resolved by the metadata builder
    (``HybridAttentionMetadata.holder_src``): same result, one index load per chunk."""
    dev = holder.device
    for n, t in (("holder", holder), ("hidden_states", hidden_states), ("paged_cache", paged_cache)):
        _check_data(n, t, dev)
    _need(holder.dim() == 2 and hidden_states.dim() == 2, "holder and hidden_states must be 2-D")
    _need(holder.size(1) == hidden_states.size(1), "holder and hidden_states widths differ")
    _need(holder.dtype == hidden_states.dtype == paged_cache.dtype, "dtypes differ")
    _check_paged(paged_cache, holder.size(1))
    for n, t in (("holder_src", holder_src), ("slot_mapping", slot_mapping),
                 ("hidden_cache_use_input", hidden_cache_use_input),
                 ("hidden_cache_store_tot", hidden_cache_store_tot)):
        _check_index(n, t, dev)
    _need(holder_src.numel() == holder.size(0), "holder_src must have one entry per holder row")
    _need(slot_mapping.numel() == holder.size(0), "slot_mapping must have one entry per holder row")
    _need(hidden_cache_use_input.numel() == hidden_cache_store_tot.numel(), "store index lengths differ")
    slot_stride = paged_cache.stride(2)
    with _on(dev):
        st = _lib.load().aps_gather_hidden_rows(
            holder.data_ptr(), hidden_states.data_ptr(), paged_cache.data_ptr(), _ptr(holder_src), holder.size(0),
            _ptr(slot_mapping), _ptr(hidden_cache_use_input), _ptr(hidden_cache_store_tot),
            hidden_cache_store_tot.numel(), hidden_states.size(0), holder.size(1), holder.stride(0),
            hidden_states.stride(0), slot_stride, paged_cache.numel() // slot_stride, holder.element_size(),
            _stream(holder))
    _lib.check(st, "gather_hidden_rows")


APS_CACHE_JOB_BYTES = 320


class CacheJob:
    """A decode step's planned, not yet launched cache writes (``decode_step_cache_ops(..., as_job=True)``):
    opaque host bytes that the library wrote, and the tensors the launch will touch, kept alive."""

    def __init__(self, anchor, tensors):
        self._buf = (ctypes.c_uint64 * (APS_CACHE_JOB_BYTES // 8))()
        self.address = ctypes.addressof(self._buf)
        self._anchor = anchor
        self._tensors = tensors

    def launch(self) -> None:
        """Launch the job by itself on the current stream of its device."""
        with _on(self._anchor.device):
            st = _lib.load().aps_cache_job_launch(self.address, _stream(self._anchor))
        _lib.check(st, "cache_job_launch")


def decode_step_cache_ops(holder, hidden_states, paged_cache, holder_src, slot_mapping, hidden_cache_use_input,
                          hidden_cache_store_tot, key, value, kv_cache_use_input, new_token_slot,
                          kv_cache=None, as_job: bool = False):
    """The cache traffic of one decode layer in one launch: ``gather_hidden_rows`` (store of the newest hidden
    rows, holder assembly: additional_designs/model_executor/models/aptserve_opt.py:108-121) and the write of
    the newest K/V rows of the K/V-cached sequences into the two planes of ``paged_cache``
    (``reshape_and_cache_flash``, additional_designs/attention/backends/aptserve_flash_attn.py:338-345).
    ``key`` / ``value`` ``[batch, H*D]`` or ``[batch, H, D]``; ``kv_cache_use_input`` and ``new_token_slot``
    from the metadata builder.  Same bytes in the cache and the holder as the two separate calls.
    ``holder`` (and ``holder_src``) may be ``None``: the stores alone, for a data flow that assembles no holder.
    ``key`` and ``value`` may be ``None``: a step without K/V-cached sequences.
    ``kv_cache``: the K/V planes when they are not ``paged_cache`` (a separate hidden-row cache).
    ``as_job=True`` checks and plans the call but launches nothing: the :class:`CacheJob` that comes back is
    launched later, by itself or as the stores that precede :func:`absorbed_hidden_attention`."""
    dev = hidden_states.device
    no_kv = key is None
    _need((value is None) == no_kv, "key and value come together")
    for n, t in (("hidden_states", hidden_states), ("paged_cache", paged_cache)) + (
            () if no_kv else (("key", key), ("value", value))):
        _check_data(n, t, dev)
    _need(hidden_states.dim() == 2, "hidden_states must be 2-D")
    width = hidden_states.size(1)
    n_rows = slot_mapping.numel()
    if holder is not None:
        _check_data("holder", holder, dev)
        _need(holder.dim() == 2 and holder.size(1) == width and holder.dtype == hidden_states.dtype,
              "holder must be 2-D, as wide as hidden_states and of its dtype")
        _need(holder.size(0) == n_rows, "slot_mapping must have one entry per holder row")
        _check_index("holder_src", holder_src, dev)
        _need(holder_src.numel() == n_rows, "holder_src must have one entry per holder row")
    kvc = paged_cache if kv_cache is None else kv_cache
    _check_data("kv_cache", kvc, dev)
    _need(hidden_states.dtype == paged_cache.dtype == kvc.dtype, "dtypes differ")
    _need(no_kv or hidden_states.dtype == key.dtype == value.dtype, "dtypes differ")
    for c in (paged_cache, kvc):
        _check_paged(c, width)
        _need(c.size(0) == 2 and c.size(3) * c.size(4) == width,
              "a cache must be (2, num_blocks, block_size, heads, head_dim) with heads*head_dim == hidden width")
    B = hidden_states.size(0)
    for n, t in (("slot_mapping", slot_mapping), ("hidden_cache_use_input", hidden_cache_use_input),
                 ("hidden_cache_store_tot", hidden_cache_store_tot)):
        _check_index(n, t, dev)
    _need(hidden_cache_use_input.numel() == hidden_cache_store_tot.numel(), "store index lengths differ")
    if not no_kv:
        key = _as_thd("key", key, kvc.size(3), kvc.size(4))
        value = _as_thd("value", value, kvc.size(3), kvc.size(4))
        _need(key.size(0) == B and value.size(0) == B, "one key / value row per sequence expected")
        for n, t in (("kv_cache_use_input", kv_cache_use_input), ("new_token_slot", new_token_slot)):
            _check_index(n, t, dev)
        _need(new_token_slot.numel() == B, "new_token_slot must have one entry per sequence")
    slot_stride = paged_cache.stride(2)
    args = (None if holder is None else _ptr(holder), hidden_states.data_ptr(), paged_cache.data_ptr(),
            None if holder is None else _ptr(holder_src), n_rows,
            _ptr(slot_mapping), _ptr(hidden_cache_use_input), _ptr(hidden_cache_store_tot),
            hidden_cache_store_tot.numel(), B, width, 0 if holder is None else holder.stride(0), hidden_states.stride(0),
            slot_stride, paged_cache.numel() // slot_stride) + (
        (None, None, None, None, None, None, 0, 0, 0) if no_kv else
        (key.data_ptr(), value.data_ptr(), kvc[0].data_ptr(), kvc[1].data_ptr(), _ptr(kv_cache_use_input),
         _ptr(new_token_slot), kv_cache_use_input.numel(), key.stride(0), value.stride(0))) + (
        kvc.size(2), kvc.stride(1), kvc.size(1), hidden_states.element_size())
    if as_job:
        job = CacheJob(hidden_states, (holder, paged_cache, holder_src, slot_mapping, hidden_cache_use_input,
                                       hidden_cache_store_tot, key, value, kvc, kv_cache_use_input, new_token_slot))
        _lib.check(_lib.load().aps_decode_step_cache_ops_job(job.address, APS_CACHE_JOB_BYTES, *args),
                   "decode_step_cache_ops_job")
        return job
    with _on(dev):
        st = _lib.load().aps_decode_step_cache_ops(*args, _stream(hidden_states))
    _lib.check(st, "decode_step_cache_ops")


# --------------------------------------------------------------------- a3 / a4

def _check_kv_cache(name: str, c: torch.Tensor, heads: int, head_size: int) -> None:
    _need(c.dim() == 4, f"{name} must be [num_blocks, block_size, heads, head_dim]")
    _need(c.size(2) == heads and c.size(3) == head_size, f"{name}: head layout differs from key/value")
    _need(c.stride(3) == 1 and c.stride(2) == head_size and c.stride(1) == heads * head_size,
          f"{name}: a block must be contiguous")


def _as_thd(name: str, t: torch.Tensor, heads: int, head_size: int) -> torch.Tensor:
    if t.dim() == 2:
        _need(t.size(1) == heads * head_size, f"{name} has the wrong width")
        return t
    _need(t.dim() == 3 and t.size(1) == heads and t.size(2) == head_size, f"{name} must be [tokens, heads, head_dim]")
    _need(t.stride(2) == 1 and t.stride(1) == head_size, f"{name}: a token row must be contiguous")
    return t


def reshape_and_cache_flash(key, value, key_cache, value_cache, slot_mapping, kv_cache_dtype: str = "auto",
                            k_scale: float = 1.0, v_scale: float = 1.0,
                            token_idx: Optional[torch.Tensor] = None) -> None:
    """Same call shape as ``vllm._custom_ops.reshape_and_cache_flash`` as used at
    additional_designs/attention/backends/aptserve_flash_attn.py:338-345.
    ``kv_cache_dtype``: ``"auto"`` (cache dtype == key dtype) or ``"fp8"``
    (uint8 / float8_e4m3fn cache holding e4m3 codes of ``x / scale``).
    ``token_idx`` selects a subset of tokens without gather copies (``:348-355``)."""
    dev = key.device
    heads, head_size = key_cache.size(2), key_cache.size(3)
    for n, t in (("key", key), ("value", value), ("key_cache", key_cache), ("value_cache", value_cache)):
        _check_data(n, t, dev)
    key = _as_thd("key", key, heads, head_size)
    value = _as_thd("value", value, heads, head_size)
    _check_kv_cache("key_cache", key_cache, heads, head_size)
    _check_kv_cache("value_cache", value_cache, heads, head_size)
    _need(key.dtype == value.dtype and key_cache.dtype == value_cache.dtype, "K and V dtypes differ")
    _need(key_cache.shape == value_cache.shape and key_cache.stride(0) == value_cache.stride(0),
          "key_cache and value_cache layouts differ")
    _check_index("slot_mapping", slot_mapping, dev)
    if kv_cache_dtype == "auto":
        _need(key_cache.dtype == key.dtype, "kv_cache_dtype='auto' needs cache dtype == key dtype")
    elif kv_cache_dtype in ("fp8", "fp8_e4m3"):
        _need(key_cache.element_size() == 1, "fp8 cache must be uint8 / float8_e4m3fn")
    else:
        raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")
    _need(key.dtype in (torch.float16, torch.bfloat16, torch.float32), f"unsupported key dtype {key.dtype}")
    if token_idx is not None:
        _check_index("token_idx", token_idx, dev)
        n = token_idx.numel()
        _need(slot_mapping.numel() >= key.size(0) or n == 0, "slot_mapping shorter than key")
        num_tokens = min(key.size(0), slot_mapping.numel())
    else:
        n = slot_mapping.numel()
        _need(n <= key.size(0) and n <= value.size(0), "slot_mapping longer than key/value")
        num_tokens = n
    with _on(dev):
        st = _lib.load().aps_reshape_and_cache_flash(
            key.data_ptr(), value.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), _ptr(slot_mapping),
            _ptr(token_idx), n, num_tokens, heads, head_size, key_cache.size(1), key.stride(0), value.stride(0),
            key_cache.stride(0), key_cache.size(0), _DTYPE_CODE[key.dtype], _DTYPE_CODE[key_cache.dtype],
            float(k_scale), float(v_scale), _stream(key))
    _lib.check(st, "reshape_and_cache_flash")


def mixed_reshape_and_cache(key, value, hidden, kv_cache, slot_mapping, is_hidden, kv_cache_dtype: str = "auto",
                            k_scale: float = 1.0, v_scale: float = 1.0, hidden_cache=None) -> None:
    """Cache write of a step whose tokens differ in cache type, one launch.

    Token ``t`` with ``is_hidden[t]`` stores ``hidden[t]`` at slot ``slot_mapping[t]`` of the
    flattened paged cache (what ``hidden_to_cache`` does for the hidden tokens of a prompt step,
    additional_designs/model_executor/models/aptserve_opt.py:125-126); every other token stores
    ``key[t]`` / ``value[t]`` by block (``reshape_and_cache_flash`` over the K/V tokens,
    additional_designs/attention/backends/aptserve_flash_attn.py:347-355).  ``kv_cache`` is the
    ``(2, N, BS, H, D)`` cache of the layer.  With ``kv_cache_dtype='fp8'`` the K/V rows are stored
    as e4m3 codes of ``x / scale`` in the 1-byte ``kv_cache`` and hidden rows go, unquantised, to
    the separate ``hidden_cache`` (same shape, activation dtype).  ``key``/``value`` or ``hidden``
    may be ``None`` to store only the other kind."""
    _need(kv_cache is not None and kv_cache.dim() == 5 and kv_cache.size(0) == 2,
          "kv_cache must be (2, num_blocks, block_size, heads, head_dim)")
    dev = kv_cache.device
    _check_data("kv_cache", kv_cache, dev)
    _need(kv_cache.is_contiguous(), "kv_cache must be contiguous")
    _, nblk, bs, heads, head_size = kv_cache.shape
    width = heads * head_size
    _need((key is None) == (value is None), "key and value must be given together")
    _need(key is not None or hidden is not None, "nothing to store")
    _check_index("slot_mapping", slot_mapping, dev)
    T = slot_mapping.numel()
    src_dtype = None
    if key is not None:
        for n, t in (("key", key), ("value", value)):
            _check_data(n, t, dev)
        key = _as_thd("key", key, heads, head_size)
        value = _as_thd("value", value, heads, head_size)
        _need(key.dtype == value.dtype, "K and V dtypes differ")
        _need(key.size(0) >= T and value.size(0) >= T, "slot_mapping longer than key/value")
        src_dtype = key.dtype
    if hidden is not None:
        _check_data("hidden", hidden, dev)
        _need(hidden.dim() == 2 and hidden.size(1) == width and hidden.size(0) >= T,
              "hidden must be [tokens, heads*head_dim]")
        _need(src_dtype is None or hidden.dtype == src_dtype, "hidden and key dtypes differ")
        src_dtype = hidden.dtype
        _need(is_hidden is not None, "hidden rows need the is_hidden mask")
    _need(src_dtype in (torch.float16, torch.bfloat16, torch.float32), f"unsupported dtype {src_dtype}")
    if is_hidden is not None:
        _need(is_hidden.device == dev and is_hidden.dtype in (torch.uint8, torch.bool) and is_hidden.is_contiguous()
              and is_hidden.numel() == T, "is_hidden must be a contiguous uint8/bool vector, one entry per token")
    if kv_cache_dtype == "auto":
        _need(kv_cache.dtype == src_dtype, "kv_cache_dtype='auto' needs cache dtype == activation dtype")
        hcache = kv_cache if hidden_cache is None else hidden_cache
    elif kv_cache_dtype in ("fp8", "fp8_e4m3"):
        _need(kv_cache.element_size() == 1, "fp8 cache must be uint8 / float8_e4m3fn")
        _need(hidden is None or hidden_cache is not None, "an fp8 K/V cache cannot hold hidden rows: pass hidden_cache")
        hcache = hidden_cache
    else:
        raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")
    hidden_slots = hidden_stride = 0
    if hidden is not None:
        _check_data("hidden_cache", hcache, dev)
        _check_paged(hcache, width)
        _need(hcache.dtype == src_dtype, "hidden cache dtype differs from the activations")
        hidden_stride = hcache.stride(2)
        hidden_slots = hcache.numel() // hidden_stride
    cache_code = _DTYPE_CODE[kv_cache.dtype] if key is not None else _DTYPE_CODE[src_dtype]
    with _on(dev):
        st = _lib.load().aps_mixed_reshape_and_cache(
            _ptr(key), _ptr(value), _ptr(hidden), kv_cache[0].data_ptr(), kv_cache[1].data_ptr(),
            None if hidden is None else hcache.data_ptr(), _ptr(slot_mapping), _ptr(is_hidden), T, heads, head_size, bs,
            0 if key is None else key.stride(0), 0 if key is None else value.stride(0),
            0 if hidden is None else hidden.stride(0), kv_cache.stride(1), nblk, hidden_stride, hidden_slots,
            _DTYPE_CODE[src_dtype], cache_code, float(k_scale), float(v_scale), _stream(kv_cache))
    _lib.check(st, "mixed_reshape_and_cache")


def mixed_kv_to_cache(key, value, k_cache, v_cache, shared_k_cache, shared_v_cache, slot_mapping,
                      slot_mapping_shared, kv_cache_use_tot, hidden_cache_use_tot, *,
                      literal_modulo: bool = False, skip_mirror: bool = False) -> None:
    """Drop-in for ``mixed_cache_ops.mixed_kv_to_cache`` (mixed_cache.cu:179-230).

    Range C uses ``off = blk - 2*nkv``.  The reference's ``blk % (2*nkv)`` (``:88``)
    is the same value while ``len(slot_mapping_shared) <= 2*len(kv_cache_use_tot)``;
    ``literal_modulo=True`` reproduces the reference beyond that point too."""
    dev = key.device
    heads, head_size = k_cache.size(2), k_cache.size(3)
    for n, t in (("key", key), ("value", value), ("k_cache", k_cache), ("v_cache", v_cache),
                 ("shared_k_cache", shared_k_cache), ("shared_v_cache", shared_v_cache)):
        _check_data(n, t, dev)
    key = _as_thd("key", key, heads, head_size)
    value = _as_thd("value", value, heads, head_size)
    for n, c in (("k_cache", k_cache), ("v_cache", v_cache), ("shared_k_cache", shared_k_cache),
                 ("shared_v_cache", shared_v_cache)):
        _check_kv_cache(n, c, heads, head_size)
        _need(c.dtype == key.dtype, f"{n} dtype differs from key")
    _need(value.dtype == key.dtype, "key and value dtypes differ")
    # the reference's single check (mixed_cache.cu:202), as a RuntimeError like TORCH_CHECK
    if k_cache.stride(0) != v_cache.stride(0):
        raise RuntimeError("k_cache.stride(0) == v_cache.stride(0) must hold")
    _need(shared_k_cache.stride(0) == shared_v_cache.stride(0), "shared cache block strides differ")
    _need(k_cache.size(1) == shared_k_cache.size(1), "block sizes differ")
    for n, t in (("slot_mapping", slot_mapping), ("slot_mapping_shared", slot_mapping_shared),
                 ("kv_cache_use_tot", kv_cache_use_tot), ("hidden_cache_use_tot", hidden_cache_use_tot)):
        _check_index(n, t, dev)
    _need(hidden_cache_use_tot.numel() >= slot_mapping_shared.numel(),
          "hidden_cache_use_tot shorter than slot_mapping_shared")
    num_tot = min(key.size(0), value.size(0))
    if kv_cache_use_tot.numel():
        num_tot = min(num_tot, slot_mapping.numel())
    n_hidden = slot_mapping_shared.numel()
    flags = (MIXED_LITERAL_MODULO if literal_modulo else 0) | (MIXED_SKIP_MIRROR if skip_mirror else 0)
    with _on(dev):
        st = _lib.load().aps_mixed_kv_to_cache(
            key.data_ptr(), value.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), shared_k_cache.data_ptr(),
            shared_v_cache.data_ptr(), _ptr(slot_mapping), _ptr(slot_mapping_shared), _ptr(kv_cache_use_tot),
            _ptr(hidden_cache_use_tot), kv_cache_use_tot.numel(), n_hidden, num_tot, heads, head_size,
            k_cache.size(1), key.stride(0), value.stride(0), k_cache.stride(0), k_cache.size(0),
            shared_k_cache.stride(0), shared_k_cache.size(0), key.element_size(), flags, _stream(key))
    _lib.check(st, "mixed_kv_to_cache")


# --------------------------------------------------------------------- a8

APS_ATTENTION_JOB_BYTES = 320


class AttentionJob:
    """A planned, not yet launched paged decode attention (``paged_decode_attention(..., as_job=True)``):
    opaque host bytes that the library wrote, and the tensors the launch will touch, kept alive."""

    def __init__(self, out, tensors):
        self._buf = (ctypes.c_uint64 * (APS_ATTENTION_JOB_BYTES // 8))()
        self.address = ctypes.addressof(self._buf)
        self.out = out
        self._tensors = tensors

    def launch(self):
        """Launch the job by itself on the current stream of its device; returns the output tensor."""
        with _on(self.out.device):
            st = _lib.load().aps_attention_job_launch(self.address, _stream(self.out))
        _lib.check(st, "attention_job_launch")
        return self.out


def paged_decode_attention(q, k_cache, v_cache, block_tables, seq_lens, softmax_scale=None, *,
                           block_types=None, ws_k_cache=None, ws_v_cache=None, k_scale: float = 1.0,
                           v_scale: float = 1.0, max_seq_len: Optional[int] = None, partition_size: int = 0,
                           out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
                           static_scratch: bool = False, as_job: bool = False):
    """Decode attention of one query token per sequence over paged K/V.

    ``q`` ``[B, H, D]`` f16/bf16; caches ``[blocks, BS, H, D]`` in ``q``'s dtype or
    uint8/float8_e4m3fn (fp8 codes, dequantised with ``k_scale``/``v_scale``);
    ``block_tables`` int32 ``[B, W]``; ``seq_lens`` int32 ``[B]``.  ``block_types``
    (uint8 ``[B, W]``, optional) sends a logical block to ``ws_k_cache``/``ws_v_cache``
    when non-zero.  ``max_seq_len`` is a host-side bound on ``seq_lens`` (default
    ``W * BS``, which needs no device read-back).  Returns ``[B, H, D]``.
    ``static_scratch=True`` (with ``out`` given) takes the entry point that allocates
    nothing: partial results go to the library's static device array, and a problem
    that does not fit it raises.  ``as_job=True`` checks and plans the call but launches nothing:
    the :class:`AttentionJob` that comes back is launched later, by itself or as the K/V-cached half
    of :func:`absorbed_hidden_attention`.
    """
    dev = q.device
    _check_data("q", q, dev)
    _need(q.dim() == 3, "q must be [batch, heads, head_dim]")
    B, H, D = q.shape
    _need(q.dtype in (torch.float16, torch.bfloat16), "q must be float16 or bfloat16")
    _need(q.stride(2) == 1 and q.stride(1) == D, "q: heads of one token must be contiguous")
    _check_data("k_cache", k_cache, dev)
    _check_data("v_cache", v_cache, dev)
    _check_kv_cache("k_cache", k_cache, H, D)
    _check_kv_cache("v_cache", v_cache, H, D)
    _need(k_cache.dtype == v_cache.dtype and k_cache.stride(0) == v_cache.stride(0) and
          k_cache.size(0) == v_cache.size(0), "k_cache and v_cache layouts differ")
    fp8 = k_cache.element_size() == 1
    _need(fp8 or k_cache.dtype == q.dtype, "cache dtype must equal q dtype or be an fp8 byte cache")
    BS = k_cache.size(1)
    _check_index("seq_lens", seq_lens, dev, torch.int32)
    _need(seq_lens.numel() == B, "one seq_len per query expected")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.size(0) == B,
          "block_tables must be int32 [batch, width]")
    _need(block_tables.device == dev and (block_tables.size(1) <= 1 or block_tables.stride(1) == 1),
          "block_tables rows must be contiguous on the same GPU")
    W = block_tables.size(1)
    ws_stride = ws_blocks = types_stride = 0
    if block_types is not None:
        _need(block_types.dtype == torch.uint8 and block_types.dim() == 2 and block_types.size(0) == B and
              block_types.size(1) >= W and block_types.device == dev, "block_types must be uint8 [batch, >=width]")
        _need(block_types.size(1) <= 1 or block_types.stride(1) == 1, "block_types rows must be contiguous")
        _need(ws_k_cache is not None and ws_v_cache is not None, "block_types needs the workspace caches")
        for n, c in (("ws_k_cache", ws_k_cache), ("ws_v_cache", ws_v_cache)):
            _check_data(n, c, dev)
            _check_kv_cache(n, c, H, D)
            _need(c.dtype == k_cache.dtype and c.size(1) == BS, f"{n} must match the cache dtype and block size")
        _need(ws_k_cache.stride(0) == ws_v_cache.stride(0) and ws_k_cache.size(0) == ws_v_cache.size(0),
              "workspace K and V layouts differ")
        ws_stride, ws_blocks, types_stride = ws_k_cache.stride(0), ws_k_cache.size(0), block_types.stride(0)
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if max_seq_len is None:
        max_seq_len = W * BS
    max_seq_len = min(int(max_seq_len), W * BS)
    if out is None:
        out = torch.empty_like(q)
    else:
        _check_data("out", out, dev)
        _need(out.shape == q.shape and out.dtype == q.dtype and out.stride(2) == 1 and out.stride(1) == D,
              "out must look like q")
    lib = _lib.load()
    if partition_size <= 0:
        partition_size = lib.aps_decode_attention_partition_size(B, H, max(max_seq_len, 1), BS)
    if static_scratch:
        with _on(dev):
            st = lib.aps_paged_decode_attention_static(
                out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                None if block_types is None else ws_k_cache.data_ptr(),
                None if block_types is None else ws_v_cache.data_ptr(),
                _ptr(block_tables), None if block_types is None else _ptr(block_types), _ptr(seq_lens), B, H, D, BS,
                W, block_tables.stride(0) if W else 0, types_stride, q.stride(0), out.stride(0), k_cache.stride(0),
                k_cache.size(0), ws_stride, ws_blocks, max_seq_len, partition_size, float(softmax_scale),
                _DTYPE_CODE[q.dtype], APS_FP8_E4M3 if fp8 else _DTYPE_CODE[q.dtype], float(k_scale),
                float(v_scale), _stream(q))
        _lib.check(st, "paged_decode_attention_static")
        return out
    need = lib.aps_decode_attention_workspace_bytes(B, H, D, max(max_seq_len, 1), partition_size)
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    ws_ptr = workspace.data_ptr() if (need and workspace is not None) else None
    ws_bytes = workspace.numel() * workspace.element_size() if (need and workspace is not None) else 0
    if as_job:
        _need(not static_scratch, "a job takes a workspace, not the static scratch")
        job = AttentionJob(out, (q, k_cache, v_cache, ws_k_cache, ws_v_cache, block_tables, block_types, seq_lens,
                                 workspace))
        st = lib.aps_paged_decode_attention_job(
            job.address, APS_ATTENTION_JOB_BYTES, out.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
            v_cache.data_ptr(), None if block_types is None else ws_k_cache.data_ptr(),
            None if block_types is None else ws_v_cache.data_ptr(),
            _ptr(block_tables), None if block_types is None else _ptr(block_types), _ptr(seq_lens), B, H, D, BS, W,
            block_tables.stride(0) if W else 0, types_stride, q.stride(0), out.stride(0), k_cache.stride(0),
            k_cache.size(0), ws_stride, ws_blocks, max_seq_len, partition_size, float(softmax_scale),
            _DTYPE_CODE[q.dtype], APS_FP8_E4M3 if fp8 else _DTYPE_CODE[q.dtype], float(k_scale), float(v_scale),
            ws_ptr, ws_bytes)
        _lib.check(st, "paged_decode_attention_job")
        return job
    with _on(dev):
        st = lib.aps_paged_decode_attention(
            out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            None if block_types is None else ws_k_cache.data_ptr(),
            None if block_types is None else ws_v_cache.data_ptr(),
            _ptr(block_tables), None if block_types is None else _ptr(block_types), _ptr(seq_lens), B, H, D, BS, W,
            block_tables.stride(0) if W else 0, types_stride, q.stride(0), out.stride(0), k_cache.stride(0),
            k_cache.size(0), ws_stride, ws_blocks, max_seq_len, partition_size, float(softmax_scale),
            _DTYPE_CODE[q.dtype], APS_FP8_E4M3 if fp8 else _DTYPE_CODE[q.dtype], float(k_scale), float(v_scale),
            ws_ptr, ws_bytes, _stream(q))
    _lib.check(st, "paged_decode_attention")
    return out


def flash_attn_with_kvcache(q, k_cache, v_cache, block_table=None, cache_seqlens=None, softmax_scale=None,
                            causal: bool = True, alibi_slopes=None, **kw):
    """Decode case of the third-party function with the keyword names used at
    additional_designs/attention/backends/aptserve_flash_attn.py:452-473:
    ``q [B,1,H,D]`` -> ``[B,1,H,D]``."""
    _need(q.dim() == 4 and q.size(1) == 1, "only one query token per sequence (decode) is supported")
    _need(alibi_slopes is None, "alibi_slopes is not supported")
    _need(block_table is not None and cache_seqlens is not None, "a paged cache needs block_table and cache_seqlens")
    o = paged_decode_attention(q[:, 0], k_cache, v_cache, block_table, cache_seqlens, softmax_scale, **kw)
    return o.unsqueeze(1)


# --------------------------------------------------------------------- a5 / a6

_TILE_COUNTERS = {}


def _tile_counters(dev) -> torch.Tensor:
    """The zero-initialised tile counters of ``aps_linear_nt`` for the current stream of ``dev``: every call
    leaves them zero again, and calls on one stream run one after the other, so one array per (device, stream)
    serves them all.  Under stream capture the array of the capturing stream is the one a replay uses."""
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    t = _TILE_COUNTERS.get(key)
    if t is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("linear_nt: the first K-split product on a stream allocates and clears its tile counters; "
                               "run one eager step on the capturing stream before recording it")
        with torch.cuda.stream(torch.cuda.default_stream(dev)):     # allocated and cleared outside any capture
            t = torch.zeros(256, dtype=torch.int32, device=dev)
        torch.cuda.default_stream(dev).synchronize()
        _TILE_COUNTERS[key] = t
    return t


def linear_nt(x, weight, bias=None, out=None, out_row_map=None, workspace=None, split_k: bool = True,
              relu: bool = False):
    """``out = x @ weight.T + bias`` on the matrix cores (f16/bf16, fp32 accumulation).

    ``x [M, K]`` and ``weight [N, K]`` may be row-strided views (a row slice of the fused
    QKV weight, a ``chunk`` of activations); ``N % 256 == 0`` and ``K % 64 == 0``.
    ``out_row_map`` (int64 ``[M]``) scatters result row ``m`` to ``out[out_row_map[m]]``.
    With ``split_k`` (default) a problem of few output tiles is split along K through an fp32
    ``workspace`` (allocated here when not given) so that enough workgroups stream the weights.
    ``relu``: negative results are stored as zero (``fc1`` with the activation that follows it,
    additional_designs/model_executor/models/aptserve_opt.py:204-205).
    The K split of a decode step's few rows is summed inside the same launch (by the workgroup that finishes a
    tile last) with the help of a small array of counters kept per device and stream (:func:`_tile_counters`).
    """
    dev = x.device
    _check_data("x", x, dev)
    _check_data("weight", weight, dev)
    _need(x.dim() == 2 and weight.dim() == 2 and x.size(1) == weight.size(1), "x [M,K] and weight [N,K] expected")
    _need(x.dtype == weight.dtype and x.dtype in (torch.float16, torch.bfloat16), "f16 or bf16 operands expected")
    M, K = x.shape
    N = weight.size(0)
    if bias is not None:
        _check_data("bias", bias, dev)
        _need(bias.dim() == 1 and bias.numel() == N and bias.dtype == x.dtype and bias.is_contiguous(),
              "bias must be a contiguous [N] vector of the operand dtype")
    if out is None:
        _need(out_row_map is None, "a row map needs a destination")
        out = torch.empty(M, N, dtype=x.dtype, device=dev)
    _check_data("out", out, dev)
    _need(out.dim() == 2 and out.size(1) >= N and out.dtype == x.dtype, "out must be [rows, >=N] of the operand dtype")
    if out_row_map is not None:
        _check_index("out_row_map", out_row_map, dev)
        _need(out_row_map.numel() == M, "one destination row per input row expected")
    else:
        _need(out.size(0) >= M, "out has fewer rows than x")
    lib = _lib.load()
    need = lib.aps_linear_nt_workspace_bytes(M, N, K) if split_k else 0
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)     # scratch is host-side plumbing
    ws_ptr = workspace.data_ptr() if need else None
    with _on(dev):
        st = lib.aps_linear_nt(
            x.data_ptr() if M else None, weight.data_ptr(), None if bias is None else bias.data_ptr(),
            out.data_ptr() if out.numel() else None, M, N, K, x.stride(0), weight.stride(0), out.stride(0),
            None if out_row_map is None else _ptr(out_row_map), out.size(0), _DTYPE_CODE[x.dtype],
            1 if relu else 0, ws_ptr,
            workspace.numel() * workspace.element_size() if need else 0,
            _tile_counters(dev).data_ptr() if need else None, _stream(x))
    _lib.check(st, "linear_nt")
    return out


def kv_reproject(x, w_kv, b_kv=None, out=None):
    """K/V re-projection of gathered hidden rows: ``[T,Hd] x w_kv[2Hd,Hd]^T + b_kv -> [T,2Hd]``
    (``k, v = out.chunk(2, -1)``), additional_designs/model_executor/models/aptserve_opt.py:123-124."""
    return linear_nt(x, w_kv, b_kv, out=out)


def kv_reproject_to_cache(x, w_kv, b_kv, ws_k_cache, ws_v_cache, k_cache, v_cache, kv_dest, workspace=None,
                          split_k: bool = True) -> None:
    """K/V re-projection whose epilogue writes every row straight into its ``[blocks, BS, H, D]``
    cache slot; replaces the ``kv_only`` projection, the ``chunk`` and ``mixed_kv_to_cache``
    (additional_designs/model_executor/models/aptserve_opt.py:123-124 and
    additional_designs/attention/backends/aptserve_flash_attn.py:359-373) without materialising
    ``[T, 2*Hd]``.  ``kv_dest[t] >= 0``: slot of the workspace caches; ``<= -2``: slot
    ``-(kv_dest[t]+2)`` of the private caches; ``-1``: skipped.  Either cache pair may be ``None``
    when no row goes there."""
    dev = x.device
    _check_data("x", x, dev)
    _check_data("w_kv", w_kv, dev)
    _need(x.dim() == 2 and w_kv.dim() == 2 and x.size(1) == w_kv.size(1), "x [T,K] and w_kv [2*Hd,K] expected")
    _need(x.dtype == w_kv.dtype and x.dtype in (torch.float16, torch.bfloat16), "f16 or bf16 operands expected")
    T, K = x.shape
    _need(w_kv.size(0) % 2 == 0, "w_kv must stack the K and V projections")
    Hd = w_kv.size(0) // 2
    if b_kv is not None:
        _check_data("b_kv", b_kv, dev)
        _need(b_kv.dim() == 1 and b_kv.numel() == 2 * Hd and b_kv.dtype == x.dtype and b_kv.is_contiguous(),
              "b_kv must be a contiguous [2*Hd] vector of the operand dtype")
    _check_index("kv_dest", kv_dest, dev)
    _need(kv_dest.numel() == T, "one destination per row expected")
    slots = [0, 0]
    stride = None
    for i, (kc, vc, nm) in enumerate(((ws_k_cache, ws_v_cache, "workspace"), (k_cache, v_cache, "private"))):
        _need((kc is None) == (vc is None), f"{nm} K and V caches must be given together")
        if kc is None:
            continue
        for c in (kc, vc):
            _check_data(f"{nm} cache", c, dev)
            _need(c.dim() == 4 and c.is_contiguous() and c.dtype == x.dtype and c.size(2) * c.size(3) == Hd,
                  f"{nm} caches must be contiguous [blocks, BS, H, D] of the operand dtype with H*D = Hd")
        _need(kc.shape == vc.shape, f"{nm} K and V caches differ in shape")
        slots[i] = kc.size(0) * kc.size(1)
        stride = Hd
    _need(stride is not None, "no destination cache given")
    lib = _lib.load()
    need = lib.aps_linear_nt_workspace_bytes(T, 2 * Hd, K) if split_k else 0
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)     # scratch is host-side plumbing
    with _on(dev):
        st = lib.aps_kv_reproject_to_cache(
            x.data_ptr() if T else None, w_kv.data_ptr(), None if b_kv is None else b_kv.data_ptr(),
            _ptr(ws_k_cache), _ptr(ws_v_cache), _ptr(k_cache), _ptr(v_cache), _ptr(kv_dest), T, Hd, K, x.stride(0),
            w_kv.stride(0), stride, slots[0], slots[1], _DTYPE_CODE[x.dtype], workspace.data_ptr() if need else None,
            workspace.numel() * workspace.element_size() if need else 0, _stream(x))
    _lib.check(st, "kv_reproject_to_cache")


def kv_reproject_gathered(hidden_states, paged_cache, holder_src, w_kv, b_kv, ws_k_cache, ws_v_cache, k_cache,
                          v_cache, kv_dest, workspace=None, split_k: bool = True) -> None:
    """``kv_reproject_to_cache`` without the holder: row ``t`` of the product's left operand is read where it is
    cached (``holder_src[t] >= 0``: that slot of ``paged_cache``; ``-(b+1)``: row ``b`` of ``hidden_states``),
    so the sequence ``torch.zeros`` / index_put / ``cache_to_hidden`` of
    additional_designs/model_executor/models/aptserve_opt.py:112-121 and its ``[num_tot, Hd]`` tensor disappear.
    Rows without a source must have ``kv_dest == -1`` (the metadata builder writes them so).  Cache contents are
    bit-identical to ``gather_hidden_rows`` + ``kv_reproject_to_cache`` for more than 48 rows (the same tile
    kernel); with fewer rows that flow runs the weight-streaming kernels, which add in another order."""
    dev = hidden_states.device
    for n, t in (("hidden_states", hidden_states), ("paged_cache", paged_cache), ("w_kv", w_kv)):
        _check_data(n, t, dev)
    _need(hidden_states.dim() == 2 and w_kv.dim() == 2 and hidden_states.size(1) == w_kv.size(1),
          "hidden_states [B,K] and w_kv [2*Hd,K] expected")
    _need(hidden_states.dtype == w_kv.dtype == paged_cache.dtype and hidden_states.dtype in (torch.float16, torch.bfloat16),
          "f16 or bf16 operands and cache expected")
    K = hidden_states.size(1)
    _check_paged(paged_cache, K)
    _need(w_kv.size(0) % 2 == 0, "w_kv must stack the K and V projections")
    Hd = w_kv.size(0) // 2
    if b_kv is not None:
        _check_data("b_kv", b_kv, dev)
        _need(b_kv.dim() == 1 and b_kv.numel() == 2 * Hd and b_kv.dtype == w_kv.dtype and b_kv.is_contiguous(),
              "b_kv must be a contiguous [2*Hd] vector of the operand dtype")
    _check_index("holder_src", holder_src, dev)
    _check_index("kv_dest", kv_dest, dev)
    T = holder_src.numel()
    _need(kv_dest.numel() == T, "one destination per row expected")
    slots = [0, 0]
    stride = None
    for i, (kc, vc, nm) in enumerate(((ws_k_cache, ws_v_cache, "workspace"), (k_cache, v_cache, "private"))):
        _need((kc is None) == (vc is None), f"{nm} K and V caches must be given together")
        if kc is None:
            continue
        for c in (kc, vc):
            _check_data(f"{nm} cache", c, dev)
            _need(c.dim() == 4 and c.is_contiguous() and c.dtype == w_kv.dtype and c.size(2) * c.size(3) == Hd,
                  f"{nm} caches must be contiguous [blocks, BS, H, D] of the operand dtype with H*D = Hd")
        _need(kc.shape == vc.shape, f"{nm} K and V caches differ in shape")
        slots[i] = kc.size(0) * kc.size(1)
        stride = Hd
    _need(stride is not None, "no destination cache given")
    if T == 0:
        return
    lib = _lib.load()
    need = lib.aps_linear_nt_workspace_bytes(T, 2 * Hd, K) if (split_k and T > 48) else 0
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)     # scratch is host-side plumbing
    slot_stride = paged_cache.stride(2)
    with _on(dev):
        st = lib.aps_kv_reproject_gathered(
            paged_cache.data_ptr(), slot_stride, paged_cache.numel() // slot_stride, hidden_states.data_ptr(),
            hidden_states.stride(0), hidden_states.size(0), holder_src.data_ptr(), T, w_kv.data_ptr(),
            None if b_kv is None else b_kv.data_ptr(), _ptr(ws_k_cache), _ptr(ws_v_cache), _ptr(k_cache),
            _ptr(v_cache), kv_dest.data_ptr(), Hd, K, w_kv.stride(0), stride, slots[0], slots[1],
            _DTYPE_CODE[w_kv.dtype], workspace.data_ptr() if need else None,
            workspace.numel() * workspace.element_size() if need else 0, _stream(hidden_states))
    _lib.check(st, "kv_reproject_gathered")


# ------------------------------------------------------------------ prompt attention

def flash_attn_varlen_func(q, k, v, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=None, max_seqlen_k=None,
                           softmax_scale=None, causal: bool = True, window_size=None, alibi_slopes=None, out=None,
                           block_table=None):
    """Prompt-step cases of the third-party function with the keywords used at
    additional_designs/attention/backends/aptserve_flash_attn.py:414-426 and :435-447.

    Without ``block_table``: q, k and v are the packed, freshly projected ``[tokens, H, D]`` tensors of the
    same sequences (``cu_seqlens_q is cu_seqlens_k``), causal.  With ``block_table`` (int32 ``[seqs, W]``, the
    prefix branch): ``k`` / ``v`` are the ``[blocks, BS, H, D]`` K/V caches, ``cu_seqlens_k`` delimits the
    sequences' total lengths (cached prefix + this step's tokens, all of them already in the cache) and query
    ``j`` of a sequence attends to keys ``0 .. j + klen - qlen``.  Returns ``[tokens, H, D]``."""
    dev = q.device
    _need(causal, "only causal attention is provided")
    _need(alibi_slopes is None, "alibi_slopes is not supported")
    _need(window_size in (None, (-1, -1)), "sliding windows are not supported")
    _need(cu_seqlens_q is not None, "cu_seqlens_q is required")
    _check_data("q", q, dev)
    _need(q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == q.size(2), "q must be [tokens, heads, head_dim]")
    _need(q.dtype in (torch.float16, torch.bfloat16), "f16 or bf16 expected")
    _check_index("cu_seqlens_q", cu_seqlens_q, dev, torch.int32)
    T, H, D = q.shape
    n_seq = cu_seqlens_q.numel() - 1
    _need(n_seq >= 0, "cu_seqlens must have a leading 0")
    max_len = int(max_seqlen_q if max_seqlen_q is not None else (max_seqlen_k if max_seqlen_k is not None else T))
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    _need(0.0 < float(softmax_scale) < float("inf"), "softmax_scale must be positive and finite")
    if out is None:
        out = torch.empty(T, H, D, dtype=q.dtype, device=dev)
    else:
        _check_data("out", out, dev)
        _need(out.shape == q.shape and out.dtype == q.dtype and out.stride(2) == 1 and out.stride(1) == D,
              "out must look like q")
    if block_table is not None:
        for n, c in (("k", k), ("v", v)):
            _check_data(n, c, dev)
            _check_kv_cache(n, c, H, D)
            _need(c.dtype == q.dtype, "the prefix branch reads caches of the query dtype")
        _need(k.shape == v.shape and k.stride(0) == v.stride(0), "key and value cache layouts differ")
        _need(cu_seqlens_k is not None, "the prefix branch needs cu_seqlens_k")
        _check_index("cu_seqlens_k", cu_seqlens_k, dev, torch.int32)
        _need(cu_seqlens_k.numel() == n_seq + 1, "cu_seqlens_q and cu_seqlens_k must delimit the same sequences")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.size(0) == n_seq and
              block_table.device == dev and (block_table.size(1) <= 1 or block_table.stride(1) == 1),
              "block_table must be int32 [seqs, width] with contiguous rows on the same GPU")
        with _on(dev):
            st = _lib.load().aps_paged_prefill_attention(
                out.data_ptr() if T else None, q.data_ptr() if T else None, k.data_ptr(), v.data_ptr(),
                _ptr(block_table), _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), n_seq if T else 0, T, max_len, H, D,
                k.size(1), block_table.stride(0), block_table.size(1), q.stride(0), out.stride(0), k.stride(0),
                k.size(0), float(softmax_scale), _DTYPE_CODE[q.dtype], _stream(q))
        _lib.check(st, "flash_attn_varlen_func (prefix branch)")
        return out
    _need(cu_seqlens_k is None or cu_seqlens_k is cu_seqlens_q or torch.equal(cu_seqlens_k, cu_seqlens_q),
          "prompt attention needs identical query and key sequence boundaries")
    for n, t in (("k", k), ("v", v)):
        _check_data(n, t, dev)
        _need(t.dim() == 3 and t.shape == q.shape, f"{n} must be [tokens, heads, head_dim] like q")
        _need(t.stride(2) == 1 and t.stride(1) == t.size(2), f"{n}: heads of one token must be contiguous")
        _need(t.dtype == q.dtype, "q, k, v dtypes differ")
    with _on(dev):
        st = _lib.load().aps_varlen_prefill_attention(
            out.data_ptr() if T else None, q.data_ptr() if T else None, k.data_ptr() if T else None,
            v.data_ptr() if T else None, _ptr(cu_seqlens_q), n_seq if T else 0, T, max_len, H, D, q.stride(0),
            k.stride(0), v.stride(0), out.stride(0), float(softmax_scale), _DTYPE_CODE[q.dtype], _stream(q))
    _lib.check(st, "flash_attn_varlen_func")
    return out


# ------------------------------------------------------------------ attention on cached hidden rows

def absorbed_hidden_attention(q, paged_cache, hidden_slots, hidden_seq_start, seq_rows, max_len, w_k, w_v, b_v,
                              softmax_scale, out, workspace=None, kv_job: Optional["AttentionJob"] = None,
                              store_job: Optional["CacheJob"] = None):
    """Decode attention of the hidden-cached sequences of a batch, computed on their cached hidden
    rows with the K/V projection weights absorbed into the query and the output:
    ``s[h,t] = scale <W_k[h]^T q[h], hidden_t>``, ``out[h] = W_v[h] (sum_t p[h,t] hidden_t) + b_v[h]``.
    Equal (up to rounding) to re-projecting every row and attending over the result — the sequence
    of additional_designs/model_executor/models/aptserve_opt.py:112-124 and
    additional_designs/attention/backends/aptserve_flash_attn.py:359-373, :464-473 — without the
    gather, the re-projection GEMM and the K/V workspace.

    ``q [B, H*D]`` query rows of the batch; ``seq_rows`` (= ``hidden_cache_use_input``) batch
    positions of the hidden-cached sequences; ``hidden_slots`` / ``hidden_seq_start`` from the
    metadata builder; ``w_k``, ``w_v [H*D, H*D]`` row slices of the fused QKV weight; the result of
    sequence ``i`` is written to ``out[seq_rows[i]]`` (``out [B, H*D]``).  The newest hidden row of
    every sequence must already be in the cache.

    ``kv_job``: the paged decode attention of the batch's K/V-cached sequences
    (``paged_decode_attention(..., as_job=True)``), launched by this call as well — inside the
    launch of the weighted sum over the hidden rows when the batch is small enough for that, by
    itself otherwise; the results are those of launching the job alone.  ``store_job``: the step's
    cache writes (``decode_step_cache_ops(..., as_job=True)``), complete before any cache row is
    read: beside the absorbed queries in one launch when they fit there, first and by themselves
    otherwise."""
    dev = q.device
    for n, t in (("q", q), ("paged_cache", paged_cache), ("w_k", w_k), ("w_v", w_v), ("out", out)):
        _check_data(n, t, dev)
    _need(paged_cache.dim() == 5 and paged_cache.is_contiguous(), "paged_cache must be contiguous (2, N, BS, H, D)")
    heads, head_size = paged_cache.size(3), paged_cache.size(4)
    hidden = heads * head_size
    _need(q.dim() == 2 and q.size(1) == hidden and out.dim() == 2 and out.size(1) == hidden,
          "q and out must be [rows, heads*head_dim]")
    _need(w_k.dim() == 2 and w_k.shape == (hidden, hidden) and w_v.shape == (hidden, hidden),
          "w_k and w_v must be [H*D, H*D]")
    _need(w_k.stride(0) == w_v.stride(0), "w_k and w_v must have the same row stride")
    _need(q.dtype in (torch.float16, torch.bfloat16), "f16 or bf16 expected")
    _need(all(t.dtype == q.dtype for t in (paged_cache, w_k, w_v, out)), "dtypes differ")
    if b_v is not None:
        _check_data("b_v", b_v, dev)
        _need(b_v.dim() == 1 and b_v.numel() == hidden and b_v.dtype == q.dtype and b_v.is_contiguous(),
              "b_v must be a contiguous [H*D] vector of the operand dtype")
    for n, t in (("hidden_slots", hidden_slots), ("hidden_seq_start", hidden_seq_start), ("seq_rows", seq_rows)):
        _check_index(n, t, dev)
    n_seqs = seq_rows.numel()
    _need(hidden_seq_start.numel() == n_seqs + 1, "hidden_seq_start needs one entry per sequence plus one")
    if n_seqs == 0:
        if store_job is not None:
            store_job.launch()
        if kv_job is not None:
            kv_job.launch()
        return out
    lib = _lib.load()
    need = lib.aps_absorbed_attention_workspace_bytes(n_seqs, int(max_len), heads, head_size)
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)      # scratch is host-side plumbing
    with _on(dev):
        st = lib.aps_hybrid_decode_attention(
            None if store_job is None else store_job.address, None if kv_job is None else kv_job.address, q.data_ptr(), q.stride(0), seq_rows.data_ptr(), q.size(0), paged_cache.data_ptr(), paged_cache.stride(2),
            paged_cache.numel() // paged_cache.stride(2), hidden_slots.data_ptr(), hidden_seq_start.data_ptr(),
            n_seqs, int(max_len), w_k.data_ptr(), w_v.data_ptr(), None if b_v is None else b_v.data_ptr(),
            w_k.stride(0), heads, head_size, float(softmax_scale), out.data_ptr(), out.stride(0), out.size(0),
            _DTYPE_CODE[q.dtype], workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream(q))
    _lib.check(st, "absorbed_hidden_attention")
    return out


# ------------------------------------------------------------------ residual add + LayerNorm

def add_layer_norm(x, residual, weight, bias, eps: float = 1e-5, out=None, sum_out=None):
    """``s = x + residual`` (rounded to the activation dtype; ``residual`` may be ``None``) and
    ``LayerNorm(s) * weight + bias`` in one launch: the residual add and the LayerNorm that follows it in
    ``OPTDecoderLayer.forward`` (additional_designs/model_executor/models/aptserve_opt.py:186-211).
    Returns ``(normed, s)``; ``s`` is ``x`` itself when there is no residual."""
    dev = x.device
    _check_data("x", x, dev)
    _need(x.dim() == 2 and x.dtype in (torch.float16, torch.bfloat16), "x must be a 2-D f16 or bf16 tensor")
    rows, width = x.shape
    for n, t in (("weight", weight), ("bias", bias)):
        if t is not None:
            _check_data(n, t, dev)
            _need(t.dim() == 1 and t.numel() == width and t.dtype == x.dtype and t.is_contiguous(),
                  f"{n} must be a contiguous [width] vector of x's dtype")
    _need(weight is not None, "weight is required")
    if residual is not None:
        _check_data("residual", residual, dev)
        _need(residual.shape == x.shape and residual.dtype == x.dtype, "residual must look like x")
    if out is None:
        out = torch.empty(rows, width, dtype=x.dtype, device=dev)
    if residual is not None and sum_out is None:
        sum_out = torch.empty(rows, width, dtype=x.dtype, device=dev)
    for n, t in (("out", out), ("sum_out", sum_out)):
        if t is not None:
            _check_data(n, t, dev)
            _need(t.shape == x.shape and t.dtype == x.dtype, f"{n} must look like x")
    with _on(dev):
        st = _lib.load().aps_add_layer_norm(
            _ptr(out), None if residual is None else _ptr(sum_out), _ptr(x), _ptr(residual), _ptr(weight), _ptr(bias),
            rows, width, x.stride(0), 0 if residual is None else residual.stride(0), out.stride(0),
            0 if residual is None or sum_out is None else sum_out.stride(0), float(eps), _DTYPE_CODE[x.dtype],
            _stream(x))
    _lib.check(st, "add_layer_norm")
    return out, (x if residual is None else sum_out)


# ------------------------------------------------------------------ block maintenance

_LAYER_BASES = {}


def _layer_bases(kv_caches, dev):
    """Device vector of the layer caches' base addresses.  The caches of a model live as long as its engine, so
    the vector is uploaded once per set of caches and not with a blocking copy in every call."""
    key = (dev.index, tuple(c.data_ptr() for c in kv_caches))
    bases = _LAYER_BASES.get(key)
    if bases is None:
        if len(_LAYER_BASES) >= 16:
            _LAYER_BASES.clear()
        bases = torch.tensor(key[1], dtype=torch.int64).to(dev)
        _LAYER_BASES[key] = bases
    return bases


def copy_blocks(kv_caches, src_to_dsts, kinds=None) -> None:
    """``FlashAttentionBackend.copy_blocks`` (additional_designs/attention/backends/aptserve_flash_attn.py:58-65)
    for the caches of all layers in one launch; ``src_to_dsts`` int64 ``[n, 2]`` on the device.
    ``kinds`` (uint8 ``[n]``, optional): 1 marks a hidden block, whose ids run over the ``2N`` plane
    slabs of a cache; 0 (default) a K/V block, both planes of block id ``< N``."""
    if not kv_caches:
        return
    c0 = kv_caches[0]
    dev = c0.device
    for c in kv_caches:
        _check_data("kv_cache", c, dev)
        _need(c.dim() == 5 and c.size(0) == 2 and c.is_contiguous() and c.shape == c0.shape and c.dtype == c0.dtype,
              "every layer cache must be a contiguous (2, N, BS, H, D) tensor of the same shape and dtype")
    _need(src_to_dsts.device == dev and src_to_dsts.dtype == torch.int64 and src_to_dsts.dim() == 2
          and src_to_dsts.size(1) == 2 and src_to_dsts.is_contiguous(), "src_to_dsts must be a contiguous int64 [n, 2] tensor")
    n = src_to_dsts.size(0)
    if kinds is not None:
        _need(kinds.device == dev and kinds.dtype in (torch.uint8, torch.bool) and kinds.is_contiguous()
              and kinds.numel() == n, "kinds must be a contiguous uint8/bool vector, one entry per pair")
    if n == 0:
        return
    bases = _layer_bases(kv_caches, dev)
    _, N, BS, H, D = c0.shape
    with _on(dev):
        st = _lib.load().aps_copy_cache_blocks(bases.data_ptr(), len(kv_caches), src_to_dsts.data_ptr(), _ptr(kinds), n,
                                               N, BS, H * D, c0.element_size(), _stream(c0))
    _lib.check(st, "copy_blocks")


def swap_blocks(src_kv_cache, dst_kv_cache, src_to_dst, kinds=None) -> None:
    """``FlashAttentionBackend.swap_blocks`` (aptserve_flash_attn.py:44-56): copies blocks of one layer between
    two caches (GPU and pinned host memory in the reference's swap-in / swap-out,
    additional_designs/worker/aptserve_cache_engine.py:88-96).  ``src_to_dst`` is a HOST int64 ``[n, 2]``
    tensor as in the reference; ``kinds`` a host uint8 ``[n]`` vector (1 = hidden block, ids over the ``2N``
    plane slabs)."""
    for c in (src_kv_cache, dst_kv_cache):
        _need(c.dim() == 5 and c.size(0) == 2 and c.is_contiguous(), "caches must be contiguous (2, N, BS, H, D)")
    _need(src_kv_cache.shape[2:] == dst_kv_cache.shape[2:] and src_kv_cache.dtype == dst_kv_cache.dtype,
          "source and destination blocks differ in shape or dtype")
    _need(src_kv_cache.is_cuda or dst_kv_cache.is_cuda, "one of the caches must live on the GPU")
    for c in (src_kv_cache, dst_kv_cache):
        _need(c.is_cuda or c.is_pinned(), "a host cache must be pinned memory")
    _need(src_to_dst.device.type == "cpu" and src_to_dst.dtype == torch.int64 and src_to_dst.dim() == 2
          and src_to_dst.size(1) == 2 and src_to_dst.is_contiguous(), "src_to_dst must be a host int64 [n, 2] tensor")
    n = src_to_dst.size(0)
    if kinds is not None:
        _need(kinds.device.type == "cpu" and kinds.dtype in (torch.uint8, torch.bool) and kinds.numel() == n
              and kinds.is_contiguous(), "kinds must be a host uint8/bool vector, one entry per pair")
    if n == 0:
        return
    gpu = src_kv_cache if src_kv_cache.is_cuda else dst_kv_cache
    block_bytes = src_kv_cache[0, 0].numel() * src_kv_cache.element_size()
    with torch.cuda.device(gpu.device):
        st = _lib.load().aps_swap_cache_blocks(src_kv_cache.data_ptr(), dst_kv_cache.data_ptr(), src_to_dst.data_ptr(),
                                               None if kinds is None else kinds.data_ptr(), n, src_kv_cache.size(1),
                                               dst_kv_cache.size(1), block_bytes, _stream(gpu))
    _lib.check(st, "swap_blocks")


# ------------------------------------------------------------------ names of the operator surface

def gather_hidden_blocks(holder, paged_cache, slot_mapping, dst_idx) -> None:
    """Hidden-block gather into a contiguous ``[T, Hd]`` buffer: ``cache_to_hidden`` under the name
    the operator surface uses for it."""
    cache_to_hidden(holder, paged_cache, slot_mapping, dst_idx)


def paged_hybrid_attention(q, kv_cache, kv_workspace, block_tables, block_types, seq_lens, scale=None,
                           kv_scale=None, **kw):
    """Decode attention over a cache whose blocks hold either K/V (read from the layer's
    ``kv_cache (2, N, BS, H, D)``) or re-projected hidden states (read from ``kv_workspace
    (2, M, BS, H, D)``), chosen per block by ``block_types`` (uint8, 1 = workspace).
    ``kv_scale``: per-tensor scale of an fp8 cache (one float, or a ``(k_scale, v_scale)`` pair)."""
    if kv_scale is not None:
        ks, vs = (kv_scale if isinstance(kv_scale, (tuple, list)) else (kv_scale, kv_scale))
        kw.update(k_scale=float(ks), v_scale=float(vs))
    ws_k = ws_v = None
    if kv_workspace is not None:
        ws_k, ws_v = kv_workspace[0], kv_workspace[1]
    return paged_decode_attention(q, kv_cache[0], kv_cache[1], block_tables, seq_lens, scale,
                                  block_types=block_types if kv_workspace is not None else None,
                                  ws_k_cache=ws_k, ws_v_cache=ws_v, **kw)


def build_hybrid_metadata(*args, **kwargs):
    """``aptserve_hip.metadata.build_metadata`` (GPU-side construction of the ragged-batch metadata)."""
    from . import metadata
    return metadata.build_metadata(*args, **kwargs)
