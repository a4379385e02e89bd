"""Host side of the ragged-batch metadata: the dataclass the attention backend
reads and the builder that fills it on the GPU.

``HybridAttentionMetadata`` carries the fields of the reference's
``AttentionMetadata`` (additional_designs/attention/backends/aptserve_abstract.py:56-80)
and ``FlashAttentionMetadata`` (additional_designs/attention/backends/aptserve_flash_attn.py:68-222)
under the same names, including the ``prefill_metadata`` / ``decode_metadata`` views.

``build_metadata`` replaces the list-building loop and the ~15 small
host-to-device copies of ``ModelRunner._prepare_model_input``
(additional_designs/worker/aptserve_model_runner.py:240-842): the host sums
O(batch) integers to size the outputs, uploads ONE packed int32 buffer
(lengths, cache-type flags, block tables) and one kernel expands everything
that scales with the number of cached tokens.
"""

from __future__ import annotations

import contextlib
import itertools
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from . import _lib


@dataclass
class HybridAttentionMetadata:
    # aptserve_abstract.py:56-80
    num_prefills: int
    num_prefill_tokens: int
    num_decode_tokens: int
    num_hidden_cache_tokens: int
    num_tot_tokens: int
    slot_mapping: torch.Tensor
    slot_mapping_shared: torch.Tensor
    hidden_cache_use_tot: torch.Tensor
    kv_cache_use_tot: torch.Tensor
    hidden_cache_use_input: torch.Tensor
    hidden_cache_store_tot: torch.Tensor
    hidden_holder_upd: torch.Tensor
    hidden_holder_pull: torch.Tensor
    # aptserve_flash_attn.py:76-121
    seq_lens: Optional[List[int]]
    seq_lens_tensor: Optional[torch.Tensor]
    max_query_len: Optional[int]
    max_prefill_seq_len: int
    max_decode_seq_len: int
    query_start_loc: Optional[torch.Tensor]
    seq_start_loc: Optional[torch.Tensor]
    context_lens_tensor: Optional[torch.Tensor]
    block_tables: Optional[torch.Tensor]
    use_cuda_graph: bool = False
    # additions of this implementation
    input_positions: Optional[torch.Tensor] = None
    block_types: Optional[torch.Tensor] = None      # uint8 [batch, width]: 1 = block read from the K/V workspace
    holder_src: Optional[torch.Tensor] = None       # int64 [num_tot]: resolved source of every holder row
    kv_dest: Optional[torch.Tensor] = None          # int64 [num_tot]: cache slot the row's re-projected K/V go to
    token_is_hidden: Optional[torch.Tensor] = None  # uint8 [prompt tokens]: 1 = token of a hidden-cached prompt
    hidden_slots: Optional[torch.Tensor] = None     # int64 [hidden rows]: private slot of every cached hidden row
    hidden_seq_start: Optional[torch.Tensor] = None  # int64 [hidden seqs + 1]: first hidden row of each hidden sequence
    max_hidden_seq_len: int = 0
    kv_cache_use_input: Optional[torch.Tensor] = None   # int64 [kv seqs]: batch positions of K/V-cached sequences
    new_token_slot: Optional[torch.Tensor] = None       # int64 [batch]: private slot of every sequence's newest token
    kv_seq_lens: Optional[torch.Tensor] = None          # int32 [batch]: seq_len, 0 for hidden-cached sequences
    max_kv_seq_len: int = 0
    private_block_tables: Optional[torch.Tensor] = None  # int32 [batch, W]: every sequence's private table
    max_prompt_context_len: int = 0   # longest already-cached prefix of a prompt step (0: plain prompts)
    _row_slots: Optional[tuple] = None
    _cached_prefill_metadata: Optional["HybridAttentionMetadata"] = None
    _cached_decode_metadata: Optional["HybridAttentionMetadata"] = None

    def row_slots_by_destination(self):
        """Two slot vectors indexed like the rows of a decode step, derived from ``kv_dest`` (cached): the
        workspace slot of every row of a hidden-cached sequence (-1 elsewhere) and the private slot of the
        newest token of every K/V-cached sequence (-1 elsewhere) — what ``reshape_and_cache_flash`` needs to
        send each kind of row to its cache."""
        if self._row_slots is None:
            d = self.kv_dest
            self._row_slots = (torch.where(d >= 0, d, -1), torch.where(d <= -2, -(d + 2), -1))
        return self._row_slots

    @property
    def prefill_metadata(self) -> Optional["HybridAttentionMetadata"]:
        """aptserve_flash_attn.py:126-175: slices by ``num_prefills`` / ``num_prefill_tokens``;
        the hybrid fields pass through unsliced."""
        if self.num_prefills == 0:
            return None
        if self._cached_prefill_metadata is None:
            self._cached_prefill_metadata = HybridAttentionMetadata(
                num_prefills=self.num_prefills, num_prefill_tokens=self.num_prefill_tokens, num_decode_tokens=0,
                num_hidden_cache_tokens=self.num_hidden_cache_tokens, num_tot_tokens=self.num_tot_tokens,
                slot_mapping=self.slot_mapping[:self.num_prefill_tokens],
                slot_mapping_shared=self.slot_mapping_shared, hidden_cache_use_tot=self.hidden_cache_use_tot,
                kv_cache_use_tot=self.kv_cache_use_tot, hidden_cache_use_input=self.hidden_cache_use_input,
                hidden_cache_store_tot=self.hidden_cache_store_tot, hidden_holder_upd=self.hidden_holder_upd,
                hidden_holder_pull=self.hidden_holder_pull, seq_lens=self.seq_lens[:self.num_prefills],
                seq_lens_tensor=self.seq_lens_tensor[:self.num_prefills], max_query_len=self.max_query_len,
                max_prefill_seq_len=self.max_prefill_seq_len, max_decode_seq_len=0,
                query_start_loc=self.query_start_loc[:self.num_prefills + 1],
                seq_start_loc=self.seq_start_loc[:self.num_prefills + 1],
                context_lens_tensor=self.context_lens_tensor[:self.num_prefills],
                block_tables=self.block_tables[:self.num_prefills], use_cuda_graph=False,
                input_positions=self.input_positions, block_types=None, token_is_hidden=self.token_is_hidden,
                max_prompt_context_len=self.max_prompt_context_len)
        return self._cached_prefill_metadata

    @property
    def decode_metadata(self) -> Optional["HybridAttentionMetadata"]:
        """aptserve_flash_attn.py:177-221."""
        if self.num_decode_tokens == 0:
            return None
        if self._cached_decode_metadata is None:
            self._cached_decode_metadata = HybridAttentionMetadata(
                num_prefills=0, num_prefill_tokens=0, num_decode_tokens=self.num_decode_tokens,
                num_hidden_cache_tokens=self.num_hidden_cache_tokens, num_tot_tokens=self.num_tot_tokens,
                slot_mapping=self.slot_mapping[self.num_prefill_tokens:],
                slot_mapping_shared=self.slot_mapping_shared, hidden_cache_use_tot=self.hidden_cache_use_tot,
                kv_cache_use_tot=self.kv_cache_use_tot, hidden_cache_use_input=self.hidden_cache_use_input,
                hidden_cache_store_tot=self.hidden_cache_store_tot, hidden_holder_upd=self.hidden_holder_upd,
                hidden_holder_pull=self.hidden_holder_pull, seq_lens=None,
                seq_lens_tensor=self.seq_lens_tensor[self.num_prefills:], max_query_len=None,
                max_prefill_seq_len=0, max_decode_seq_len=self.max_decode_seq_len, query_start_loc=None,
                seq_start_loc=None, context_lens_tensor=None, block_tables=self.block_tables[self.num_prefills:],
                use_cuda_graph=self.use_cuda_graph, input_positions=self.input_positions,
                block_types=None if self.block_types is None else self.block_types[self.num_prefills:],
                holder_src=self.holder_src, kv_dest=self.kv_dest, hidden_slots=self.hidden_slots,
                hidden_seq_start=self.hidden_seq_start, max_hidden_seq_len=self.max_hidden_seq_len,
                kv_cache_use_input=self.kv_cache_use_input, new_token_slot=self.new_token_slot,
                kv_seq_lens=self.kv_seq_lens, max_kv_seq_len=self.max_kv_seq_len,
                private_block_tables=self.private_block_tables)
        return self._cached_decode_metadata


class _Staging:
    """Ring of pinned int32 staging buffers for the packed upload.  A buffer is
    reused only after the copy that last read it has completed (its event)."""

    def __init__(self, depth: int = 4):
        self.bufs = [None] * depth
        self.events = [None] * depth
        self.next = 0

    def take(self, n: int):
        i = self.next
        self.next = (i + 1) % len(self.bufs)
        if self.events[i] is not None:
            self.events[i].synchronize()
        if self.bufs[i] is None or self.bufs[i].numel() < n:
            self.bufs[i] = torch.empty(max(n, 4096), dtype=torch.int32, pin_memory=True)
        return i, self.bufs[i][:n]

    def upload(self, i: int, host: torch.Tensor, device, stream) -> torch.Tensor:
        dev = host.to(device, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record(stream)
        self.events[i] = ev
        return dev


    def upload_into(self, i: int, host: torch.Tensor, dst: torch.Tensor, stream) -> torch.Tensor:
        """Like ``upload`` into device memory the caller keeps (same address in every step)."""
        dst.copy_(host, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record(stream)
        self.events[i] = ev
        return dst


class StaticDecodeBuffers:
    """Device storage for the metadata of decode steps of one shape class: ``batch`` sequences of which
    ``n_hidden`` are hidden-cached, none longer than ``cap_len`` tokens.  ``build_metadata(..., static=this)``
    writes every step's metadata to the same addresses, which is what lets a step that was recorded into a HIP
    graph be replayed on the next step's batch."""

    def __init__(self, batch: int, n_hidden: int, cap_len: int, block_size: int, device) -> None:
        if cap_len % block_size:
            raise ValueError("cap_len must be a whole number of blocks")
        self.batch, self.n_hidden, self.cap_len, self.block_size = batch, n_hidden, cap_len, block_size
        self.device = torch.device(device)
        self.width = cap_len // block_size
        self.cap_hidden_rows = n_hidden * cap_len
        self.cap_rows = self.cap_hidden_rows + (batch - n_hidden)
        self.packed = torch.zeros(2 * batch + 2 * batch * self.width, dtype=torch.int32, device=self.device)
        self._b64 = self._b32 = None

    def check(self, batch: int, n_hidden: int, max_len: int, block_size: int, device) -> None:
        if (batch, n_hidden, block_size) != (self.batch, self.n_hidden, self.block_size) or max_len > self.cap_len \
                or torch.device(device) != self.device:
            raise ValueError("this batch does not fit the static metadata buffers (batch size, number of "
                             "hidden-cached sequences, block size and device must match; lengths must not exceed "
                             f"{self.cap_len})")

    def take64(self, n: int) -> torch.Tensor:
        if self._b64 is None:
            self._b64 = torch.zeros(n, dtype=torch.int64, device=self.device)
        if self._b64.numel() != n:
            raise RuntimeError("static metadata layout changed")
        return self._b64

    def take32(self, n: int) -> torch.Tensor:
        if self._b32 is None:
            self._b32 = torch.zeros(n, dtype=torch.int32, device=self.device)
        if self._b32.numel() != n:
            raise RuntimeError("static metadata layout changed")
        return self._b32


_staging = {}


def _stage(device, n: int, zero: bool = True):
    st = _staging.setdefault(device, _Staging())
    i, host = st.take(n)
    if zero:                       # ragged lists leave the padding untouched; packed arrays overwrite everything
        host.zero_()
    return st, i, host


def _table_lens(tables, need_blocks=None) -> np.ndarray:
    """Entries per table.  A packed ``[B, W]`` array carries no lengths: every table is then taken to be exactly
    as long as its sequence needs (what a block manager that grows tables one block at a time produces), or
    empty when the array has no columns."""
    if isinstance(tables, np.ndarray):
        if tables.ndim != 2:
            raise ValueError("packed block tables must be a [batch, width] array")
        if tables.shape[1] == 0 or need_blocks is None:
            return np.zeros(tables.shape[0], dtype=np.int64)
        if int(need_blocks.max()) > tables.shape[1]:
            raise ValueError("packed block table narrower than ceil(seq_len/block_size)")
        return need_blocks.astype(np.int64)
    return np.fromiter(map(len, tables), dtype=np.int64, count=len(tables))


def _pack_tables(tables, lens: np.ndarray, out: np.ndarray, rows: Optional[np.ndarray] = None) -> None:
    """Ragged lists -> 0-padded ``out[B, W]`` with one flat copy instead of a Python loop per row.  A packed
    ``[B, >=W]`` int array is copied as it is (``rows``: boolean mask of the tables that count, the others are
    left empty)."""
    if isinstance(tables, np.ndarray):       # 0-padded by contract: one block copy
        w = min(out.shape[1], tables.shape[1])
        out[:, :w] = tables[:, :w]
        out[:, w:] = 0
        if rows is not None:
            out[~rows] = 0
        return
    total = int(lens.sum())
    if total == 0:
        return
    flat = np.fromiter(itertools.chain.from_iterable(tables), dtype=np.int32, count=total)
    starts = np.cumsum(lens) - lens
    rows = np.repeat(np.arange(len(tables)), lens)
    cols = np.arange(total) - np.repeat(starts, lens)
    out[rows, cols] = flat


def build_metadata(is_prompt: bool, seq_lens: Sequence[int], use_hidden: Sequence[bool],
                   block_tables: Sequence[Sequence[int]], block_tables_4_shared: Sequence[Sequence[int]],
                   block_size: int, device, context_lens: Optional[Sequence[int]] = None,
                   check_totals: bool = False, static: Optional["StaticDecodeBuffers"] = None
                   ) -> HybridAttentionMetadata:
    """Build the metadata of one homogeneous batch (all prompts or all decodes, as the
    reference's scheduler emits them, additional_designs/core/aptserve_scheduler.py:1613-1625).

    ``block_tables[b]`` is sequence b's private table, ``block_tables_4_shared[b]`` its
    shared (workspace) table (empty for K/V-cached sequences).  An empty private table
    (the memory-profiling run) yields padding slots.

    Tables may be lists of lists (what the reference's scheduler hands over) or packed, 0-padded
    ``[batch, width]`` int arrays that the caller keeps up to date between steps: flattening ~10 k Python
    integers of a 256-sequence batch costs more host time than everything else in this function together.

    ``static`` (decode steps only): persistent device buffers of fixed capacity (:class:`StaticDecodeBuffers`).
    The metadata is built into them, at the same addresses in every step, and the row-indexed fields come back
    at their capacity instead of the step's own length (entries past the step's rows are never referenced) —
    what a step recorded into a HIP graph needs.
    """
    device = torch.device(device)
    B = len(seq_lens)
    if B == 0:
        raise ValueError("empty batch")
    lens = np.asarray(seq_lens, dtype=np.int64)
    hid = np.asarray(use_hidden, dtype=bool)
    if len(hid) != B or len(block_tables) != B:
        raise ValueError("seq_lens, use_hidden and block_tables must have one entry per sequence")
    if np.any(lens <= 0):
        raise ValueError("sequence lengths must be positive")
    need_blocks = -(-lens // block_size)
    max_len = int(lens.max())
    # packed arrays carry no lengths of their own: every table is as long as its sequence needs, so the checks
    # and reductions the ragged lists need fall away
    arrays = isinstance(block_tables, np.ndarray)
    bt_lens = _table_lens(block_tables, need_blocks)
    if arrays:
        have_tables = block_tables.shape[1] > 0
        W = -(-max_len // block_size) if have_tables else 0
    else:
        have_tables = bool(bt_lens.any())
        W = int(bt_lens.max()) if have_tables else 0
        if have_tables and np.any(bt_lens < need_blocks):
            b = int(np.nonzero(bt_lens < need_blocks)[0][0])
            raise ValueError(f"sequence {b}: private block table shorter than ceil(seq_len/block_size)")
    lib = _lib.load()
    i64 = dict(dtype=torch.int64, device=device)
    i32 = dict(dtype=torch.int32, device=device)
    stream = torch.cuda.current_stream(device)
    on_device = (contextlib.nullcontext() if torch.cuda.current_device() == stream.device_index
                 else torch.cuda.device(device))

    if not is_prompt:
        if len(block_tables_4_shared) != B:
            raise ValueError("block_tables_4_shared must have one entry per sequence")
        n_hs = int(np.count_nonzero(hid))
        n_kv = B - n_hs
        hid_lens = lens[hid]
        n_hr = int(hid_lens.sum())
        num_tot = n_hr + n_kv
        max_hid_len = int(hid_lens.max()) if n_hs else 0
        shared_arrays = isinstance(block_tables_4_shared, np.ndarray)
        if arrays and shared_arrays:
            bts_lens = None
            if have_tables and n_hs and -(-max_hid_len // block_size) > block_tables_4_shared.shape[1]:
                raise ValueError("packed block table narrower than ceil(seq_len/block_size)")
            Ws = -(-max_hid_len // block_size) if (have_tables and n_hs) else 0
            Wo = W            # both tables are exactly as long as their sequences need
        else:
            bts_lens = _table_lens(block_tables_4_shared, need_blocks * hid) * hid   # K/V-cached sequences: ignored
            if have_tables and np.any(bts_lens[hid] < need_blocks[hid]):
                b = int(np.nonzero(hid & (bts_lens < need_blocks))[0][0])
                raise ValueError(f"sequence {b}: shared block table shorter than ceil(seq_len/block_size)")
            Ws = int(bts_lens.max()) if (have_tables and n_hs) else 0
            # width of the table handed to attention: the longest *selected* table (:601-609)
            Wo = int(np.where(hid, bts_lens, bt_lens).max()) if have_tables else 0
        if static is not None:
            static.check(B, n_hs, max_len, block_size, device)
            if have_tables:
                W = Wo = static.width
                Ws = static.width if n_hs else 0
        # one packed upload: lens | flags | private tables | shared tables
        stg, slot, host = _stage(device, 2 * B + B * W + B * Ws,
                                 zero=static is not None or not (arrays and (Ws == 0 or shared_arrays)))
        hv = host.numpy()
        hv[:B] = lens
        hv[B:2 * B] = hid
        if W:
            _pack_tables(block_tables, bt_lens, hv[2 * B:2 * B + B * W].reshape(B, W))
        if Ws:
            if isinstance(block_tables_4_shared, np.ndarray):
                _pack_tables(block_tables_4_shared, bts_lens, hv[2 * B + B * W:].reshape(B, Ws), rows=hid)
            else:
                shared = [t if h else () for t, h in zip(block_tables_4_shared, hid)]
                _pack_tables(shared, bts_lens, hv[2 * B + B * W:].reshape(B, Ws))
        if static is None:
            packed = stg.upload(slot, host, device, stream)
        else:
            packed = stg.upload_into(slot, host, static.packed[:host.numel()], stream)
            # capacities in place of this step's row counts: same buffer layout in every step
            num_tot_step, num_tot, n_hr = num_tot, static.cap_rows, static.cap_hidden_rows
        d_lens, d_hid = packed[:B], packed[B:2 * B]
        d_bt = packed[2 * B:2 * B + B * W].view(B, W)
        d_bts = packed[2 * B + B * W:].view(B, Ws)
        # one allocation per output dtype
        sizes64 = [num_tot, n_hr, n_hr, n_kv, n_hs, n_hs, B, num_tot - B, B, 4, num_tot, num_tot, n_hr, n_hs + 1,
                   n_kv, B]
        buf64 = torch.empty(sum(sizes64), **i64) if static is None else static.take64(sum(sizes64))
        (slot_mapping, slot_mapping_shared, use_tot, kv_use, use_input, store_tot, upd, pull, positions,
         totals, holder_src, kv_dest, hidden_slots, hidden_seq_start, kv_use_input,
         new_token_slot) = torch.split(buf64, sizes64)
        n_types = (B * Wo + 3) // 4 if (n_hs and Wo) else 0          # uint8 [B, Wo] carried in the int32 buffer
        sizes32 = [B * Wo, B + 1, B + 1, B, B, n_types]
        buf32 = torch.empty(sum(sizes32), **i32) if static is None else static.take32(sum(sizes32))
        bt_out, seq_start, query_start, ctx, kv_seq_lens, types32 = torch.split(buf32, sizes32)
        bt_out = bt_out.view(B, Wo)
        # per-block source for the hybrid attention: every block of a hidden sequence is a workspace block
        block_types = types32.view(torch.uint8)[:B * Wo].view(B, Wo) if n_types else None
        with on_device:
            st = lib.aps_build_decode_metadata(
                d_lens.data_ptr(), d_hid.data_ptr(), d_bt.data_ptr() if W else None, W, W,
                d_bts.data_ptr() if Ws else None, Ws, Ws, B, block_size, slot_mapping.data_ptr(),
                slot_mapping_shared.data_ptr() if n_hr else None, use_tot.data_ptr() if n_hr else None,
                kv_use.data_ptr() if n_kv else None, use_input.data_ptr() if n_hs else None,
                store_tot.data_ptr() if n_hs else None, upd.data_ptr(), pull.data_ptr() if num_tot > B else None,
                holder_src.data_ptr(), kv_dest.data_ptr(), hidden_slots.data_ptr() if n_hr else None,
                hidden_seq_start.data_ptr() if n_hs else None, kv_use_input.data_ptr() if n_kv else None,
                new_token_slot.data_ptr(), kv_seq_lens.data_ptr(), num_tot, n_hr, n_hs, n_kv,
                bt_out.data_ptr() if Wo else None, Wo, Wo,
                None if block_types is None else block_types.data_ptr(), seq_start.data_ptr(),
                query_start.data_ptr(), ctx.data_ptr(), positions.data_ptr(), totals.data_ptr(),
                stream.cuda_stream)
        _lib.check(st, "build_decode_metadata")
        if static is not None:
            num_tot, n_hr = num_tot_step, int(hid_lens.sum())
            max_len = max_hid_len = static.cap_len      # host-side bounds that stay put while the bucket lasts
        if check_totals:
            got = totals.tolist()
            if got != [num_tot, n_hr, n_hs, n_kv]:
                raise RuntimeError(f"device totals {got} disagree with the host's {[num_tot, n_hr, n_hs, n_kv]}")
        return HybridAttentionMetadata(
            num_prefills=0, num_prefill_tokens=0, num_decode_tokens=B, num_hidden_cache_tokens=n_hs,
            num_tot_tokens=num_tot, slot_mapping=slot_mapping, slot_mapping_shared=slot_mapping_shared,
            hidden_cache_use_tot=use_tot, kv_cache_use_tot=kv_use, hidden_cache_use_input=use_input,
            hidden_cache_store_tot=store_tot, hidden_holder_upd=upd, hidden_holder_pull=pull,
            seq_lens=lens.tolist(), seq_lens_tensor=d_lens, max_query_len=1, max_prefill_seq_len=0,
            max_decode_seq_len=max_len, query_start_loc=query_start, seq_start_loc=seq_start,
            context_lens_tensor=ctx, block_tables=bt_out, use_cuda_graph=False, input_positions=positions,
            block_types=block_types, holder_src=holder_src, kv_dest=kv_dest, hidden_slots=hidden_slots,
            hidden_seq_start=hidden_seq_start, max_hidden_seq_len=max_hid_len,
            kv_cache_use_input=kv_use_input, new_token_slot=new_token_slot, kv_seq_lens=kv_seq_lens,
            max_kv_seq_len=(max_len if static is not None else int(lens[~hid].max())) if n_kv else 0,
            private_block_tables=d_bt)

    # ------------------------------------------------------------------ prompts
    ctxs = np.zeros(B, dtype=np.int64) if context_lens is None else np.asarray(context_lens, dtype=np.int64)
    qlens = lens - ctxs
    if np.any(qlens <= 0):
        raise ValueError("every prompt needs at least one new token")
    n_tok = int(qlens.sum())
    n_ht = int(qlens[hid].sum())
    n_kt = n_tok - n_ht
    stg, slot, host = _stage(device, 3 * B + B * W)
    hv = host.numpy()
    hv[:B] = lens
    hv[B:2 * B] = hid
    hv[2 * B:3 * B] = ctxs
    if W:
        _pack_tables(block_tables, bt_lens, hv[3 * B:].reshape(B, W))
    packed = stg.upload(slot, host, device, stream)
    d_lens, d_hid, d_ctx_in = packed[:B], packed[B:2 * B], packed[2 * B:3 * B]
    d_bt = packed[3 * B:].view(B, W)
    sizes64 = [n_tok, n_tok, n_ht, n_kt, 4]
    buf64 = torch.empty(sum(sizes64), **i64)
    slot_mapping, positions, use_input, kv_use, totals = torch.split(buf64, sizes64)
    sizes32 = [B + 1, B + 1, B]
    buf32 = torch.empty(sum(sizes32), **i32)
    seq_start, query_start, ctx = torch.split(buf32, sizes32)
    token_is_hidden = torch.empty(n_tok, dtype=torch.uint8, device=device)
    with on_device:
        st = lib.aps_build_prefill_metadata(
            d_lens.data_ptr(), d_ctx_in.data_ptr(), d_hid.data_ptr(), d_bt.data_ptr() if W else None, W, W, B,
            block_size, slot_mapping.data_ptr(), positions.data_ptr(), use_input.data_ptr() if n_ht else None,
            kv_use.data_ptr() if n_kt else None, token_is_hidden.data_ptr(), n_tok, n_ht, n_kt,
            seq_start.data_ptr(), query_start.data_ptr(),
            ctx.data_ptr(), totals.data_ptr(), stream.cuda_stream)
    _lib.check(st, "build_prefill_metadata")
    if check_totals:
        got = totals.tolist()
        if got[:2] != [n_tok, n_ht] or got[3] != n_kt:
            raise RuntimeError(f"device totals {got} disagree with the host's {[n_tok, n_ht, n_kt]}")
    empty64 = torch.empty(0, **i64)
    return HybridAttentionMetadata(
        num_prefills=B, num_prefill_tokens=n_tok, num_decode_tokens=0, num_hidden_cache_tokens=n_ht,
        num_tot_tokens=n_tok, slot_mapping=slot_mapping, slot_mapping_shared=empty64,
        hidden_cache_use_tot=use_input, kv_cache_use_tot=kv_use, hidden_cache_use_input=use_input,
        hidden_cache_store_tot=use_input, hidden_holder_upd=empty64, hidden_holder_pull=empty64,
        seq_lens=lens.tolist(), seq_lens_tensor=d_lens, max_query_len=int(qlens.max()),
        max_prefill_seq_len=int(lens.max()), max_decode_seq_len=0, query_start_loc=query_start,
        seq_start_loc=seq_start, context_lens_tensor=ctx,
        # the tables travel with a prompt step only when it continues a cached prefix (the reference fills them for
        # prefix hits and chunked prompts: aptserve_model_runner.py:410-437)
        block_tables=d_bt if (W and int(ctxs.max()) > 0) else torch.empty(B, 0, **i32), use_cuda_graph=False,
        input_positions=positions, block_types=None,
        token_is_hidden=token_is_hidden, max_prompt_context_len=int(ctxs.max()))


def build_from_batch(batch, device, packed: bool = False, **kw) -> HybridAttentionMetadata:
    """Convenience for :class:`aptserve_hip.workloads.Batch`; ``packed`` hands over the batch's block tables as
    the 0-padded int32 arrays ``batch.packed_tables()`` keeps instead of as lists of lists."""
    if packed:
        bt, bts = batch.packed_tables()
        return build_metadata(batch.is_prompt, batch.seq_lens_np, batch.use_hidden_np, bt, bts, batch.block_size,
                              device, **kw)
    return build_metadata(batch.is_prompt, batch.seq_lens, batch.use_hidden, batch.block_tables,
                          batch.block_tables_4_shared, batch.block_size, device, **kw)
