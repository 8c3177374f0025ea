"""Per-batch sequence bookkeeping shared by every kernel call of a forward pass.

The reference recomputes the prefix of ``seq_lens`` inside every block of every
kernel (csrc/transpose_pad_fusion_kernel.cu:24-27,70-73).  Here the prefix is
computed once per batch by one small kernel and reused by every op of every
layer; the public functions still accept the plain ``seq_lens`` tensor of the
reference API (int32 or int64, examples/bert/bert.py:100-103) and find the
cached offsets through :func:`seq_info`.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Optional

import torch

from . import _lib

_CACHE_SIZE = 16
TILES_FIRST_MAX_KV_BYTES = 256 << 10     # see SeqInfo.tile_table


class SeqInfo:
    """Device-resident int32 lengths and exclusive prefix for one batch."""

    __slots__ = ("lens", "cu_seqlens", "batch_size", "_total", "_source", "_row_offsets", "_tile_tables", "_ready",
                 "_ordered", "ephemeral", "_lens_host")

    def __init__(self, lens: torch.Tensor, cu_seqlens: torch.Tensor, batch_size: int, total: Optional[int], source):
        self.lens = lens                # int32 [B] on the device
        self.cu_seqlens = cu_seqlens    # int32 [B+1] on the device
        self.batch_size = batch_size
        self._total = total
        self._source = source           # keeps the caller's tensor alive while cached
        self._row_offsets = {}          # (max_seq_len, left_padded, version of lens) -> int32 [T]
        self._tile_tables = {}          # (head_num, q_seq_len, order, version of lens, tile height) -> int32 workgroup order
        self._ready = []                # events recorded behind the kernels that produced the arrays above
        self._ordered = set()           # raw streams already ordered behind every event of _ready
        self.ephemeral = False          # built for one call only (lengths that cannot be cached): see tile_table_ptr
        self._lens_host = None          # (version of lens, the lengths as a Python list)

    def produced_on_current_stream(self) -> None:
        """Call right after launching a kernel that writes one of this object's arrays: remembers the point
        in the launching stream where they are complete."""
        if not self.lens.is_cuda:
            return
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(self.lens.device))
        self._ready.append(ev)
        del self._ready[:-8]            # lengths that change every step rebuild their tables every step
        self._ordered = {_lib.stream_of(self.lens)}

    def order_current_stream(self) -> None:
        """Makes torch's current stream wait for the kernels that produced the offsets when they were launched
        on another stream (the arrays are cached and reused by later calls, whichever stream those run on)."""
        if not self._ready:
            return
        raw = _lib.stream_of(self.lens)
        if raw in self._ordered:
            return
        cur = torch.cuda.current_stream(self.lens.device)
        for ev in self._ready:
            cur.wait_event(ev)
        self._ordered.add(raw)

    @property
    def device(self) -> torch.device:
        return self.lens.device

    @property
    def total(self) -> int:
        """Sum of the lengths as a Python int.  The first use copies one int from
        the device (a sync), like ``valid_word_num[0].item()`` in the reference
        callers (examples/gpt/gpt.py:303); later uses are free."""
        if self._total is None:
            self._total = int(self.cu_seqlens[self.batch_size].item())
        return self._total


    def lens_host(self):
        """The lengths as a list of Python ints.  The first use copies them from the device (a sync, like
        ``total``); later uses of the same lengths are free, so every layer of a stack can ask."""
        version = self._lens_version()
        if self._lens_host is None or version is None or self._lens_host[0] != version:
            self.order_current_stream()
            self._lens_host = (version, [int(n) for n in self.lens.tolist()])
        return list(self._lens_host[1])

    def _lens_version(self):
        """Version counter of the lengths, part of every key under which something derived from them is kept:
        a caller that owns ``lens`` may change it in place (the K/V cache advances its lengths every step), and
        what was derived from the old lengths must then not be found again.  Tensors created under
        ``torch.inference_mode()`` have no counter; ``None`` then means "do not keep"."""
        try:
            return self.lens._version
        except RuntimeError:
            return None

    def row_offsets(self, max_seq_len: int, left_padded: bool) -> torch.Tensor:
        """``off[t]`` = row of token ``t`` in the padded ``[B*S]`` numbering minus ``t``; computed once per
        batch and bucket by one small kernel (the reference's ft offsets, csrc/transpose_pad_fusion_kernel.cu:
        112-131, made aware of left padding)."""
        version = self._lens_version()
        key = (int(max_seq_len), bool(left_padded), version)
        off = None if version is None and self._mutable() else self._row_offsets.get(key)
        self.order_current_stream()
        if off is None:
            off = torch.empty(max(self.total, 1), dtype=torch.int32, device=self.lens.device)
            with _lib.device_guard(self.lens):
                _lib.check(_lib.fn.en_padding_offsets(self.lens.data_ptr(), self.batch_size, key[0], int(key[1]),
                                                      off.data_ptr(), _lib.stream_of(self.lens)), "padding_offsets")
                self.produced_on_current_stream()
            if version is not None or not self._mutable():
                self._row_offsets = {k: o for k, o in self._row_offsets.items() if k[2] == version}
                self._row_offsets[key] = off
        return off

    def _mutable(self) -> bool:
        """True when the lengths belong to a caller that may edit them in place (no prefix was computed from
        them, or they are the caller's own tensor)."""
        return self.cu_seqlens is None or self._source is self.lens


    def tile_table(self, head_num: int, q_seq_len: int, unit_kv_bytes: int = 1 << 30, query_tile: int = 128) -> torch.Tensor:
        """Workgroup order of the attention kernels for this batch (``en_attn_tile_table``): the query tiles the
        sequences really have, longest sequence first.  ``unit_kv_bytes`` is what one (batch, head) unit's K and V
        hold at full length: up to 256 KB the last tiles of all units run first, above that a unit's tiles stay
        together.  ``query_tile`` is the tile height of the kernel that will read the table (128; 256 for the fused
        kernel's 64-queries-per-wave form).  Computed once per batch, head count, bucket, order and tile height by one
        small kernel and reused by every layer."""
        version = self._lens_version()
        key = (int(head_num), int(q_seq_len), int(unit_kv_bytes) <= TILES_FIRST_MAX_KV_BYTES, version, int(query_tile))
        tab = None if version is None and self._mutable() else self._tile_tables.get(key)
        self.order_current_stream()
        if tab is None:
            n = int(_lib.fn.en_attn_tile_table_elems(self.batch_size, key[0], key[1], key[4]))
            tab = torch.empty(max(n, 1), dtype=torch.int32, device=self.lens.device)
            with _lib.device_guard(self.lens):
                _lib.check(_lib.fn.en_attn_tile_table(self.lens.data_ptr(), self.batch_size, key[0], key[1], int(key[2]),
                                                      key[4], tab.data_ptr(), _lib.stream_of(self.lens)), "attn_tile_table")
                self.produced_on_current_stream()
            if version is not None or not self._mutable():
                # tables of older versions of the lengths can never be found again: drop them
                self._tile_tables = {k: t for k, t in self._tile_tables.items() if k[3] == version}
                self._tile_tables[key] = tab
        return tab


    def tile_table_ptr(self, head_num: int, q_seq_len: int, unit_kv_bytes: int = 1 << 30, query_tile: int = 128):
        """Raw pointer of the workgroup order for an attention call, or ``None`` (the kernels then compute their
        own order) when this object lives for one call only: building the table is a launch of its own, which pays
        off when every layer reuses it, not when every call would rebuild it (lengths given as Python lists or as
        tensors made under ``torch.inference_mode()`` are never cached -- pass a ``SeqInfo`` to keep one)."""
        if self.ephemeral:
            return None
        return self.tile_table(head_num, q_seq_len, unit_kv_bytes, query_tile).data_ptr()


_cache: "OrderedDict[tuple, SeqInfo]" = OrderedDict()


def build_seq_info(seq_lens, batch_size: int, device=None, total: Optional[int] = None) -> SeqInfo:
    """Runs the prefix-sum kernel.  ``seq_lens`` is a CUDA int32/int64 tensor, or
    a CPU tensor / list (then the total is known without a sync)."""
    if not isinstance(seq_lens, torch.Tensor):
        seq_lens = torch.as_tensor(list(seq_lens), dtype=torch.int32)
    if seq_lens.dtype not in (torch.int32, torch.int64):
        raise RuntimeError(f"seq_lens must be int32 or int64, got {seq_lens.dtype}")
    if seq_lens.numel() < batch_size:
        raise RuntimeError(f"seq_lens has {seq_lens.numel()} entries, batch_size is {batch_size}")
    source = seq_lens
    if not seq_lens.is_cuda:
        if total is None:
            total = int(seq_lens[:batch_size].sum())
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        seq_lens = seq_lens.to(device, non_blocking=False)
    seq_lens = seq_lens.contiguous()
    lib = _lib.load()
    with _lib.device_guard(seq_lens):
        cu = torch.empty(batch_size + 1, dtype=torch.int32, device=seq_lens.device)
        lens32 = torch.empty(batch_size, dtype=torch.int32, device=seq_lens.device)
        _lib.check(lib.en_prefix_sum(seq_lens.data_ptr(), int(seq_lens.dtype == torch.int64), batch_size,
                                     cu.data_ptr(), lens32.data_ptr(), _lib.stream_of(seq_lens)), "prefix_sum")
        info = SeqInfo(lens32, cu, batch_size, total, source)
        info.produced_on_current_stream()
    return info


def seq_info(seq_lens, batch_size: int, device=None) -> SeqInfo:
    """Returns the (cached) SeqInfo for ``seq_lens``.

    A SeqInfo passes through unchanged.  Tensors are cached by identity and
    version counter, and the cache holds a reference to the tensor so its
    storage cannot be recycled under a stale entry; in-place edits through torch
    bump the version and miss the cache.  Tensors created inside
    ``torch.inference_mode()`` (the reference worker runs the whole forward there,
    energonai/worker.py:79) carry no version counter, so an edit could not be
    noticed: they are never cached and the prefix kernel runs on every call.
    A cached entry used on another stream than the one its kernels were launched
    on makes that stream wait for them first.
    """
    if isinstance(seq_lens, SeqInfo):
        if seq_lens.batch_size != batch_size:
            raise RuntimeError(f"SeqInfo was built for batch {seq_lens.batch_size}, call passes {batch_size}")
        seq_lens.order_current_stream()
        return seq_lens
    if not isinstance(seq_lens, torch.Tensor) or torch.is_inference(seq_lens):
        info = build_seq_info(seq_lens, batch_size, device)
        info.ephemeral = True
        return info
    key = (id(seq_lens), seq_lens._version, seq_lens.data_ptr(), batch_size, str(device))
    hit = _cache.get(key)
    if hit is not None and hit._source is seq_lens:
        _cache.move_to_end(key)
        hit.order_current_stream()
        return hit
    info = build_seq_info(seq_lens, batch_size, device)
    _cache[key] = info
    while len(_cache) > _CACHE_SIZE:
        _cache.popitem(last=False)
    return info


def clear_cache() -> None:
    _cache.clear()
