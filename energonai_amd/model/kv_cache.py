"""Preallocated per-sequence K/V cache for incremental decode.

The reference keeps the whole projection history and ``torch.cat``s one more
position onto it on every step, then recomputes attention for every position
(energonai/model/attention.py:61-71,89-98).  Here K and V live in two
``[B,H,Smax,D]`` buffers with a device-side length per sequence: prefill writes
each sequence's rows at positions ``0..len-1`` (whatever side the batch was
padded on), a decode step appends one row per sequence and reads only the
valid prefix.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernel import decode_attn, decode_attn_paged, kv_cache_append, kv_cache_fill, kv_pages_append, kv_pages_fill
from ..seqinfo import SeqInfo


class KVCache:
    def __init__(self, batch_size: int, head_num: int, max_seq_len: int, size_per_head: int, dtype, device):
        self.k = torch.zeros((batch_size, head_num, max_seq_len, size_per_head), dtype=dtype, device=device)
        self.v = torch.zeros_like(self.k)
        self.lens = torch.zeros(batch_size, dtype=torch.int32, device=device)
        self.batch_size = batch_size
        self.max_seq_len = max_seq_len
        self._longest = 0       # host-side bound of the longest cached sequence (no device read per step)
        # lengths are advanced in place, so the kernels are handed this fixed view instead of
        # going through the per-tensor offset cache
        self.info = SeqInfo(self.lens, None, batch_size, None, self.lens)

    def fill(self, k_src: torch.Tensor, v_src: torch.Tensor, info: SeqInfo, k_head_first: int = 0,
             v_head_first: int = 0, longest: Optional[int] = None) -> None:
        """Prefill from packed projections seen as ``[T,Hs,D]`` (see ``kv_cache_fill``).  ``longest`` is the
        longest sequence length if the caller knows it on the host (the bucket length is an upper bound)."""
        # the buffers were zeroed when they were allocated and no reader goes past the lengths
        kv_cache_fill(k_src, self.k, self.batch_size, info, k_head_first, zero_padding=False)
        kv_cache_fill(v_src, self.v, self.batch_size, info, v_head_first, zero_padding=False)
        self.lens.copy_(info.lens)
        # the fill kernel is given at most max_seq_len rows per sequence; the bound is tightened when the
        # caller has the true maximum on the host
        self._longest = self.max_seq_len if longest is None else min(int(longest), self.max_seq_len)

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor) -> None:
        """One new ``[B,H,D]`` row per sequence; lengths advance by one.  Raises when a sequence may already
        fill the cache: the kernel would drop its new row and decoding would go on without the newest token
        (the reference's torch.cat cache grows instead, energonai/model/attention.py:66-71)."""
        if self._longest >= self.max_seq_len:
            raise RuntimeError(f"KVCache.append: the cache holds max_seq_len = {self.max_seq_len} positions and a "
                               f"sequence may already be that long; allocate the cache for prompt + generated tokens")
        self._longest += 1
        kv_cache_append(k_new, v_new, self.k, self.v, self.info)
        self.lens.add_(1)

    def attend(self, q: torch.Tensor, scale: float) -> torch.Tensor:
        """Attention of one new query per sequence over the cached positions: ``[B,H,1,D]``."""
        return decode_attn(q, self.k, self.v, self.info, scale=scale)


class PagedKVCache:
    """The same cache kept in pages of ``page_size`` positions taken from one pool: a sequence holds the pages its
    length needs, not ``max_seq_len`` positions, so a batch of uneven lengths (or a server that keeps many
    sequences resident) holds memory for the tokens it has.  ``pool_pages`` defaults to what the contiguous cache
    would hold (every sequence at full length); a caller that knows its mix passes less.

    The page table lives on the device (``int32 [B, max_pages]``, -1 where no page is assigned); which pages are
    free, and each sequence's length, are tracked on the host, so neither ``append`` nor ``attend`` reads the
    device: a sequence gets its next page when its host-side length reaches a page boundary (one small copy to the
    device, every ``page_size`` steps)."""

    def __init__(self, batch_size: int, head_num: int, max_seq_len: int, size_per_head: int, dtype, device,
                 page_size: int = 64, pool_pages: Optional[int] = None):
        if page_size < 16 or page_size & (page_size - 1):
            raise ValueError("page_size must be a power of two, at least 16")
        self.page_size = page_size
        self.max_pages = (max_seq_len + page_size - 1) // page_size
        self.pool_pages = batch_size * self.max_pages if pool_pages is None else int(pool_pages)
        self.k = torch.zeros((self.pool_pages, head_num, page_size, size_per_head), dtype=dtype, device=device)
        self.v = torch.zeros_like(self.k)
        self.table = torch.full((batch_size, self.max_pages), -1, dtype=torch.int32, device=device)
        self.lens = torch.zeros(batch_size, dtype=torch.int32, device=device)
        self.info = SeqInfo(self.lens, None, batch_size, None, self.lens)
        self.batch_size = batch_size
        self.max_seq_len = self.max_pages * page_size
        self._free = list(range(self.pool_pages - 1, -1, -1))
        self._pages = [[] for _ in range(batch_size)]
        self._host_lens = [0] * batch_size

    def pages_in_use(self) -> int:
        return self.pool_pages - len(self._free)

    def _assign(self, wants) -> None:
        """``wants``: (sequence, number of pages it must hold).  Takes pages off the free list and writes the new
        table entries in one copy."""
        wants = list(wants)
        extra = 0
        for b, n in wants:                       # nothing is taken unless everything asked for can be given
            if n > self.max_pages:
                raise RuntimeError(f"PagedKVCache: a sequence would pass max_seq_len = {self.max_seq_len}")
            extra += max(0, n - len(self._pages[b]))
        if extra > len(self._free):
            raise RuntimeError(f"PagedKVCache: the pool of {self.pool_pages} pages is used up")
        rows, cols, ids = [], [], []
        for b, n in wants:
            while len(self._pages[b]) < n:
                pid = self._free.pop()
                rows.append(b)
                cols.append(len(self._pages[b]))
                ids.append(pid)
                self._pages[b].append(pid)
        if ids:
            dev = self.table.device
            self.table[torch.tensor(rows, device=dev), torch.tensor(cols, device=dev)] = \
                torch.tensor(ids, dtype=torch.int32, device=dev)

    def release(self, b: int) -> None:
        """Returns the pages of sequence ``b`` to the pool (the sequence has finished)."""
        self._free.extend(reversed(self._pages[b]))
        self._pages[b] = []
        self._host_lens[b] = 0
        self.table[b].fill_(-1)
        self.lens[b] = 0

    def fill(self, k_src: torch.Tensor, v_src: torch.Tensor, info: SeqInfo, k_head_first: int = 0,
             v_head_first: int = 0, longest: Optional[int] = None, lens_host=None) -> None:
        """Prefill from packed projections seen as ``[T,Hs,D]``.  The pages are assigned on the host, which needs
        the lengths there: ``lens_host`` if the caller has them, else ``info.lens_host()`` (one copy from the device per
        batch, shared by every layer that fills its cache from the same ``info``)."""
        if lens_host is None:
            lens_host = info.lens_host()
        lens_host = [int(n) for n in lens_host]
        P = self.page_size
        for b in range(self.batch_size):
            if self._pages[b]:
                self.release(b)
        self._assign([(b, (n + P - 1) // P) for b, n in enumerate(lens_host)])
        bound = self.max_seq_len if longest is None else min(int(longest), self.max_seq_len)
        kv_pages_fill(k_src, self.k, self.batch_size, bound, info, self.table, k_head_first)
        kv_pages_fill(v_src, self.v, self.batch_size, bound, info, self.table, v_head_first)
        self.lens.copy_(info.lens)
        self._host_lens = lens_host

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor) -> None:
        """One new ``[B,H,D]`` row per sequence; lengths advance by one.  A sequence whose length sits on a page
        boundary is given a page first (raises when the pool or the sequence's table row is full)."""
        P = self.page_size
        self._assign([(b, n // P + 1) for b, n in enumerate(self._host_lens) if n % P == 0])
        kv_pages_append(k_new, v_new, self.k, self.v, self.info, self.table)
        self.lens.add_(1)
        self._host_lens = [n + 1 for n in self._host_lens]

    def attend(self, q: torch.Tensor, scale: float) -> torch.Tensor:
        return decode_attn_paged(q, self.k, self.v, self.info, self.table, scale=scale)


class OutputHistory:
    """The padded ``[B, S_so_far, hid]`` output a cached module hands back on every call
    (``past_cache['dense']`` and friends in the reference, energonai/model/attention.py:126-135),
    kept in one preallocated buffer: a decode step writes one position and returns a view,
    where the reference concatenates the whole history again."""

    def __init__(self) -> None:
        self.buf = None
        self.cur = 0

    def start(self, out: torch.Tensor, max_seq_len: int) -> torch.Tensor:
        B, S, hid = out.shape
        self.buf = torch.empty((B, max(int(max_seq_len), S), hid), dtype=out.dtype, device=out.device)
        self.buf[:, :S].copy_(out)
        self.cur = S
        return self.buf[:, :S]

    def push(self, new: torch.Tensor) -> torch.Tensor:
        if self.buf is None:
            raise RuntimeError("decode step before a first_cache=True call")
        if self.cur == self.buf.shape[1]:      # past the planned length: grow geometrically
            grown = torch.empty((self.buf.shape[0], 2 * self.cur, self.buf.shape[2]), dtype=self.buf.dtype,
                                device=self.buf.device)
            grown[:, :self.cur].copy_(self.buf)
            self.buf = grown
        self.buf[:, self.cur:self.cur + 1].copy_(new)
        self.cur += 1
        return self.buf[:, :self.cur]
