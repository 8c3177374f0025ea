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

from ..kernel import kv_cache_append, kv_cache_fill
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
