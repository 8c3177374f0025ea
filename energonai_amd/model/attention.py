"""Self-attention with the interface of the reference's ``MultiHeadAttention1D``
(energonai/model/attention.py:9-136), computed on packed tokens.

Differences in mechanism, not in result: padding rows are dropped before the projections
and restored after the output projection; attention runs in the fused variable-length
kernel (16-bit) or the QK^T / scale_mask_softmax / PV kernels (fp32); incremental decode
appends to a preallocated K/V cache and computes the newest position only, where the
reference concatenates and recomputes every position (attention.py:61-71).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from ..kernel import (attn_fused_varlen, attn_pv, attn_qk, decode_attn, decode_pv, decode_qk, depad, repad, scale_mask_softmax,
                      transpose_depad)
from ..kernel.attention import kv_cache_fill
from ..seqinfo import SeqInfo, seq_info
from .gemm import project
from .kv_cache import KVCache, OutputHistory, PagedKVCache


def lens_from_mask(attention_mask: torch.Tensor) -> torch.Tensor:
    """Valid length per sequence from the additive ``[B,1,1,S]`` mask the reference builds
    (0 for tokens, -10000 for padding; energonai/model/model_factory.py:117-121)."""
    m = attention_mask.reshape(attention_mask.shape[0], -1, attention_mask.shape[-1])[:, 0, :]
    return (m > -1.0).sum(-1).to(torch.int32)


class MultiHeadAttention1D(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, bias: bool = True, dtype: torch.dtype = torch.float16,
                 max_seq_len: int = 512, fused_qkv: bool = True, is_decoder: bool = True, disable_past_cache=False,
                 left_padded: Optional[bool] = None, kv_page_size: Optional[int] = None,
                 kv_pool_pages: Optional[int] = None) -> None:
        super().__init__()
        if hidden_size % num_heads != 0:
            raise ValueError(f"{hidden_size} is not divisible by {num_heads}")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.attention_head_size = hidden_size // num_heads
        self.fused_qkv = fused_qkv
        self.is_decoder = is_decoder
        self.disable_past_cache = disable_past_cache
        self.max_seq_len = max_seq_len
        self.scaling = self.attention_head_size ** -0.5
        # generation batches are padded on the left (examples/opt/batch.py:12-24), encoder batches on the right
        self.left_padded = is_decoder if left_padded is None else left_padded
        if fused_qkv:
            self.query_key_value = nn.Linear(hidden_size, 3 * hidden_size, bias=bias, dtype=dtype)
        else:
            self.query_ = nn.Linear(hidden_size, hidden_size, bias=bias, dtype=dtype)
            self.key_ = nn.Linear(hidden_size, hidden_size, bias=bias, dtype=dtype)
            self.value_ = nn.Linear(hidden_size, hidden_size, bias=bias, dtype=dtype)
        self.dense = nn.Linear(hidden_size, hidden_size, bias=True, dtype=dtype)
        # None: one [B,H,max_seq_len,D] buffer per cache; a page size: pages of a pool (PagedKVCache)
        self.kv_page_size = kv_page_size
        self.kv_pool_pages = kv_pool_pages
        self.kv_cache = None
        self._history = OutputHistory()     # what the reference keeps in past_cache['dense']

    # ---- projections: packed rows in, [rows, H, D] views of q, k, v out --------------------
    def _project(self, x: torch.Tensor):
        H, D = self.num_heads, self.attention_head_size
        rows = x.numel() // self.hidden_size
        if self.fused_qkv:
            # the fused output is ordered k, v, q (attention.py:74)
            kvq = project(self.query_key_value, x).view(rows, 3 * H, D)
            return kvq[:, 2 * H:], kvq[:, :H], kvq[:, H:2 * H], kvq
        q = project(self.query_, x).view(rows, H, D)
        k = project(self.key_, x).view(rows, H, D)
        v = project(self.value_, x).view(rows, H, D)
        return q, k, v, None

    # ---- attention over packed tokens --------------------------------------------------------
    def forward_packed(self, x: torch.Tensor, info: SeqInfo, batch_size: int, max_seq_len: int,
                       fill_cache: bool = False) -> torch.Tensor:
        """``x`` is ``[1,T,hid]`` (valid tokens only); returns the attention output ``[1,T,hid]``."""
        H, D = self.num_heads, self.attention_head_size
        T = x.numel() // self.hidden_size
        q, k, v, kvq = self._project(x)
        if x.dtype in (torch.float16, torch.bfloat16):
            ctx = attn_fused_varlen(q, k, v, batch_size, max_seq_len, info, scale=self.scaling,
                                    causal=self.is_decoder)
        else:
            # fp32: the three separate kernels on padded [B,H,S,D] operands
            pads = []
            for t in (q, k, v):
                buf = torch.empty((batch_size, H, max_seq_len, D), dtype=x.dtype, device=x.device)
                pads.append(kv_cache_fill(t.contiguous(), buf, batch_size, info, zero_padding=False))
            scores = attn_qk(pads[0], pads[1], info, causal=self.is_decoder)
            probs = scale_mask_softmax(batch_size, max_seq_len, H, scores, info, scale=self.scaling,
                                       causal=self.is_decoder, tail_rows=1)
            ctx = transpose_depad(attn_pv(probs, pads[2], info, causal=self.is_decoder), batch_size, T, max_seq_len,
                                  info, H, D)
        if fill_cache:
            if max_seq_len > self.max_seq_len:
                raise RuntimeError(f"the batch is padded to {max_seq_len} positions but the K/V cache was planned for "
                                   f"max_seq_len = {self.max_seq_len}")
            if self.kv_page_size:
                self.kv_cache = PagedKVCache(batch_size, H, self.max_seq_len, D, x.dtype, x.device,
                                             page_size=self.kv_page_size, pool_pages=self.kv_pool_pages)
            else:
                self.kv_cache = KVCache(batch_size, H, self.max_seq_len, D, x.dtype, x.device)
            if kvq is not None:
                self.kv_cache.fill(kvq, kvq, info, 0, H, longest=max_seq_len)
            else:
                self.kv_cache.fill(k.contiguous(), v.contiguous(), info, longest=max_seq_len)
        return project(self.dense, ctx.view(1, T, self.hidden_size))

    # ---- one decode step: newest position only ----------------------------------------------
    def forward_last(self, last: torch.Tensor) -> torch.Tensor:
        """``last`` is ``[B,1,hid]``, the newest position of every sequence; returns ``[B,1,hid]``."""
        if self.kv_cache is None:
            raise RuntimeError("decode step before a first_cache=True call")
        H, D = self.num_heads, self.attention_head_size
        B = last.shape[0]
        cache = self.kv_cache
        q, k, v, _ = self._project(last)
        cache.append(k, v)
        ctx = cache.attend(q, self.scaling)      # [B,H,1,D], one pass over the caches
        return project(self.dense, ctx.view(B, 1, self.hidden_size))

    def forward(self, hidden_states, attention_mask=None, first_cache=False, seq_lens=None):
        B, S, hid = hidden_states.shape
        if not self.disable_past_cache and not first_cache:
            return self._history.push(self.forward_last(hidden_states[:, -1:, :]))
        if seq_lens is None:
            seq_lens = lens_from_mask(attention_mask) if attention_mask is not None else \
                torch.full((B,), S, dtype=torch.int32, device=hidden_states.device)
        info = seq_info(seq_lens, B, hidden_states.device)
        x = depad(hidden_states, B, info, left_padded=self.left_padded)
        y = self.forward_packed(x, info, B, S, fill_cache=not self.disable_past_cache)
        out = repad(y, B, S, info, left_padded=self.left_padded)
        if not self.disable_past_cache:
            return self._history.start(out, self.max_seq_len)
        return out


_ONES = {}


def _ones(batch: int, device) -> torch.Tensor:
    key = (batch, str(device))
    if key not in _ONES:
        _ONES[key] = torch.ones(batch, dtype=torch.int32, device=device)
    return _ONES[key]
