"""Transformer block with the interface of the reference's ``Block1D``
(energonai/model/endecoder.py:11-70), computed on packed tokens: padding rows are dropped
once at the block entry and restored at its exit; the residual add in front of the second
LayerNorm is fused into that LayerNorm.
"""
from __future__ import annotations

from typing import Callable, Optional

import torch
from torch import nn

from ..kernel import LayerNorm, depad, layer_norm_forward, repad
from ..seqinfo import SeqInfo, seq_info
from .attention import MultiHeadAttention1D, lens_from_mask
from .kv_cache import OutputHistory
from .mlp import MLP1D


class Block1D(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, mlp_ratio: float, activation: Callable = nn.functional.gelu,
                 layernorm_epsilon: float = 1e-5, dtype: torch.dtype = torch.float16, bias: bool = True,
                 apply_post_layernorm: bool = False, max_seq_len: int = 512, fused_qkv: bool = True,
                 is_decoder: bool = True, disable_past_cache=False, kv_page_size: Optional[int] = None,
                 kv_pool_pages: Optional[int] = None) -> None:
        super().__init__()
        self.apply_post_layernorm = apply_post_layernorm
        self.disable_past_cache = disable_past_cache
        self.norm1 = LayerNorm(hidden_size, eps=layernorm_epsilon, dtype=dtype)
        self.attn = MultiHeadAttention1D(hidden_size=hidden_size, num_heads=num_heads, bias=bias, dtype=dtype,
                                         max_seq_len=max_seq_len, fused_qkv=fused_qkv, is_decoder=is_decoder,
                                         disable_past_cache=disable_past_cache, kv_page_size=kv_page_size,
                                         kv_pool_pages=kv_pool_pages)
        self.norm2 = LayerNorm(hidden_size, eps=layernorm_epsilon, dtype=dtype)
        self.mlp = MLP1D(hidden_size=hidden_size, mlp_ratio=mlp_ratio, activation=activation, dtype=dtype, bias=bias,
                         disable_past_cache=disable_past_cache)
        self.max_seq_len = max_seq_len
        self._history = OutputHistory()

    def _rows(self, x: torch.Tensor, attend) -> torch.Tensor:
        """endecoder.py:48-70 on any ``[.., rows, hid]`` tensor; ``attend`` maps normalised rows
        to the attention output for the same rows."""
        h = self.norm1(x)
        if self.apply_post_layernorm:
            s1 = h + attend(h)
            h2 = self.norm2(s1)
            return h2 + self.mlp.forward_rows(h2)
        # pre-LN: the sum x + attention is needed twice (as the next residual and under norm2),
        # so the second LayerNorm produces both in one pass
        h2, s1 = layer_norm_forward(attend(h), self.norm2.weight.detach(), self.norm2.bias.detach(),
                                    self.norm2.normalized_shape, self.norm2.eps, residual=x, return_sum=True)
        return s1 + self.mlp.forward_rows(h2)

    def forward_packed(self, x: torch.Tensor, info: SeqInfo, batch_size: int, max_seq_len: int,
                       fill_cache: bool = False) -> torch.Tensor:
        """``[1,T,hid]`` valid tokens in, ``[1,T,hid]`` out: lets a model drop the padding once
        in front of its first block instead of once per block."""
        return self._rows(x, lambda h: self.attn.forward_packed(h, info, batch_size, max_seq_len, fill_cache))

    def forward(self, hidden_states, attention_mask=None, first_cache=False, seq_lens=None):
        B, S, hid = hidden_states.shape
        if not self.disable_past_cache and not first_cache:
            return self._history.push(self._rows(hidden_states[:, -1:, :].contiguous(), self.attn.forward_last))
        if seq_lens is None:
            seq_lens = lens_from_mask(attention_mask) if attention_mask is not None else \
                torch.full((B,), S, dtype=torch.int32, device=hidden_states.device)
        info = seq_info(seq_lens, B, hidden_states.device)
        left = self.attn.left_padded
        x = depad(hidden_states, B, info, left_padded=left)
        y = self.forward_packed(x, info, B, S, fill_cache=not self.disable_past_cache)
        out = repad(y, B, S, info, left_padded=left)
        if not self.disable_past_cache:
            return self._history.start(out, self.max_seq_len)
        return out
