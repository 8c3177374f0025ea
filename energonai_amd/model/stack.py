"""A run of blocks on packed tokens: the padding is dropped once in front of the first block and
restored once behind the last one, which is how the reference's example models bracket their
layer loop (examples/gpt/gpt.py:292-323: offsets and remove-padding before the loop,
ft_rebuild_padding after it), instead of once per block."""
from __future__ import annotations

from typing import Iterable, Optional

import torch
from torch import nn

from ..kernel import depad, repad
from ..seqinfo import seq_info
from .attention import lens_from_mask
from .endecoder import Block1D


class PackedStack(nn.Module):
    def __init__(self, blocks: Iterable[Block1D], norm: Optional[nn.Module] = None) -> None:
        super().__init__()
        self.blocks = nn.ModuleList(blocks)
        self.norm = norm      # final LayerNorm of a decoder stack (energonai/model/model_factory.py:127-128), if any

    def forward(self, hidden_states, attention_mask=None, first_cache=False, seq_lens=None):
        """``[B,S,hid]`` padded batch in and out, like a loop over ``Block1D.forward``.

        With the past cache enabled in the blocks, ``first_cache=True`` runs the prefill (and fills every
        block's K/V cache); later calls run each block on the newest position only.
        """
        B, S, hid = hidden_states.shape
        caching = len(self.blocks) > 0 and not self.blocks[0].disable_past_cache
        if caching and not first_cache:
            for blk in self.blocks:
                hidden_states = blk(hidden_states, attention_mask=attention_mask, first_cache=False)
            return hidden_states if self.norm is None else self.norm(hidden_states)
        if seq_lens is None:
            seq_lens = lens_from_mask(attention_mask) if attention_mask is not None else \
                torch.full((B,), S, dtype=torch.int32, device=hidden_states.device)
        info = seq_info(seq_lens, B, hidden_states.device)
        left = self.blocks[0].attn.left_padded if len(self.blocks) else False
        x = depad(hidden_states, B, info, left_padded=left)
        for blk in self.blocks:
            x = blk.forward_packed(x, info, B, S, fill_cache=caching)
            if caching:   # each block keeps its own padded output for the later steps, as the reference blocks do
                blk._history.start(repad(x, B, S, info, left_padded=left), blk.max_seq_len)
        if self.norm is not None:
            x = self.norm(x)
        return repad(x, B, S, info, left_padded=left)
