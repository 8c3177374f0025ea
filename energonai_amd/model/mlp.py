"""MLP block with the interface of the reference's ``MLP1D`` (energonai/model/mlp.py:7-51)."""
from __future__ import annotations

from typing import Callable, Optional

import torch
from torch import nn


class MLP1D(nn.Module):

    def __init__(self, hidden_size: int, mlp_ratio: float, activation: Callable, dtype: torch.dtype = torch.float16,
                 bias: bool = True, disable_past_cache=False):
        super().__init__()
        self.disable_past_cache = disable_past_cache
        intermediate_dim = int(hidden_size * mlp_ratio)
        self.dense_1 = nn.Linear(hidden_size, intermediate_dim, bias=bias, dtype=dtype)
        self.activation = activation
        self.dense_2 = nn.Linear(intermediate_dim, hidden_size, bias=bias, dtype=dtype)
        self._out = None    # [B, S_so_far, hid]: what the reference keeps in past_cache['dense_2']

    def forward_rows(self, x: torch.Tensor) -> torch.Tensor:
        """The MLP on any ``[..., hid]`` rows (packed tokens or the last position of a batch)."""
        return self.dense_2(self.activation(self.dense_1(x)))

    def forward(self, hidden_states, first_cache: Optional[bool] = True):
        if self.disable_past_cache:
            return self.forward_rows(hidden_states)
        if first_cache:
            self._out = self.forward_rows(hidden_states)
            return self._out
        # later steps compute the newest position only and return it behind the earlier ones (mlp.py:42-49)
        new = self.forward_rows(hidden_states[:, -1:, :])
        self._out = torch.cat((self._out, new), 1)
        return self._out
