"""MLP block with the interface of the reference's ``MLP1D`` (energonai/model/mlp.py:7-51)."""
from __future__ import annotations

from typing import Callable, Optional

import torch
from torch import nn

from ..kernel.cuda_native.linear_func import linear
from .gemm import gemm_algo


def _epilogue_of(activation) -> Optional[str]:
    """Name of the GEMM epilogue that computes ``activation`` exactly, if there is one."""
    if activation in (nn.functional.relu, torch.relu) or isinstance(activation, nn.ReLU):
        return "relu"
    if isinstance(activation, nn.GELU) and activation.approximate == "tanh":
        return "gelu_tanh"
    if getattr(activation, "func", None) is nn.functional.gelu and \
            getattr(activation, "keywords", {}).get("approximate") == "tanh":
        return "gelu_tanh"
    return None


class MLP1D(nn.Module):

    def __init__(self, hidden_size: int, mlp_ratio: float, activation: Callable, dtype: torch.dtype = torch.float16,
                 bias: bool = True, disable_past_cache=False):
        super().__init__()
        self.disable_past_cache = disable_past_cache
        intermediate_dim = int(hidden_size * mlp_ratio)
        self.dense_1 = nn.Linear(hidden_size, intermediate_dim, bias=bias, dtype=dtype)
        self.activation = activation
        self.dense_2 = nn.Linear(intermediate_dim, hidden_size, bias=bias, dtype=dtype)
        self._epilogue = _epilogue_of(activation)
        self._out = None    # [B, S_so_far, hid]: what the reference keeps in past_cache['dense_2']

    def forward_rows(self, x: torch.Tensor) -> torch.Tensor:
        """The MLP on any ``[..., hid]`` rows (packed tokens or the last position of a batch).

        ReLU (the OPT models) and tanh-GELU are applied, with the bias, in the epilogue of the first GEMM;
        any other activation runs as its own op between two library GEMMs, as in mlp.py:31-33.
        """
        if self._epilogue is not None and x.is_cuda and x.dim() == 3 and x.is_contiguous():
            h = linear(x, self.dense_1.weight.detach(), gemm_algo(), bias=_detached(self.dense_1.bias),
                       activation=self._epilogue)
            return linear(h, self.dense_2.weight.detach(), gemm_algo(), bias=_detached(self.dense_2.bias))
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


def _detached(t):
    return None if t is None else t.detach()
