"""How the modules of this package run their projection GEMMs.

By default ``torch.nn.Linear`` does (and the MLP's fused-epilogue GEMMs take hipBLASLt's first choice).  With
``set_gemm_tuning(True)`` every projection goes through ``energonai_amd.kernel.linear`` with ``algo="auto"``:
the candidates are timed once per problem shape and the fastest is used from then on -- what the reference's
``find_algo`` is for (energonai/kernel/cuda_native/linear_func.py:35-92), done per shape.
"""
from __future__ import annotations

import torch
from torch import nn

from ..kernel.cuda_native.linear_func import linear

_tuning = False


def set_gemm_tuning(enabled: bool) -> None:
    """Switches the per-shape candidate search on or off for all modules of this package."""
    global _tuning
    _tuning = bool(enabled)


def gemm_tuning() -> bool:
    return _tuning


def gemm_algo():
    """The ``algo`` argument the modules pass to ``linear``."""
    return "auto" if _tuning else -1


def project(layer: nn.Linear, x: torch.Tensor) -> torch.Tensor:
    """``layer(x)``; with tuning on, 16-bit ``[batch, rows, din]`` inputs take the tuned hipBLASLt GEMM."""
    if _tuning and x.is_cuda and x.dim() == 3 and x.is_contiguous() and x.dtype in (torch.float16, torch.bfloat16) \
            and layer.weight.dtype == x.dtype:
        bias = None if layer.bias is None else layer.bias.detach()
        return linear(x, layer.weight.detach(), "auto", bias=bias)
    return layer(x)
