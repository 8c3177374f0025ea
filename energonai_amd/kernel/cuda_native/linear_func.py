"""``linear`` / ``find_algo`` keep their names so ``from energonai.kernel import
linear, find_algo`` still works (energonai/kernel/cuda_native/linear_func.py:11-92).

The dense projection GEMM is not part of the padding-removal path; on ROCm
``torch.nn.functional.linear`` already dispatches to hipBLASLt, which chooses
its own algorithm, so there is nothing for ``find_algo`` to search.
"""
from __future__ import annotations

import torch


def linear(inputs, param, algo=-1):
    """fp16 ``inputs[B,S,din] @ param[dout,din]^T`` (linear_func.py:11-32); ``algo`` is accepted and ignored."""
    if not inputs.is_cuda or not param.is_cuda:
        raise RuntimeError("linear: inputs and param must be CUDA tensors")
    return torch.nn.functional.linear(inputs, param)


def find_algo():
    """The reference brute-forces cuBLAS algorithm ids (linear_func.py:35-92); hipBLASLt
    selects per problem at run time, so the default id is returned."""
    return -1
