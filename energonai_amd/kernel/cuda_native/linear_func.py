"""``linear`` / ``find_algo`` of the reference (energonai/kernel/cuda_native/linear_func.py:11-92) on hipBLASLt.

The reference calls ``cublasGemmEx`` with an algorithm id and finds the best id by timing them all.  hipBLASLt
ranks candidate solutions per problem instead, so ``algo`` is an index into that list (``-1`` = first choice)
and ``find_algo`` times the candidates of the reference's probe problem.  ``algo="auto"`` does that search for
the problem at hand, once, and remembers the winner (``tuned_algo``): the library's first choice is often not the
fastest for the skinny GEMMs of a decode step.  ``bias`` and ``activation`` are
additions: hipBLASLt applies them in the GEMM epilogue, where the reference's callers run separate ops
(energonai/model/mlp.py:30-35).
"""
from __future__ import annotations

import time
from typing import Dict, Optional

import torch

from ... import _lib

_ACTIVATIONS = {None: 0, "none": 0, "relu": 1, "gelu_tanh": 2}
_WORKSPACE_BYTES = 64 << 20
_workspaces: Dict[int, torch.Tensor] = {}
_tuned: Dict[tuple, int] = {}


def _workspace(device: torch.device) -> torch.Tensor:
    """hipBLASLt scratch, one buffer per device from torch's allocator (the library never allocates)."""
    ws = _workspaces.get(device.index)
    if ws is None:
        ws = torch.empty(_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _workspaces[device.index] = ws
    return ws


def _check(status: int, op: str) -> None:
    if status < 0:
        raise RuntimeError(f"{op}: {_lib.load_linear().en_linear_status_string(status).decode()}")


def linear(inputs, param, algo=-1, bias=None, activation: Optional[str] = None):
    """``inputs[batch, seq_len, din] @ param[dout, din]^T`` -> ``[batch, seq_len, dout]`` (linear_func.py:11-32).

    fp16 like the reference, also bf16 and fp32; fp32 accumulation.  ``bias`` ``[dout]`` and ``activation``
    (``"relu"`` or ``"gelu_tanh"``) are applied in the GEMM epilogue.
    """
    lib = _lib.load_linear()
    _lib.require_gpu(inputs, "inputs")
    _lib.require_gpu(param, "param")
    if inputs.dim() != 3 or param.dim() != 2 or inputs.shape[2] != param.shape[1]:
        raise RuntimeError("linear: inputs must be [batch, seq_len, din] and param [dout, din]")
    if isinstance(algo, str) and algo == "auto":
        algo = tuned_algo(inputs, param, bias=bias, activation=activation)
    if not isinstance(algo, int) or algo < -1:
        raise RuntimeError("linear: algo must be -1, \"auto\" or an index below find_algo's candidate count")
    if param.dtype != inputs.dtype or (bias is not None and bias.dtype != inputs.dtype):
        raise RuntimeError("linear: inputs, param and bias must share one dtype")
    if activation not in _ACTIVATIONS:
        raise RuntimeError(f"linear: activation must be one of {sorted(k for k in _ACTIVATIONS if k)}")
    if bias is not None:
        _lib.require_gpu(bias, "bias")
        if bias.numel() != param.shape[0]:
            raise RuntimeError("linear: bias must be [dout]")
    B, S, din = inputs.shape
    dout = param.shape[0]
    if algo >= 0 and (algo <= 23 or 99 <= algo <= 115):
        # every id the reference accepts (cuBLAS constants -1..23 and 99..115, csrc/linear_wrapper.cpp:133-140)
        # is valid here too: one that lies past this problem's candidate list means the first choice
        with _lib.device_guard(inputs):
            if algo >= algo_count(B * S, din, dout, inputs.dtype, bias is not None, activation):
                algo = -1
    out = torch.empty((B, S, dout), dtype=inputs.dtype, device=inputs.device)
    ws = _workspace(inputs.device)
    with _lib.device_guard(inputs):
        _check(lib.en_linear(inputs.data_ptr(), param.data_ptr(), _lib.ptr(bias), out.data_ptr(), B * S, din, dout,
                             _ACTIVATIONS[activation], _lib.dtype_tag(inputs, "linear"), algo, ws.data_ptr(),
                             ws.numel(), _lib.stream_of(inputs)), "linear")
    return out


def algo_count(rows: int, din: int, dout: int, dtype=torch.float16, has_bias: bool = False,
               activation: Optional[str] = None) -> int:
    """How many candidate solutions ``algo`` may index for this problem."""
    lib = _lib.load_linear()
    n = lib.en_linear_algo_count(rows, din, dout, int(has_bias), _ACTIVATIONS[activation],
                                 _lib._DTYPE_TAG[dtype], _WORKSPACE_BYTES)
    _check(n, "algo_count")
    return n


@torch.no_grad()
def tuned_algo(inputs, param, bias=None, activation: Optional[str] = None, inner_loop: int = 5) -> int:
    """Index of the fastest candidate for ``linear(inputs, param, bias=bias, activation=activation)``.

    Every candidate is timed with HIP events on the given tensors the first time a problem
    ``(rows, din, dout, dtype, bias, activation)`` is seen on a device (the reference finds its cuBLAS algorithm
    the same way on one probe problem, linear_func.py:35-92); later calls return the remembered index.  The
    search launches and synchronises, so the first call of a problem must not sit inside a stream capture.
    """
    rows = inputs.shape[0] * inputs.shape[1]
    key = (inputs.device.index, rows, inputs.shape[2], param.shape[0], inputs.dtype, bias is not None, activation)
    best = _tuned.get(key)
    if best is not None:
        return best
    n = algo_count(rows, inputs.shape[2], param.shape[0], inputs.dtype, bias is not None, activation)
    best, best_t = -1, float("inf")
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for algo in range(n):
        linear(inputs, param, algo, bias=bias, activation=activation)
        start.record()
        for _ in range(inner_loop):
            linear(inputs, param, algo, bias=bias, activation=activation)
        stop.record()
        stop.synchronize()
        dt = start.elapsed_time(stop)
        if dt < best_t:
            best, best_t = algo, dt
    _tuned[key] = best
    return best


@torch.no_grad()
def find_algo(batch_size: int = 16, seq_len: int = 64, din: int = 12288, dout: int = 49152, inner_loop: int = 3):
    """Times every candidate on the reference's probe problem (linear_func.py:43-46) and returns the best index."""
    x = torch.randn(batch_size, seq_len, din, device="cuda").half()
    w = torch.randn(dout, din, device="cuda").half()
    n = algo_count(batch_size * seq_len, din, dout)
    best, best_t = -1, float("inf")
    for algo in range(n):
        linear(x, w, algo)
        torch.cuda.synchronize()
        t0 = time.time()
        for _ in range(inner_loop):
            linear(x, w, algo)
        torch.cuda.synchronize()
        dt = time.time() - t0
        if dt < best_t:
            best, best_t = algo, dt
    return best
