"""Fused LayerNorm forward with the reference module's interface
(energonai/kernel/cuda_native/layer_norm.py:16-78, apex-derived).

``MixedFusedLayerNorm`` keeps the constructor, parameters (``weight`` ones,
``bias`` zeros), ``forward`` and ``__repr__`` of the reference.  The kernel
computes in fp32 with one rounding at the store (the reference rounds the
normalised value to the output type before applying gamma and beta,
csrc/layer_norm_cuda_kernel.cu:266).  Inference only: a backward pass is not
provided and asking for one raises.

``layer_norm_forward`` is the functional form and adds the fused residual:
``y = LN(input + residual)`` in one pass, optionally also returning the sum
(the new residual stream of a pre-LN block) and the fp32 row statistics.
"""
from __future__ import annotations

import numbers

import torch
from torch.nn import init
from torch.nn.parameter import Parameter

from ... import _lib

_PAIRS = {
    (torch.float32, torch.float32), (torch.float32, torch.float16), (torch.float32, torch.bfloat16),
    (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
}


def _check_shapes(input, normalized_shape, weight, bias):
    """Mirrors check_args of csrc/layer_norm_cuda.cpp:26-66 (same messages)."""
    normalized_shape = tuple(normalized_shape)
    if len(normalized_shape) < 1:
        raise RuntimeError("Expected normalized_shape to be at least 1-dimensional, i.e., containing at least one "
                           f"element, but got normalized_shape={list(normalized_shape)}")
    if input.dim() < len(normalized_shape) or tuple(input.shape[input.dim() - len(normalized_shape):]) != normalized_shape:
        raise RuntimeError(f"Given normalized_shape={list(normalized_shape)}, expected input with shape [*, "
                           + ", ".join(str(s) for s in normalized_shape) + f"], but got input of size{list(input.shape)}")
    if tuple(weight.shape) != normalized_shape or tuple(bias.shape) != normalized_shape:
        raise RuntimeError("gamma and beta must have normalized_shape")
    n2 = 1
    for s in normalized_shape:
        n2 *= s
    return input.numel() // n2 if n2 else 0, n2


def layer_norm_forward(input, weight, bias, normalized_shape, eps=1e-5, residual=None, return_stats=False,
                       return_sum=False, residual_row_offsets=None):
    """forward_affine of the reference extension (csrc/layer_norm_cuda.cpp:82-103) plus a fused residual.

    Returns ``output`` (dtype of ``weight``), or a tuple
    ``(output[, mean, invvar][, sum])`` when the optional results are asked for.
    With ``residual_row_offsets`` (int32 ``[n1]`` on the device, ``SeqInfo.row_offsets``) the residual of row
    ``t`` is row ``t + offsets[t]`` of ``residual``, i.e. it is read straight from the padded ``[B,S,hid]``
    activations and no depad copy is needed.
    """
    if isinstance(normalized_shape, numbers.Integral):
        normalized_shape = (normalized_shape,)
    _lib.require_gpu(input, "input", contiguous=False)
    _lib.require_gpu(weight, "gamma", contiguous=False)
    _lib.require_gpu(bias, "beta", contiguous=False)
    input_ = input.contiguous()
    weight_ = weight.contiguous()
    bias_ = bias.contiguous()
    if weight_.dtype != bias_.dtype:
        raise RuntimeError("gamma and beta must share one dtype")
    if (input_.dtype, weight_.dtype) not in _PAIRS:
        raise RuntimeError(f"layer_norm: unsupported (input, output) dtypes ({input_.dtype}, {weight_.dtype})")
    n1, n2 = _check_shapes(input_, normalized_shape, weight_, bias_)
    res_ = None
    if residual is not None:
        _lib.require_gpu(residual, "residual", contiguous=False)
        if residual.dtype != input_.dtype or (residual_row_offsets is None and residual.shape != input_.shape):
            raise RuntimeError("residual must match input in shape and dtype")
        if residual_row_offsets is not None and (residual.shape[-1] != input_.shape[-1] or
                                                 residual_row_offsets.numel() < n1 or
                                                 residual_row_offsets.dtype != torch.int32):
            raise RuntimeError("residual_row_offsets must be int32 [rows] and residual [.., hidden]")
        res_ = residual.contiguous()
    output = torch.empty_like(input_, dtype=weight_.dtype)
    mean = invvar = sum_out = None
    if return_stats:
        mean = torch.empty(n1, dtype=torch.float32, device=input_.device)
        invvar = torch.empty_like(mean)
    if return_sum:
        sum_out = torch.empty_like(input_)
    with _lib.device_guard(input_):
        _lib.check(_lib.fn.en_layernorm_fwd(
            output.data_ptr(), _lib.ptr(mean), _lib.ptr(invvar), _lib.ptr(sum_out), input_.data_ptr(),
            _lib.ptr(res_), _lib.ptr(residual_row_offsets), weight_.data_ptr(), bias_.data_ptr(), n1, n2, float(eps),
            _lib.dtype_tag(input_, "layer_norm"), _lib.dtype_tag(weight_, "layer_norm"),
            _lib.stream_of(input_)), "layer_norm")
    extra = ()
    if return_stats:
        extra += (mean, invvar)
    if return_sum:
        extra += (sum_out,)
    return (output,) + extra if extra else output


class FusedLayerNormAffineFunction(torch.autograd.Function):
    """Forward only.  Under autocast the inputs are taken as fp32, as the
    reference's ``custom_fwd(cast_inputs=torch.float32)`` does (layer_norm.py:19)."""

    @staticmethod
    def forward(ctx, input, weight, bias, normalized_shape, eps):
        if torch.is_autocast_enabled():
            with torch.autocast(device_type="cuda", enabled=False):
                return layer_norm_forward(input.float(), weight.float(), bias.float(), normalized_shape, eps)
        return layer_norm_forward(input, weight, bias, normalized_shape, eps)

    @staticmethod
    def backward(ctx, grad_output):
        raise RuntimeError("MixedFusedLayerNorm is inference-only here: backward is not implemented")


class MixedFusedLayerNorm(torch.nn.Module):

    def __init__(self, normalized_shape, eps=1e-5, device=None, dtype=None):
        super(MixedFusedLayerNorm, self).__init__()
        try:
            _lib.load()
        except RuntimeError as exc:
            raise RuntimeError('MixedFusedLayerNorm requires cuda extensions') from exc
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.weight = Parameter(torch.empty(*normalized_shape, device=device, dtype=dtype))
        self.bias = Parameter(torch.empty(*normalized_shape, device=device, dtype=dtype))
        self.reset_parameters()

    def reset_parameters(self):
        init.ones_(self.weight)
        init.zeros_(self.bias)

    def forward(self, input, residual=None):
        if residual is not None:
            return layer_norm_forward(input, self.weight.detach(), self.bias.detach(), self.normalized_shape,
                                      self.eps, residual=residual)
        if torch.is_grad_enabled() and (input.requires_grad or self.weight.requires_grad):
            return FusedLayerNormAffineFunction.apply(input, self.weight, self.bias, self.normalized_shape, self.eps)
        return FusedLayerNormAffineFunction.forward(None, input, self.weight.detach(), self.bias.detach(),
                                                    self.normalized_shape, self.eps)

    def __repr__(self):
        return f'MixedFusedLayerNorm(normalized_shape={self.normalized_shape}, eps={self.eps})'
