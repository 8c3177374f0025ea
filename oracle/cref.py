"""ctypes front end of oracle/_build/liboracle_c.so (test oracle only).

TEST INFRASTRUCTURE ONLY.  Wraps the plain-C replay of the reference kernels
(oracle/kernels_ref.c) so tests can call it on torch CPU tensors.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle_c.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(t: torch.Tensor) -> ctypes.c_void_p:
    assert t.device.type == "cpu" and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _i32(x) -> torch.Tensor:
    return torch.as_tensor(x).to(torch.int32).contiguous()


def transpose_pad(src, B, S, lens, H, D):
    lens = _i32(lens)
    src = src.contiguous()
    dst = torch.full((B, H, S, D), 7, dtype=src.dtype)
    lib().orc_transpose_pad(_p(src), _p(dst), _p(lens), B, S, H, D, src.element_size())
    return dst


def transpose_depad(src, B, T, S, lens, H, D):
    lens = _i32(lens)
    src = src.contiguous()
    dst = torch.zeros((1, T, H, D), dtype=src.dtype)
    lib().orc_transpose_depad(_p(src), _p(dst), _p(lens), B, S, H, D, src.element_size())
    return dst


def build_offsets(lens, B, S):
    lens = _i32(lens)
    valid = torch.zeros(1, dtype=torch.int32)
    off = torch.zeros(B * S, dtype=torch.int32)
    lib().orc_build_offsets(_p(lens), B, S, _p(valid), _p(off))
    return valid, off[: int(valid[0])].clone()


def remove_padding(src, tmp_off, valid, hid):
    src = src.contiguous()
    tmp_off = _i32(tmp_off)
    mask_off = torch.zeros(valid, dtype=torch.int32)
    tgt = torch.zeros((1, valid, hid), dtype=src.dtype)
    lib().orc_remove_padding(_p(src), _p(tgt), _p(tmp_off), _p(mask_off), valid, hid, src.element_size())
    return tgt, mask_off


def rebuild_padding(src, mask_off, valid, hid, B, S):
    src = src.contiguous()
    mask_off = _i32(mask_off)
    tgt = torch.zeros((B, S, hid), dtype=src.dtype)
    lib().orc_rebuild_padding(_p(src), _p(tgt), _p(mask_off), valid, hid, src.element_size())
    return tgt


def transpose_rebuild_padding(Q, buf, S, H, D, mask_off, valid):
    Q = Q.contiguous()
    mask_off = _i32(mask_off)
    lib().orc_transpose_rebuild_padding(_p(Q), _p(buf), S, H, D, _p(mask_off), valid, Q.element_size())


def transpose_remove_padding(src, S, H, D, mask_off, valid):
    src = src.contiguous()
    mask_off = _i32(mask_off)
    dst = torch.zeros((1, valid, H * D), dtype=src.dtype)
    lib().orc_transpose_remove_padding(_p(src), _p(dst), S, H, D, _p(mask_off), valid, src.element_size())
    return dst


def softmax_f32(src, lens, B, H, S):
    out = src.detach().clone().float().contiguous()
    lens = _i32(lens)
    lib().orc_softmax_f32(_p(out), _p(lens), B, H, S)
    return out


def layer_norm_f32(x, gamma, beta, eps):
    n2 = gamma.numel()
    xs = x.detach().float().reshape(-1, n2).contiguous()
    n1 = xs.shape[0]
    out = torch.empty_like(xs)
    mean = torch.empty(n1, dtype=torch.float32)
    invvar = torch.empty(n1, dtype=torch.float32)
    g = gamma.detach().float().contiguous()
    b = beta.detach().float().contiguous()
    lib().orc_layer_norm_f32(_p(out), _p(mean), _p(invvar), _p(xs), n1, n2, ctypes.c_float(eps), _p(g), _p(b))
    return out.reshape(x.shape), mean, invvar
