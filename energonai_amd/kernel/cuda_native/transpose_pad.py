"""Packing / unpacking ops with the reference's names and signatures
(energonai/kernel/cuda_native/transpose_pad.py:12-87).

Differences from the reference, all backwards compatible:

* ``seq_len_list`` may be int32 or int64 (the reference test passes int64 to
  kernels that read int32), a CPU tensor, a list, or a prebuilt
  :class:`energonai_amd.seqinfo.SeqInfo`;
* outputs are allocated uninitialised and every byte is written by one kernel
  (the reference zero-fills with ``torch::zeros`` and then writes again);
* kernels run on torch's current stream, not the legacy default stream;
* ``depad`` is one kernel instead of a Python loop of ``torch.cat`` and takes
  ``left_padded=True`` for batches padded on the left (OPT).
"""
from __future__ import annotations

import operator

import torch

from ... import _lib
from ...seqinfo import SeqInfo, seq_info

try:
    _lib.load()
except RuntimeError as _exc:  # same failure mode as the reference at import
    raise RuntimeError('transpose_pad requires cuda extensions') from _exc


def _as_int(x) -> int:
    """sum_seq / valid_word_num arrive as Python ints or 0-d tensors (examples/bert/bert.py:122-123)."""
    if isinstance(x, torch.Tensor):
        return int(x.item())
    return operator.index(x)


def _elem_size(t: torch.Tensor, op: str) -> int:
    if t.element_size() not in (2, 4):
        raise RuntimeError(f"{op}: Datatype not implemented ({t.dtype})")
    return t.element_size()


def _int32_gpu(t: torch.Tensor, name: str) -> torch.Tensor:
    _lib.require_gpu(t, name)
    if t.dtype != torch.int32:
        raise RuntimeError(f"{name} must be an int32 tensor")
    return t


def transpose_pad(src, batch_size, max_seq_len, seq_len_list, head_num, size_per_head, zero_padding=True):
    """[1,T,H,Dk] -> zero-padded [B,H,S,Dk]  (transpose_pad.py:12-18).

    ``zero_padding=False`` (not in the reference) writes the valid rows only and leaves the padding rows of the
    new tensor uninitialised: for callers whose consumers are bounded by the sequence lengths, as the attention
    kernels of this package are.
    """
    src = src.contiguous()
    _lib.require_gpu(src, "src")
    info = seq_info(seq_len_list, batch_size, src.device)
    if src.numel() % (head_num * size_per_head) != 0:
        raise RuntimeError("transpose_pad: src size is not a multiple of head_num * size_per_head")
    dst = torch.empty((batch_size, head_num, max_seq_len, size_per_head), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src):
        if zero_padding:
            rc = _lib.fn.en_transpose_pad(src.data_ptr(), dst.data_ptr(), info.cu_seqlens.data_ptr(), batch_size,
                                          max_seq_len, head_num, size_per_head, _elem_size(src, "transpose_pad"),
                                          _lib.stream_of(src))
        else:
            rc = _lib.fn.en_transpose_pad_heads(src.data_ptr(), dst.data_ptr(), info.cu_seqlens.data_ptr(), batch_size,
                                                max_seq_len, head_num, size_per_head, head_num, 0, 0,
                                                _elem_size(src, "transpose_pad"), _lib.stream_of(src))
        _lib.check(rc, "transpose_pad")
    return dst


def transpose_depad(src, batch_size, sum_seq, max_seq_len, seq_len_list, head_num, size_per_head):
    """[B,H,S,D] -> [1,T,H,D]  (transpose_pad.py:21-27)."""
    src = src.contiguous()
    _lib.require_gpu(src, "src")
    info = seq_info(seq_len_list, batch_size, src.device)
    total = _as_int(sum_seq)
    if src.numel() != batch_size * head_num * max_seq_len * size_per_head:
        raise RuntimeError("transpose_depad: src does not have batch*head*seq*size_per_head elements")
    dst = torch.empty((1, total, head_num, size_per_head), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_transpose_depad(src.data_ptr(), dst.data_ptr(), info.cu_seqlens.data_ptr(),
                                                  batch_size, max_seq_len, head_num, size_per_head,
                                                  _elem_size(src, "transpose_depad"), _lib.stream_of(src)),
                   "transpose_depad")
    return dst


def depad(src, batch_size, seq_lens, left_padded=False, sum_seq=None):
    """[B,S,hid] -> [1,T,hid]  (transpose_pad.py:30-37).

    ``sum_seq`` (optional) is the known total length; without it the total is
    read from the device once per distinct ``seq_lens`` (the reference's slicing
    with tensor lengths synchronises on every sequence).
    """
    _lib.require_gpu(src, "src", contiguous=False)
    src = src.contiguous()
    if src.dim() != 3:
        raise RuntimeError("depad: src must be [batch, seq, hidden]")
    info = seq_info(seq_lens, batch_size, src.device)
    total = info.total if sum_seq is None else _as_int(sum_seq)
    S, hid = src.shape[1], src.shape[2]
    dst = torch.empty((1, total, hid), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_depad(src.data_ptr(), dst.data_ptr(), info.cu_seqlens.data_ptr(), batch_size, S,
                                        hid, _elem_size(src, "depad"), int(bool(left_padded)), _lib.stream_of(src)),
                   "depad")
    return dst


def repad(src, batch_size, max_seq_len, seq_lens, left_padded=False):
    """[1,T,hid] -> [B,S,hid] with zero padding rows: the inverse of :func:`depad`.

    An addition for the exit of the packed path; the reference callers rebuild
    right-padded batches with ``ft_rebuild_padding`` (examples/gpt/gpt.py:321-323)
    while their generation batches are left-padded (examples/opt/batch.py:12-24).
    """
    _lib.require_gpu(src, "src", contiguous=False)
    src = src.contiguous()
    hid = src.shape[-1]
    info = seq_info(seq_lens, batch_size, src.device)
    if src.numel() % hid != 0 or src.dim() < 2:
        raise RuntimeError("repad: src must be [1, total, hidden]")
    S = _as_int(max_seq_len)
    dst = torch.empty((batch_size, S, hid), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_repad(src.data_ptr(), dst.data_ptr(), info.cu_seqlens.data_ptr(), batch_size, S, hid,
                                    _elem_size(src, "repad"), int(bool(left_padded)), _lib.stream_of(src)), "repad")
    return dst


# From FasterTransformer


def ft_build_padding_offsets(seq_lens, batch_size, max_seq_len, valid_word_num, tmp_mask_offset):
    """Writes valid_word_num[0] and tmp_mask_offset[:T] in place  (transpose_pad.py:43-48)."""
    seq_lens = seq_lens.contiguous()
    _lib.require_gpu(seq_lens, "sequence_length")
    _int32_gpu(valid_word_num, "valid_word_num")
    _int32_gpu(tmp_mask_offset, "tmp_mask_offset")
    if seq_lens.dtype == torch.int64:
        seq_lens = seq_info(seq_lens, batch_size).lens
    elif seq_lens.dtype != torch.int32:
        raise RuntimeError("sequence_length must be an int32 or int64 tensor")
    if tmp_mask_offset.numel() < batch_size * max_seq_len:
        raise RuntimeError("tmp_mask_offset must hold batch_size * max_seq_len entries")
    with _lib.device_guard(seq_lens):
        _lib.check(_lib.fn.en_ft_build_offsets(seq_lens.data_ptr(), batch_size, max_seq_len,
                                                   valid_word_num.data_ptr(), tmp_mask_offset.data_ptr(),
                                                   _lib.stream_of(seq_lens)), "ft_build_padding_offsets")


def ft_remove_padding(src, tmp_mask_offset, mask_offset, valid_word_num, hidden_dim):
    """[B,S,hid] -> [1,valid,hid]; also fills mask_offset  (transpose_pad.py:51-57)."""
    src = src.contiguous()
    _lib.require_gpu(src, "src")
    _int32_gpu(tmp_mask_offset, "tmp_mask_offset")
    _int32_gpu(mask_offset, "mask_offset")
    valid = _as_int(valid_word_num)
    if mask_offset.numel() < valid or tmp_mask_offset.numel() < valid:
        raise RuntimeError("ft_remove_padding: offset tensors are shorter than valid_word_num")
    tgt = torch.empty((1, valid, hidden_dim), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_ft_remove_padding(src.data_ptr(), tgt.data_ptr(), tmp_mask_offset.data_ptr(),
                                                    mask_offset.data_ptr(), valid, hidden_dim,
                                                    _elem_size(src, "ft_remove_padding"), _lib.stream_of(src)),
                   "ft_remove_padding")
    return tgt


def ft_rebuild_padding(src, mask_offset, valid_word_num, hidden_dim, batch_size, max_seq_len):
    """[1,valid,hid] -> [B,S,hid] with zero padding rows  (transpose_pad.py:60-66)."""
    src = src.contiguous()
    _lib.require_gpu(src, "src")
    _int32_gpu(mask_offset, "mask_offset")
    valid = _as_int(valid_word_num)
    if mask_offset.numel() < valid:
        raise RuntimeError("ft_rebuild_padding: mask_offset is shorter than valid_word_num")
    tgt = torch.empty((batch_size, max_seq_len, hidden_dim), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_ft_rebuild_padding(src.data_ptr(), tgt.data_ptr(), mask_offset.data_ptr(), valid,
                                                     hidden_dim, batch_size, max_seq_len,
                                                     _elem_size(src, "ft_rebuild_padding"), _lib.stream_of(src)),
                   "ft_rebuild_padding")
    return tgt


def ft_transpose_rebuild_padding(Q, K, V, q_buf, k_buf, v_buf, batch_size, seq_len, head_num, size_per_head,
                                 valid_word_num, mask_offset):
    """Q,K,V [valid,H,D] scattered into caller-owned [B,H,S,D] buffers  (transpose_pad.py:69-79).

    The buffers are written in place, so they must already be contiguous (the
    reference calls ``.contiguous()`` on them, which would silently write into
    a temporary for a strided buffer).
    """
    Q, K, V = Q.contiguous(), K.contiguous(), V.contiguous()
    for t, name in ((Q, "Q"), (K, "K"), (V, "V"), (q_buf, "q_buf"), (k_buf, "k_buf"), (v_buf, "v_buf")):
        _lib.require_gpu(t, name)
        if t.dtype != Q.dtype:
            raise RuntimeError("ft_transpose_rebuild_padding: all tensors must share one dtype")
    _int32_gpu(mask_offset, "mask_offset")
    valid = _as_int(valid_word_num)
    need = batch_size * head_num * seq_len * size_per_head
    if min(q_buf.numel(), k_buf.numel(), v_buf.numel()) < need:
        raise RuntimeError("ft_transpose_rebuild_padding: buffers are smaller than [B,H,S,D]")
    with _lib.device_guard(Q):
        _lib.check(_lib.fn.en_ft_transpose_rebuild(Q.data_ptr(), K.data_ptr(), V.data_ptr(), q_buf.data_ptr(),
                                                       k_buf.data_ptr(), v_buf.data_ptr(), batch_size, seq_len,
                                                       head_num, size_per_head, valid, mask_offset.data_ptr(),
                                                       _elem_size(Q, "ft_transpose_rebuild_padding"),
                                                       _lib.stream_of(Q)), "ft_transpose_rebuild_padding")


def ft_transpose_remove_padding(src, valid_word_num, batch_size, seq_len, head_num, size_per_head, mask_offset):
    """[B,H,S,D] -> [1,valid,H*D]  (transpose_pad.py:82-87)."""
    src = src.contiguous()
    _lib.require_gpu(src, "src")
    _int32_gpu(mask_offset, "mask_offset")
    valid = _as_int(valid_word_num)
    dst = torch.empty((1, valid, head_num * size_per_head), dtype=src.dtype, device=src.device)
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_ft_transpose_remove(src.data_ptr(), dst.data_ptr(), valid, batch_size, seq_len,
                                                      head_num, size_per_head, mask_offset.data_ptr(),
                                                      _elem_size(src, "ft_transpose_remove_padding"),
                                                      _lib.stream_of(src)), "ft_transpose_remove_padding")
    return dst
