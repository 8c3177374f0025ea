"""scale + mask + softmax with the reference's signature
(energonai/kernel/cuda_native/scale_mask_softmax.py:10-13).

The five positional arguments behave exactly like the reference kernel
(csrc/scale_mask_softmax_kernel.cu:11-42): in place on ``src`` [B,H,S,S], causal,
no scaling, rows of padded queries left untouched, the same tensor returned.
Keyword extensions (defaults preserve the reference behaviour):

``scale``      multiply scores before the softmax (the reference name promises a
               scale but the kernel applies none; callers pre-scale)
``causal``     False masks only keys >= len[b] (BERT key-padding mask)
``k_seq_len``  key extent when src is rectangular [B,H,batch_seq_len,k_seq_len]
``q_len_list`` valid query rows per sequence when they differ from the key
               lengths (decode: one query against a longer cache)
``tail_rows``  0 zeroes the whole masked tail of each row (reference); a power of
               two n zeroes only up to what the last row of the row's n-row tile
               sees and leaves the rest untouched.  1 writes just the visible
               prefix (to the end of its last 16-byte vector), which is all that
               ``attn_pv`` reads of a row

There is no limit on the sequence length (the reference cannot launch above
1024) and offsets are 64-bit.
"""
from __future__ import annotations

import torch

from ... import _lib
from ...seqinfo import seq_info

try:
    _lib.load()
except RuntimeError as _exc:
    raise RuntimeError('energonai_scale_mask requires cuda extensions') from _exc


def scale_mask_softmax(batch_size, batch_seq_len, head_num, src, seq_len_list, *, scale=1.0, causal=True,
                       k_seq_len=None, q_len_list=None, tail_rows=0):
    _lib.require_gpu(src, "correlation", contiguous=False)
    if src.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise RuntimeError("Datatype not implemented")
    if not src.is_contiguous():
        # the reference would run on a contiguous copy and return that copy
        src = src.contiguous()
    k_seq_len = batch_seq_len if k_seq_len is None else int(k_seq_len)
    if src.numel() != batch_size * head_num * batch_seq_len * k_seq_len:
        raise RuntimeError("scale_mask_softmax: src does not have batch*head*q_seq*k_seq elements")
    k_info = seq_info(seq_len_list, batch_size, src.device)
    q_ptr = 0
    if q_len_list is not None:
        q_info = seq_info(q_len_list, batch_size, src.device)
        q_ptr = q_info.lens.data_ptr()
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_scale_mask_softmax(src.data_ptr(), k_info.lens.data_ptr(), q_ptr, batch_size,
                                                     head_num, batch_seq_len, k_seq_len, float(scale),
                                                     int(bool(causal)), int(tail_rows), _lib.dtype_tag(src, "scale_mask_softmax"),
                                                     _lib.stream_of(src)), "scale_mask_softmax")
    return src
