"""One transformer layer's padding-removal hot path, composed from the kernel API.

    depad -> transpose_pad -> QK^T -> scale_mask_softmax -> PV -> transpose_depad
          -> residual + LayerNorm

This is the call sequence of the reference's BERT/GPT blocks
(examples/bert/bert.py:54-62,91-134, examples/gpt/gpt.py:93-137) with the dense
projections left to the caller: ``qkv_packed`` is what ``query_key_value``
returns, and the residual + LayerNorm consumes either the attention output
itself (when heads*size_per_head equals the LayerNorm width) or ``dense_out``,
the output of the row-parallel ``dense``.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .kernel import (attn_fused, attn_fused_packed, attn_pv, attn_pv_varlen, attn_qk, attn_qk_varlen, decode_attn, decode_pv, decode_qk,
                     depad, layer_norm_forward, scale_mask_softmax, scale_mask_softmax_packed, transpose_depad,
                     transpose_pad)
from . import _lib
from .kernel.attention import packed_scores_elems
from .seqinfo import SeqInfo, seq_info


# attn_pv reads a row of probabilities only as far as the row's own query sees, so the softmax writes no tail
SOFTMAX_TAIL_ROWS = 1


def three_kernel_form(causal: bool, dtype: torch.dtype, max_seq_len: int) -> str:
    """QK^T, softmax and PV as three kernels on packed operands: with the scores in the packed causal layout where
    that layout exists and is smaller than ``[B,H,S,S]``."""
    if causal and dtype in (torch.float16, torch.bfloat16) and max_seq_len >= 256:
        return "varlen_packed"
    return "varlen"


def default_attention_form(causal: bool, dtype: torch.dtype, max_seq_len: int, size_per_head: int,
                           scale: float = 1.0) -> str:
    """The form ``padding_removal_layer`` runs when the caller names none: the fused kernel on the packed
    projections wherever it applies (16-bit storage with heads of at most 128 channels in multiples of 8, fp32
    with heads of at most 64 in multiples of 4, a positive scale) -- the score tensor then never exists and the
    step is two launches -- else the three kernels."""
    if dtype in (torch.float16, torch.bfloat16) and size_per_head <= 128 and size_per_head % 8 == 0 and scale > 0:
        return "packed"
    if dtype == torch.float32 and size_per_head <= 64 and size_per_head % 4 == 0 and scale > 0:
        return "packed"      # the fp32 fused kernel (heads of up to 64 channels: the BERT-base shape)
    return three_kernel_form(causal, dtype, max_seq_len)


def padding_removal_layer(hidden_padded: torch.Tensor, qkv_packed: torch.Tensor, seq_lens, head_num: int,
                          size_per_head: int, gamma: torch.Tensor, beta: torch.Tensor, eps: float = 1e-5,
                          scale: Optional[float] = None, causal: bool = True, left_padded: bool = False,
                          dense_out: Optional[torch.Tensor] = None, sum_seq: Optional[int] = None,
                          keep: bool = False, fused_attention=None, fold_depad: Optional[bool] = None,
                          ctx_out: Optional[torch.Tensor] = None):
    """Runs the step on ``hidden_padded`` [B,S,hid] and ``qkv_packed`` [1,T,H,3D].

    Returns the normalised ``[1,T,hid]`` output, or a dict of every intermediate when ``keep`` is set.
    ``fused_attention`` picks how the attention core runs:

    ``False``            the reference's sequence of ops: transpose_pad, QK^T, scale_mask_softmax, PV,
                         transpose_depad on padded ``[B,H,S,*]`` tensors;
    ``"varlen"``         QK^T and PV read the packed projections and write the packed context directly
                         (row offsets): neither transpose runs, no padded tensor exists;
    ``"varlen_packed"``  the same with the scores in the packed causal layout (causal, 16-bit dtypes);
    ``True``             QK^T / softmax / PV in the single fused kernel on the padded buffer (16-bit dtypes
                         only); the score tensor is then never written;
    ``"packed"``         the fused kernel on the packed projections;
    ``None`` (default)   ``"packed"`` wherever the fused kernel applies (16-bit dtypes, heads of at most 128
                         channels), else the three kernels: ``"varlen_packed"`` under a causal mask with rows of
                         at least 256 keys, ``"varlen"`` otherwise; with ``keep`` the reference's sequence, whose
                         intermediates are the ones a caller can name.  (The packed score layout halves the score
                         tensor and keeps every row on whole 128-byte groups: the three kernels together take
                         415 -> 349 us on 2048-key rows, 461 -> 457 us on 1024-key rows; short rows would only grow.)

    ``fold_depad`` drops the depad launch: the LayerNorm takes its residual rows straight from
    ``hidden_padded`` (default: on, unless ``keep`` asks for the packed residual).  ``ctx_out``
    (``[1,T,H,D]``, not with ``keep``) receives the packed attention context, otherwise a temporary.
    The three-kernel forms compute every score, probability and context entry with the same arithmetic, so
    their results are bit-identical as long as the softmax gives a row the same lanes in both layouts (rows of
    up to 1024 keys); beyond that the row sums are added up in another order and the last bit may differ.
    """
    B, S, hid = hidden_padded.shape
    H, D = head_num, size_per_head
    info = seq_info(seq_lens, B, hidden_padded.device)
    T = info.total if sum_seq is None else int(sum_seq)
    scale = float(D) ** -0.5 if scale is None else scale
    if fused_attention is None:
        fused_attention = False if keep else default_attention_form(causal, hidden_padded.dtype, S, D, scale)
    if fold_depad is None:
        fold_depad = not keep
    if not keep:
        return _layer_one_call(hidden_padded, qkv_packed, info, B, S, H, D, hid, T, gamma, beta, eps, scale, causal,
                               left_padded, dense_out, fused_attention, fold_depad, ctx_out)
    if fold_depad:
        raise RuntimeError("padding_removal_layer: fold_depad has no intermediates to keep")

    x = depad(hidden_padded, B, info, left_padded=left_padded, sum_seq=T)
    if fused_attention in ("packed", "varlen", "varlen_packed"):
        probs = None
        if fused_attention == "packed":
            ctx_packed = attn_fused_packed(qkv_packed, B, S, info, H, D, scale=scale, causal=causal)
        else:
            pk = fused_attention == "varlen_packed"
            q, k, v = torch.chunk(qkv_packed.view(-1, H, 3 * D), 3, dim=-1)
            scores = attn_qk_varlen(q, k, B, S, info, causal=causal, packed_scores=pk)
            if pk:
                probs = scale_mask_softmax_packed(B, S, H, scores, info, scale=scale)
            else:
                probs = scale_mask_softmax(B, S, H, scores, info, scale=scale, causal=causal,
                                           tail_rows=SOFTMAX_TAIL_ROWS)
            ctx_packed = attn_pv_varlen(probs, v, B, S, info, causal=causal, packed_scores=pk)
        attn_out = ctx_packed.view(1, T, H * D) if dense_out is None else dense_out
        y = layer_norm_forward(attn_out, gamma, beta, (hid,), eps, residual=x)
        return dict(x=x, qkv=None, probs=probs, ctx=None, ctx_packed=ctx_packed, y=y)
    qkv = transpose_pad(qkv_packed, B, S, info, H, 3 * D)
    q, k, v = torch.chunk(qkv, 3, dim=-1)
    if fused_attention:
        probs = None
        ctx = attn_fused(q, k, v, info, scale=scale, causal=causal)
    else:
        scores = attn_qk(q, k, info, causal=causal)
        probs = scale_mask_softmax(B, S, H, scores, info, scale=scale, causal=causal, tail_rows=SOFTMAX_TAIL_ROWS)
        ctx = attn_pv(probs, v, info, causal=causal)
    ctx_packed = transpose_depad(ctx, B, T, S, info, H, D)
    attn_out = ctx_packed.view(1, T, H * D) if dense_out is None else dense_out
    y = layer_norm_forward(attn_out, gamma, beta, (hid,), eps, residual=x)
    return dict(x=x, qkv=qkv, probs=probs, ctx=ctx, ctx_packed=ctx_packed, y=y)


_FORMS = {False: 0, True: 1, "packed": 2, "varlen": 3, "varlen_packed": 4}


def _layer_one_call(hidden_padded, qkv_packed, info, B, S, H, D, hid, T, gamma, beta, eps, scale, causal, left_padded,
                    dense_out, fused_attention, fold_depad=False, ctx_out=None):
    """The same seven ops through ``en_padding_removal_layer``: one foreign call per step."""
    dev, dt = hidden_padded.device, hidden_padded.dtype
    form = _FORMS[fused_attention]
    _lib.require_gpu(hidden_padded, "hidden_padded")
    _lib.require_gpu(qkv_packed, "qkv_packed")
    if qkv_packed.numel() != T * H * 3 * D or qkv_packed.dtype != dt:
        raise RuntimeError("padding_removal_layer: qkv_packed must be [1,T,H,3D] of the activation dtype")
    if gamma.dtype != dt or beta.dtype != dt or gamma.numel() != hid or beta.numel() != hid:
        raise RuntimeError("padding_removal_layer: gamma and beta must be [hidden] of the activation dtype")
    if dense_out is not None:
        _lib.require_gpu(dense_out, "dense_out")
        if dense_out.numel() != T * hid or dense_out.dtype != dt:
            raise RuntimeError("padding_removal_layer: dense_out must be [1,T,hidden] of the activation dtype")
    elif hid != H * D:
        raise RuntimeError("padding_removal_layer: without dense_out the LayerNorm width must equal heads * size_per_head")
    if form == 4 and dt == torch.float32:
        raise RuntimeError("padding_removal_layer: the packed scores are for float16 and bfloat16")
    if form in (1, 2) and dt == torch.float32 and D > 64:
        raise RuntimeError("padding_removal_layer: the fused kernel takes float32 heads of up to 64 channels")
    if form == 4 and not causal:
        raise RuntimeError("padding_removal_layer: the packed score layout is that of a causal mask")
    x = None if fold_depad else torch.empty((1, T, hid), dtype=dt, device=dev)
    offs = info.row_offsets(S, left_padded) if fold_depad else None
    y = torch.empty((1, T, hid), dtype=dt, device=dev)
    if ctx_out is None:
        ctx_packed = torch.empty((1, T, H, D), dtype=dt, device=dev)
    else:
        _lib.require_gpu(ctx_out, "ctx_out")
        if ctx_out.numel() != T * H * D or ctx_out.dtype != dt or not ctx_out.is_contiguous():
            raise RuntimeError("padding_removal_layer: ctx_out must be a contiguous [1,T,H,D] tensor of the activation dtype")
        ctx_packed = ctx_out
    qkv = torch.empty((B, H, S, 3 * D), dtype=dt, device=dev) if form < 2 else None
    ctx = torch.empty((B, H, S, D), dtype=dt, device=dev) if form < 2 else None
    scores = None
    if form in (0, 3):
        scores = torch.empty((B, H, S, S), dtype=dt, device=dev)
    elif form == 4:
        scores = torch.empty(packed_scores_elems(B, H, S, dt), dtype=dt, device=dev)
    with _lib.device_guard(hidden_padded):
        _lib.check(_lib.fn.en_padding_removal_layer(
            hidden_padded.data_ptr(), qkv_packed.data_ptr(), _lib.ptr(dense_out), gamma.data_ptr(), beta.data_ptr(),
            _lib.ptr(x), _lib.ptr(qkv), _lib.ptr(scores), _lib.ptr(ctx), ctx_packed.data_ptr(), y.data_ptr(),
            info.cu_seqlens.data_ptr(), info.lens.data_ptr(), B, S, H, D, hid, T, float(scale), float(eps),
            int(bool(causal)), int(bool(left_padded)), form, _lib.ptr(offs),
            _lib.dtype_tag(hidden_padded, "padding_removal_layer"),
            info.tile_table_ptr(H, S, 2 * S * D * hidden_padded.element_size()),
            _lib.stream_of(hidden_padded)), "padding_removal_layer")
    return y


def padding_removal_layer_noalloc(hidden_padded: torch.Tensor, qkv_packed: torch.Tensor, seq_lens: torch.Tensor,
                                  head_num: int, size_per_head: int, gamma: torch.Tensor, beta: torch.Tensor,
                                  out: torch.Tensor, sum_seq: int, eps: float = 1e-5, scale: Optional[float] = None,
                                  causal: bool = True, left_padded: bool = False,
                                  dense_out: Optional[torch.Tensor] = None, fused_attention=False,
                                  fold_depad: bool = False) -> torch.Tensor:
    """The same step for callers that may not allocate device memory (a step recorded into a HIP graph, a tight
    serving loop): ``en_padding_removal_layer_noalloc`` keeps every intermediate, the sequence offsets included,
    in a static array inside the library (64 MiB per GPU; larger steps raise).  Nothing is allocated here
    either: ``seq_lens`` must already be a contiguous int32/int64 tensor on the device, ``sum_seq`` its total
    and ``out`` the ``[1,T,hid]`` result tensor.  Calls that overlap on one GPU share the array and race.
    """
    B, S, hid = hidden_padded.shape
    H, D = head_num, size_per_head
    T = int(sum_seq)
    dt = hidden_padded.dtype
    for t, name in ((hidden_padded, "hidden_padded"), (qkv_packed, "qkv_packed"), (seq_lens, "seq_lens"), (out, "out"),
                    (gamma, "gamma"), (beta, "beta")):
        _lib.require_gpu(t, name)
    if seq_lens.dtype not in (torch.int32, torch.int64) or seq_lens.numel() < B:
        raise RuntimeError("padding_removal_layer_noalloc: seq_lens must hold batch int32 or int64 lengths")
    if qkv_packed.numel() != T * H * 3 * D or qkv_packed.dtype != dt or not qkv_packed.is_contiguous():
        raise RuntimeError("padding_removal_layer_noalloc: qkv_packed must be a contiguous [1,T,H,3D] tensor of the "
                           "activation dtype")
    if out.numel() != T * hid or out.dtype != dt or not out.is_contiguous():
        raise RuntimeError("padding_removal_layer_noalloc: out must be a contiguous [1,T,hidden] tensor of the "
                           "activation dtype")
    if not hidden_padded.is_contiguous() or not seq_lens.is_contiguous():
        raise RuntimeError("padding_removal_layer_noalloc: hidden_padded and seq_lens must be contiguous")
    if gamma.dtype != dt or beta.dtype != dt or gamma.numel() != hid or beta.numel() != hid:
        raise RuntimeError("padding_removal_layer_noalloc: gamma and beta must be [hidden] of the activation dtype")
    if dense_out is not None:
        _lib.require_gpu(dense_out, "dense_out")
        if dense_out.numel() != T * hid or dense_out.dtype != dt or not dense_out.is_contiguous():
            raise RuntimeError("padding_removal_layer_noalloc: dense_out must be a contiguous [1,T,hidden] tensor of the "
                               "activation dtype")
    elif hid != H * D:
        raise RuntimeError("padding_removal_layer_noalloc: without dense_out the LayerNorm width must equal "
                           "heads * size_per_head")
    scale = float(D) ** -0.5 if scale is None else scale
    with _lib.device_guard(hidden_padded):
        _lib.check(_lib.fn.en_padding_removal_layer_noalloc(
            hidden_padded.data_ptr(), qkv_packed.data_ptr(), _lib.ptr(dense_out), gamma.data_ptr(), beta.data_ptr(),
            out.data_ptr(), seq_lens.data_ptr(), int(seq_lens.dtype == torch.int64), B, S, H, D, hid, T, float(scale),
            float(eps), int(bool(causal)), int(bool(left_padded)), _FORMS[fused_attention], int(bool(fold_depad)),
            _lib.dtype_tag(hidden_padded, "padding_removal_layer_noalloc"), _lib.stream_of(hidden_padded)),
            "padding_removal_layer_noalloc")
    return out


def decode_layer(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, kv_lens, residual: torch.Tensor,
                 gamma: torch.Tensor, beta: torch.Tensor, eps: float = 1e-5, scale: Optional[float] = None,
                 dense_out: Optional[torch.Tensor] = None, keep: bool = False, single_pass: Optional[bool] = None):
    """One cached decode step: a single new query per sequence against a ragged
    cache, then residual + LayerNorm on the B new tokens (transpose_depad of a
    one-row sequence is the identity, so the context is passed on as a view).

    q [B,H,1,D]; caches [B,H,Smax,D]; residual [1,B,hid].  ``single_pass`` (default: on, unless ``keep`` asks
    for the probabilities) runs QK^T, softmax and PV as one kernel that reads K and V once and writes no scores:
    two launches per step.  Otherwise ``decode_qk`` -> ``scale_mask_softmax`` -> ``decode_pv``, four launches.
    """
    B, H, _, D = q.shape
    Smax = k_cache.shape[2]
    hid = gamma.numel()
    info = seq_info(kv_lens, B, q.device)
    scale = float(D) ** -0.5 if scale is None else scale
    if single_pass is None:
        single_pass = not keep and scale > 0
    probs = None
    if single_pass:
        ctx = decode_attn(q, k_cache, v_cache, info, scale=scale)
    else:
        ones = _ones_info(B, q.device)
        scores = decode_qk(q, k_cache, info)
        probs = scale_mask_softmax(B, 1, H, scores, info, scale=scale, causal=True, k_seq_len=Smax, q_len_list=ones)
        ctx = decode_pv(probs, v_cache, info)
    ctx_packed = ctx.view(1, B, H, D)      # [B,H,1,D] with one query per sequence is [1,T=B,H,D] already
    attn_out = ctx_packed.view(1, B, H * D) if dense_out is None else dense_out
    y = layer_norm_forward(attn_out, gamma, beta, (hid,), eps, residual=residual)
    if keep:
        return dict(scores_probs=probs, ctx=ctx, ctx_packed=ctx_packed, y=y)
    return y


_ones_cache: Dict[tuple, SeqInfo] = {}


def _ones_info(batch: int, device) -> SeqInfo:
    key = (batch, str(device))
    info = _ones_cache.get(key)
    if info is None:
        info = seq_info(torch.ones(batch, dtype=torch.int32), batch, device)
        _ones_cache[key] = info
    return info
