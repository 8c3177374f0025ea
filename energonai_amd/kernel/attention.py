"""The two attention contractions of the padding-removal path.

The reference callers use ``torch.matmul`` on the padded ``[B,H,S,*]`` tensors
(examples/bert/bert.py:108-119, examples/gpt/gpt.py:108-125) and therefore pay
for every padded row and every masked key.  ``attn_qk`` / ``attn_pv`` compute
only what the softmax uses: valid query rows and, under a causal mask, the keys
at or left of the diagonal.  ``q``, ``k`` and ``v`` may be the strided
``chunk(3, -1)`` views of the fused ``[B,H,S,3D]`` buffer; no copy is made.
``decode_qk`` / ``decode_pv`` are the single-query forms for cached decode.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .. import _lib
from ..seqinfo import seq_info


def _bhsd(t: torch.Tensor, name: str):
    _lib.require_gpu(t, name, contiguous=False)
    if t.dim() != 4:
        raise RuntimeError(f"{name} must be [batch, head, seq, size_per_head]")
    if t.stride(3) != 1:
        raise RuntimeError(f"{name}: the last dimension must be contiguous")
    return t.stride(0), t.stride(1), t.stride(2)


def _lens_ptrs(seq_len_list, q_len_list, batch_size, device):
    """Key lengths, query lengths (or None) and the raw pointer of the latter.  The caller keeps both objects
    until its kernel is launched: lengths given as a list live in a device tensor that only they own, and a
    tensor allocated in between could otherwise be handed the same memory."""
    k_info = seq_info(seq_len_list, batch_size, device)
    q_info = None if q_len_list is None else seq_info(q_len_list, batch_size, device)
    return k_info, q_info, (0 if q_info is None else q_info.lens.data_ptr())


def _unit_kv_bytes(k_seq_len: int, size_per_head: int, t: torch.Tensor) -> int:
    """Bytes of one (batch, head) unit's K and V at full length: picks the workgroup order (SeqInfo.tile_table)."""
    return 2 * int(k_seq_len) * int(size_per_head) * t.element_size()


def _tile_table_ptr(k_info, q_ptr, head_num: int, q_seq_len: int, unit_kv_bytes: int, query_tile: int = 128):
    """Workgroup order for the batch (cached in its SeqInfo) when the query lengths are the key lengths."""
    return None if q_ptr else k_info.tile_table_ptr(head_num, q_seq_len, unit_kv_bytes, query_tile)


def _fused_dtype_ok(t: torch.Tensor, size_per_head: int, who: str) -> None:
    """float16 / bfloat16 with heads of up to 128 channels, float32 with heads of up to 64."""
    if t.dtype in (torch.float16, torch.bfloat16):
        return
    if t.dtype == torch.float32 and size_per_head <= 64:
        return
    raise RuntimeError(f"{who}: Datatype not implemented (float16 and bfloat16; float32 for heads of up to 64 channels)")


def fused_query_tile(q_seq_len: int, k_seq_len: int, size_per_head: int, causal: bool, t: torch.Tensor,
                     query_tile: Optional[int] = None) -> int:
    """Query rows per workgroup of the fused kernel: the caller's choice (128, or 256 for the form with 64
    queries per wave, heads of 65..128 channels) or what the library picks for the shape."""
    if query_tile and t.dtype != torch.float32:
        if query_tile not in (128, 256) or (query_tile == 256 and size_per_head <= 64):
            raise RuntimeError("attn_fused: query_tile must be 128, or 256 for heads of 65..128 channels")
        return int(query_tile)
    return int(_lib.fn.en_attn_fused_query_tile(int(q_seq_len), int(k_seq_len), int(size_per_head), int(bool(causal)),
                                                _lib.dtype_tag(t, "attn_fused")))


def attn_qk(q, k, seq_len_list, *, alpha: float = 1.0, causal: bool = True, q_len_list=None,
            out: Optional[torch.Tensor] = None):
    """scores[b,h,i,j] = alpha * <q[b,h,i,:], k[b,h,j,:]> as a new ``[B,H,Sq,Sk]`` tensor.

    Only rows of valid queries and (rounded up to a 16-byte vector) the keys
    they can see are written; the rest of ``scores`` is uninitialised, exactly
    the region ``scale_mask_softmax`` never reads.
    """
    qs = _bhsd(q, "q")
    ks = _bhsd(k, "k")
    B, H, Sq, D = q.shape
    if k.shape[0] != B or k.shape[1] != H or k.shape[3] != D or k.dtype != q.dtype:
        raise RuntimeError("attn_qk: q and k disagree in batch, heads, size_per_head or dtype")
    Sk = k.shape[2]
    k_info, q_info, q_ptr = _lens_ptrs(seq_len_list, q_len_list, B, q.device)
    if out is None:
        out = torch.empty((B, H, Sq, Sk), dtype=q.dtype, device=q.device)
    else:
        _lib.require_gpu(out, "out")
        if out.shape != (B, H, Sq, Sk) or out.dtype != q.dtype:
            raise RuntimeError("attn_qk: out must be a contiguous [B,H,Sq,Sk] tensor of q's dtype")
    with _lib.device_guard(q):
        _lib.check(_lib.fn.en_attn_qk(q.data_ptr(), k.data_ptr(), out.data_ptr(), k_info.lens.data_ptr(), q_ptr,
                                          B, H, Sq, Sk, D, *qs, *ks, float(alpha), int(bool(causal)),
                                          _lib.dtype_tag(q, "attn_qk"), None, None, 0,
                                          _tile_table_ptr(k_info, q_ptr, H, Sq, _unit_kv_bytes(Sk, D, q)), _lib.stream_of(q)), "attn_qk")
    return out


def attn_pv(p, v, seq_len_list, *, causal: bool = True, q_len_list=None, zero_padding: bool = False,
            out: Optional[torch.Tensor] = None):
    """ctx[b,h,i,:] = sum_j p[b,h,i,j] v[b,h,j,:] as ``[B,H,Sq,D]``; ``p`` as left by scale_mask_softmax.

    Rows of padded queries are left uninitialised unless ``zero_padding``.
    """
    _lib.require_gpu(p, "p")
    vs = _bhsd(v, "v")
    if p.dim() != 4:
        raise RuntimeError("p must be [batch, head, q_seq, k_seq]")
    B, H, Sq, Sk = p.shape
    D = v.shape[3]
    if v.shape[0] != B or v.shape[1] != H or v.shape[2] != Sk or v.dtype != p.dtype:
        raise RuntimeError("attn_pv: p and v disagree in batch, heads, key length or dtype")
    k_info, q_info, q_ptr = _lens_ptrs(seq_len_list, q_len_list, B, p.device)
    if out is None:
        out = torch.empty((B, H, Sq, D), dtype=p.dtype, device=p.device)
    else:
        _bhsd(out, "out")
        if out.shape != (B, H, Sq, D) or out.dtype != p.dtype:
            raise RuntimeError("attn_pv: out must be [B,H,Sq,D] of p's dtype")
    cs = (out.stride(0), out.stride(1), out.stride(2))
    with _lib.device_guard(p):
        _lib.check(_lib.fn.en_attn_pv(p.data_ptr(), v.data_ptr(), out.data_ptr(), k_info.lens.data_ptr(), q_ptr,
                                          B, H, Sq, Sk, D, *vs, *cs, int(bool(causal)), int(bool(zero_padding)),
                                          _lib.dtype_tag(p, "attn_pv"), None, None, 0,
                                          _tile_table_ptr(k_info, q_ptr, H, Sq, _unit_kv_bytes(Sk, D, p)), _lib.stream_of(p)), "attn_pv")
    return out


def attn_fused(q, k, v, seq_len_list, *, scale: Optional[float] = None, causal: bool = True, q_len_list=None,
               out: Optional[torch.Tensor] = None, query_tile: Optional[int] = None):
    """ctx = softmax(scale * q k^T, mask) v in one kernel; the score tensor is never materialised.

    Same masking rule as ``scale_mask_softmax`` (``causal``, key lengths, optional query lengths);
    ``scale`` defaults to ``size_per_head ** -0.5``.  fp16 / bf16 (heads of up to 128 channels) and fp32 (up to 64).
    Returns ``[B,H,Sq,D]``; rows of
    padded queries are left uninitialised.  ``query_tile``: see :func:`fused_query_tile`.
    """
    qs = _bhsd(q, "q")
    ks = _bhsd(k, "k")
    vs = _bhsd(v, "v")
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    if k.shape != (B, H, Sk, D) or v.shape != (B, H, Sk, D) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("attn_fused: q, k, v disagree in batch, heads, size_per_head, key length or dtype")
    _fused_dtype_ok(q, D, "attn_fused")
    k_info, q_info, q_ptr = _lens_ptrs(seq_len_list, q_len_list, B, q.device)
    if out is None:
        out = torch.empty((B, H, Sq, D), dtype=q.dtype, device=q.device)
    else:
        _bhsd(out, "out")
        if out.shape != (B, H, Sq, D) or out.dtype != q.dtype:
            raise RuntimeError("attn_fused: out must be [B,H,Sq,D] of q's dtype")
    cs = (out.stride(0), out.stride(1), out.stride(2))
    arr = ctypes.c_int64 * 3
    scale = float(D) ** -0.5 if scale is None else float(scale)
    qt = fused_query_tile(Sq, Sk, D, causal, q, query_tile)
    with _lib.device_guard(q):
        _lib.check(_lib.fn.en_attn_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                         k_info.lens.data_ptr(), q_ptr, B, H, Sq, Sk, D, arr(*qs), arr(*ks), arr(*vs),
                                         arr(*cs), None, None, scale, int(bool(causal)),
                                         _lib.dtype_tag(q, "attn_fused"),
                                         None if qt == 64 else _tile_table_ptr(k_info, q_ptr, H, Sq, _unit_kv_bytes(Sk, D, q), qt),
                                         qt, _lib.stream_of(q)), "attn_fused")
    return out


def _thd(t: torch.Tensor, name: str):
    _lib.require_gpu(t, name, contiguous=False)
    if t.dim() != 3 or t.stride(2) != 1:
        raise RuntimeError(f"{name} must be a [tokens, head, size_per_head] view with contiguous channels")
    return 0, t.stride(1), t.stride(0)


def attn_fused_varlen(q, k, v, batch_size: int, max_seq_len: int, seq_len_list, *, scale: Optional[float] = None,
                      causal: bool = True, out: Optional[torch.Tensor] = None, query_tile: Optional[int] = None):
    """Self-attention on packed tokens: ``q``, ``k``, ``v`` are ``[T,H,D]`` views (any token and head
    strides) of the projection output, the result is the packed context ``[1,T,H,D]``.  Batch ``b``
    occupies rows ``cu_seqlens[b] .. cu_seqlens[b+1]``; no padded tensor is built.  fp16 / bf16 only.
    """
    qs, ks, vs = _thd(q, "q"), _thd(k, "k"), _thd(v, "v")
    T, H, D = q.shape
    if k.shape != q.shape or v.shape != q.shape or k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("attn_fused_varlen: q, k, v disagree in shape or dtype")
    _fused_dtype_ok(q, D, "attn_fused_varlen")
    info = seq_info(seq_len_list, batch_size, q.device)
    if out is None:
        out = torch.empty((1, T, H, D), dtype=q.dtype, device=q.device)
    elif out.numel() != T * H * D or out.dtype != q.dtype or not out.is_contiguous():
        raise RuntimeError("attn_fused_varlen: out must be contiguous [1,T,H,D] of q's dtype")
    arr = ctypes.c_int64 * 3
    cu = info.cu_seqlens.data_ptr()
    scale = float(D) ** -0.5 if scale is None else float(scale)
    qt = fused_query_tile(max_seq_len, max_seq_len, D, causal, q, query_tile)
    with _lib.device_guard(q):
        _lib.check(_lib.fn.en_attn_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                         info.lens.data_ptr(), None, batch_size, H, int(max_seq_len),
                                         int(max_seq_len), D, arr(*qs), arr(*ks), arr(*vs), arr(0, D, H * D), cu, cu,
                                         scale, int(bool(causal)), _lib.dtype_tag(q, "attn_fused_varlen"),
                                         None if qt == 64 else
                                         info.tile_table_ptr(H, int(max_seq_len), _unit_kv_bytes(max_seq_len, D, q), qt),
                                         qt, _lib.stream_of(q)), "attn_fused_varlen")
    return out


def packed_scores_elems(batch_size: int, head_num: int, seq_len: int, dtype) -> int:
    """Elements of the packed causal score tensor of a self-attention batch: per (batch, head) unit the visible
    prefix of every row, rounded up to a whole 128-byte group (``V`` = 64 fp16 / bf16 or 32 fp32 entries), back to
    back: row ``q`` starts ``V * (V*t*(t+1)/2 + (q - V*t) * (t+1))`` elements into its unit, ``t = q // V``, and holds
    ``V * (t+1)`` elements; each unit owns the slot of a full-length one.  QK^T writes and the softmax zeroes a row
    only up to the end of the 16-byte vector that holds its last visible entry."""
    n = _lib.fn.en_packed_scores_elems(int(batch_size), int(head_num), int(seq_len), _lib._DTYPE_TAG[dtype])
    if n <= 0:
        raise RuntimeError("packed_scores_elems: bad arguments")
    return n


def attn_qk_varlen(q, k, batch_size: int, max_seq_len: int, seq_len_list, *, alpha: float = 1.0, causal: bool = True,
                   packed_scores: bool = False, out: Optional[torch.Tensor] = None):
    """QK^T of a self-attention batch straight on packed tokens: ``q`` and ``k`` are ``[T,H,D]`` views of the
    projection output (batch ``b`` at rows ``cu_seqlens[b]`` ..), so no ``transpose_pad`` is needed first.
    Returns ``[B,H,S,S]`` scores as ``attn_qk`` does, or with ``packed_scores`` (causal, fp16 / bf16) the flat packed
    tensor of :func:`packed_scores_elems` elements that ``scale_mask_softmax_packed`` and ``attn_pv_varlen`` read."""
    qs, ks = _thd(q, "q"), _thd(k, "k")
    T, H, D = q.shape
    if k.shape != q.shape or k.dtype != q.dtype:
        raise RuntimeError("attn_qk_varlen: q and k disagree in shape or dtype")
    B, S = int(batch_size), int(max_seq_len)
    info = seq_info(seq_len_list, B, q.device)
    shape = (packed_scores_elems(B, H, S, q.dtype),) if packed_scores else (B, H, S, S)
    if out is None:
        out = torch.empty(shape, dtype=q.dtype, device=q.device)
    elif out.numel() < (shape[0] if packed_scores else B * H * S * S) or out.dtype != q.dtype or not out.is_contiguous():
        raise RuntimeError("attn_qk_varlen: out is too small, strided or of another dtype")
    cu = info.cu_seqlens.data_ptr()
    with _lib.device_guard(q):
        _lib.check(_lib.fn.en_attn_qk(q.data_ptr(), k.data_ptr(), out.data_ptr(), info.lens.data_ptr(), None, B, H, S, S, D,
                                      *qs, *ks, float(alpha), int(bool(causal)), _lib.dtype_tag(q, "attn_qk_varlen"), cu, cu,
                                      int(bool(packed_scores)), info.tile_table_ptr(H, S, _unit_kv_bytes(S, D, q)),
                                      _lib.stream_of(q)), "attn_qk_varlen")
    return out


def scale_mask_softmax_packed(batch_size: int, seq_len: int, head_num: int, scores, seq_len_list, *, scale: float = 1.0):
    """``scale_mask_softmax`` (causal) in place on the packed scores of :func:`attn_qk_varlen`; returns its input."""
    _lib.require_gpu(scores, "scores")
    B, S, H = int(batch_size), int(seq_len), int(head_num)
    if scores.numel() < packed_scores_elems(B, H, S, scores.dtype):
        raise RuntimeError("scale_mask_softmax_packed: scores is smaller than the packed tensor of this batch")
    info = seq_info(seq_len_list, B, scores.device)
    with _lib.device_guard(scores):
        _lib.check(_lib.fn.en_scale_mask_softmax_packed(scores.data_ptr(), info.lens.data_ptr(), B, H, S, float(scale),
                                                        _lib.dtype_tag(scores, "scale_mask_softmax_packed"),
                                                        _lib.stream_of(scores)), "scale_mask_softmax_packed")
    return scores


def attn_pv_varlen(p, v, batch_size: int, max_seq_len: int, seq_len_list, *, causal: bool = True,
                   packed_scores: bool = False, out: Optional[torch.Tensor] = None):
    """PV of a self-attention batch with ``v`` a ``[T,H,D]`` view of the packed projection output and the context
    written as packed ``[1,T,H,D]`` rows (what ``transpose_depad`` would return).  ``p`` is ``[B,H,S,S]`` as left by
    ``scale_mask_softmax`` or, with ``packed_scores``, the flat tensor left by ``scale_mask_softmax_packed``."""
    _lib.require_gpu(p, "p")
    vs = _thd(v, "v")
    T, H, D = v.shape
    B, S = int(batch_size), int(max_seq_len)
    if p.dtype != v.dtype or p.numel() < (packed_scores_elems(B, H, S, v.dtype) if packed_scores else B * H * S * S):
        raise RuntimeError("attn_pv_varlen: p is too small for this batch or of another dtype than v")
    info = seq_info(seq_len_list, B, v.device)
    if out is None:
        out = torch.empty((1, T, H, D), dtype=v.dtype, device=v.device)
    elif out.numel() != T * H * D or out.dtype != v.dtype or not out.is_contiguous():
        raise RuntimeError("attn_pv_varlen: out must be contiguous [1,T,H,D] of v's dtype")
    cu = info.cu_seqlens.data_ptr()
    with _lib.device_guard(v):
        _lib.check(_lib.fn.en_attn_pv(p.data_ptr(), v.data_ptr(), out.data_ptr(), info.lens.data_ptr(), None, B, H, S, S, D,
                                      *vs, 0, D, H * D, int(bool(causal)), 0, _lib.dtype_tag(v, "attn_pv_varlen"), cu, cu,
                                      int(bool(packed_scores)), info.tile_table_ptr(H, S, _unit_kv_bytes(S, D, v)),
                                      _lib.stream_of(v)), "attn_pv_varlen")
    return out


def attn_fused_packed(qkv, batch_size: int, max_seq_len: int, seq_len_list, head_num: int, size_per_head: int, *,
                      scale: Optional[float] = None, causal: bool = True, out: Optional[torch.Tensor] = None,
                      query_tile: Optional[int] = None):
    """Self-attention straight on the packed projection output: ``qkv`` is ``[1,T,H,3D]`` (or ``[T,H,3D]``,
    the layout ``transpose_pad`` is fed with in examples/bert/bert.py:100-104), the result is the packed
    context ``[1,T,H,D]`` that ``transpose_depad`` would return (bert.py:123).  fp16 / bf16 only.
    """
    _lib.require_gpu(qkv, "qkv")
    H, D = int(head_num), int(size_per_head)
    if qkv.numel() % (3 * H * D) != 0:
        raise RuntimeError("attn_fused_packed: qkv must be [1,T,H,3D]")
    q, k, v = torch.chunk(qkv.view(-1, H, 3 * D), 3, dim=-1)
    return attn_fused_varlen(q, k, v, batch_size, max_seq_len, seq_len_list, scale=scale, causal=causal, out=out,
                             query_tile=query_tile)


def kv_cache_fill(src, cache, batch_size: int, seq_len_list, head_first: int = 0, zero_padding: bool = True):
    """Writes ``cache[b,h,s,:] = src[cu[b]+s, head_first+h, :]`` for ``s < len[b]`` and zeros for the rest of
    the ``[B,H,Smax,D]`` cache.  ``src`` is the packed projection output seen as ``[T,Hs,D]`` (contiguous),
    so K and V caches are filled from their thirds of a fused projection without copying them out first.
    ``zero_padding=False`` leaves the rows past each length as they are (the attention and decode kernels
    never read them), which saves writing them.
    """
    _lib.require_gpu(src, "src")
    _lib.require_gpu(cache, "cache")
    if src.dim() != 3 or cache.dim() != 4 or cache.shape[0] != batch_size or cache.shape[3] != src.shape[2] \
            or cache.dtype != src.dtype:
        raise RuntimeError("kv_cache_fill: src must be [T,Hs,D] and cache [B,H,Smax,D] of one dtype")
    B, H, Smax, D = cache.shape
    info = seq_info(seq_len_list, batch_size, src.device)
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_transpose_pad_heads(src.data_ptr(), cache.data_ptr(), info.cu_seqlens.data_ptr(), B, Smax,
                                                  H, D, src.shape[1], int(head_first), int(bool(zero_padding)),
                                                  src.element_size(), _lib.stream_of(src)), "kv_cache_fill")
    return cache


def kv_cache_append(k_new, v_new, k_cache, v_cache, kv_len_list, overflow: Optional[torch.Tensor] = None):
    """Writes the new token's rows ``k_new`` / ``v_new`` (``[B,H,D]`` views) into the ``[B,H,Smax,D]`` caches at
    position ``kv_len[b]``.  The caller advances the lengths afterwards.  A sequence whose cache is full keeps
    its rows and loses the new one; ``overflow`` (one int32 on the device) is incremented once per such
    sequence, so that a caller without a host-side bound of the lengths can still notice."""
    for t, n in ((k_new, "k_new"), (v_new, "v_new")):
        _lib.require_gpu(t, n, contiguous=False)
        if t.dim() != 3 or t.stride(2) != 1:
            raise RuntimeError(f"kv_cache_append: {n} must be a [B,H,D] view with contiguous channels")
    cs = _bhsd(k_cache, "k_cache")
    if _bhsd(v_cache, "v_cache") != cs or k_new.stride() != v_new.stride() or k_cache.shape != v_cache.shape:
        raise RuntimeError("kv_cache_append: K and V must share shapes and strides")
    B, H, Smax, D = k_cache.shape
    if k_new.shape != (B, H, D) or v_new.shape != (B, H, D) or k_new.dtype != k_cache.dtype:
        raise RuntimeError("kv_cache_append: new rows must be [B,H,D] of the cache dtype")
    info = seq_info(kv_len_list, B, k_cache.device)
    if overflow is not None:
        _lib.require_gpu(overflow, "overflow")
        if overflow.dtype != torch.int32 or overflow.numel() < 1:
            raise RuntimeError("kv_cache_append: overflow must be an int32 tensor of at least one element")
    with _lib.device_guard(k_cache):
        _lib.check(_lib.fn.en_kv_append(k_new.data_ptr(), v_new.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                        info.lens.data_ptr(), B, H, Smax, D, k_new.stride(0), k_new.stride(1), *cs,
                                        k_cache.element_size(), _lib.ptr(overflow), _lib.stream_of(k_cache)),
                   "kv_cache_append")


def _pool(t, name: str):
    """Strides (page, head, row) in elements of a ``[pages, H, page_size, D]`` pool with contiguous channels."""
    _lib.require_gpu(t, name, contiguous=False)
    if t.dim() != 4 or t.stride(3) != 1:
        raise RuntimeError(f"{name} must be a [pages, H, page_size, D] tensor with contiguous channels")
    return (t.stride(0), t.stride(1), t.stride(2))


def _page_table(page_table, batch: int, name: str):
    _lib.require_gpu(page_table, "page_table")
    if page_table.dim() != 2 or page_table.shape[0] != batch or page_table.dtype != torch.int32:
        raise RuntimeError(f"{name}: page_table must be a contiguous int32 [batch, max_pages_per_seq] tensor")
    return int(page_table.shape[1])


def _overflow(overflow, name: str):
    if overflow is not None:
        _lib.require_gpu(overflow, "overflow")
        if overflow.dtype != torch.int32 or overflow.numel() < 1:
            raise RuntimeError(f"{name}: overflow must be an int32 tensor of at least one element")


def kv_pages_fill(src, pool, batch_size: int, max_seq_len: int, seq_len_list, page_table, head_first: int = 0,
                  overflow: Optional[torch.Tensor] = None):
    """Prefill of a paged cache: ``pool[page_table[b, s // P], h, s % P, :] = src[cu[b]+s, head_first+h, :]`` for
    ``s < len[b]``; ``src`` is the packed projection output seen as ``[T,Hs,D]`` (as ``kv_cache_fill``), ``pool`` is
    ``[pages, H, P, D]``.  A row whose page id lies outside the pool is not written and counted in ``overflow``."""
    _lib.require_gpu(src, "src")
    ps = _pool(pool, "pool")
    if src.dim() != 3 or pool.shape[3] != src.shape[2] or pool.dtype != src.dtype:
        raise RuntimeError("kv_pages_fill: src must be [T,Hs,D] and pool [pages,H,P,D] of one dtype")
    N, H, P, D = pool.shape
    max_pages = _page_table(page_table, batch_size, "kv_pages_fill")
    _overflow(overflow, "kv_pages_fill")
    info = seq_info(seq_len_list, batch_size, src.device)
    arr = ctypes.c_int64 * 3
    with _lib.device_guard(src):
        _lib.check(_lib.fn.en_kv_fill_paged(src.data_ptr(), pool.data_ptr(), info.cu_seqlens.data_ptr(),
                                            page_table.data_ptr(), int(batch_size), int(max_seq_len), H, D, src.shape[1],
                                            int(head_first), max_pages, P, N, arr(*ps), src.element_size(),
                                            _lib.ptr(overflow), _lib.stream_of(src)), "kv_pages_fill")
    return pool


def kv_pages_append(k_new, v_new, k_pool, v_pool, kv_len_list, page_table, overflow: Optional[torch.Tensor] = None):
    """``kv_cache_append`` for paged caches: the new ``[B,H,D]`` rows go to row ``kv_len[b] % P`` of page
    ``page_table[b, kv_len[b] // P]``.  A sequence whose next position has no page in the pool keeps its rows, loses
    the new one and is counted in ``overflow``."""
    for t, n in ((k_new, "k_new"), (v_new, "v_new")):
        _lib.require_gpu(t, n, contiguous=False)
        if t.dim() != 3 or t.stride(2) != 1:
            raise RuntimeError(f"kv_pages_append: {n} must be a [B,H,D] view with contiguous channels")
    ps = _pool(k_pool, "k_pool")
    if _pool(v_pool, "v_pool") != ps or k_new.stride() != v_new.stride() or k_pool.shape != v_pool.shape:
        raise RuntimeError("kv_pages_append: K and V must share shapes and strides")
    N, H, P, D = k_pool.shape
    B = k_new.shape[0]
    if k_new.shape != (B, H, D) or v_new.shape != (B, H, D) or k_new.dtype != k_pool.dtype:
        raise RuntimeError("kv_pages_append: new rows must be [B,H,D] of the pool dtype")
    max_pages = _page_table(page_table, B, "kv_pages_append")
    _overflow(overflow, "kv_pages_append")
    info = seq_info(kv_len_list, B, k_pool.device)
    arr = ctypes.c_int64 * 3
    with _lib.device_guard(k_pool):
        _lib.check(_lib.fn.en_kv_append_paged(k_new.data_ptr(), v_new.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(),
                                              info.lens.data_ptr(), page_table.data_ptr(), B, H, max_pages, P, N, D,
                                              k_new.stride(0), k_new.stride(1), arr(*ps), k_pool.element_size(),
                                              _lib.ptr(overflow), _lib.stream_of(k_pool)), "kv_pages_append")


def decode_attn_paged(q, k_pool, v_pool, kv_len_list, page_table, *, scale: Optional[float] = None,
                      out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None, split: bool = True):
    """``decode_attn`` over paged caches: position ``j`` of sequence ``b`` is row ``j % P`` of page
    ``page_table[b, j // P]`` of the ``[pages, H, P, D]`` pools (``P`` a power of two, at least 16).  ``[B,H,1,D]``.
    A page id outside the pool reads as zeros."""
    _lib.require_gpu(q, "q", contiguous=False)
    ks = _pool(k_pool, "k_pool")
    vs = _pool(v_pool, "v_pool")
    N, H, P, D = k_pool.shape
    if v_pool.shape != k_pool.shape or v_pool.dtype != k_pool.dtype:
        raise RuntimeError("decode_attn_paged: k_pool and v_pool must share shape and dtype")
    if q.dim() < 2 or q.numel() % (H * D) != 0 or q.dtype != k_pool.dtype:
        raise RuntimeError("decode_attn_paged: q must be [B,H,1,D] of the pools' dtype")
    B = q.numel() // (H * D)
    max_pages = _page_table(page_table, B, "decode_attn_paged")
    q_ = q.reshape(B, H, D).contiguous()
    info = seq_info(kv_len_list, B, q.device)
    if out is None:
        out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    else:
        _lib.require_gpu(out, "out")
        if out.numel() != B * H * D or out.dtype != q.dtype:
            raise RuntimeError("decode_attn_paged: out must be a contiguous [B,H,1,D] tensor of q's dtype")
    arr = ctypes.c_int64 * 3
    scale = float(D) ** -0.5 if scale is None else float(scale)
    need = decode_attn_workspace_bytes(B, H, max_pages * P, D) if split else 0
    if need and workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    ws_bytes = 0
    if workspace is not None and need:
        _lib.require_gpu(workspace, "workspace")
        ws_bytes = workspace.numel() * workspace.element_size()
    with _lib.device_guard(q):
        _lib.check(_lib.fn.en_decode_attn_paged(q_.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), out.data_ptr(),
                                                info.lens.data_ptr(), page_table.data_ptr(), B, H, max_pages, P, N, D,
                                                arr(*ks), arr(*vs), scale, _lib.dtype_tag(q, "decode_attn_paged"),
                                                _lib.ptr(workspace) if ws_bytes else None, ws_bytes,
                                                _lib.stream_of(q)), "decode_attn_paged")
    return out


def decode_qk(q, k_cache, kv_len_list, *, alpha: float = 1.0, out: Optional[torch.Tensor] = None):
    """scores[b,h,0,j] = alpha * <q[b,h,0,:], k_cache[b,h,j,:]> for j < kv_len[b]; ``[B,H,1,Smax]``."""
    _lib.require_gpu(q, "q", contiguous=False)
    ks = _bhsd(k_cache, "k_cache")
    B, H, Smax, D = k_cache.shape
    q_ = q.reshape(B, H, D).contiguous()
    if q_.dtype != k_cache.dtype:
        raise RuntimeError("decode_qk: q and k_cache must share one dtype")
    info = seq_info(kv_len_list, B, q.device)
    if out is None:
        out = torch.empty((B, H, 1, Smax), dtype=q.dtype, device=q.device)
    with _lib.device_guard(q):
        _lib.check(_lib.fn.en_decode_qk(q_.data_ptr(), k_cache.data_ptr(), out.data_ptr(), info.lens.data_ptr(),
                                            B, H, Smax, D, *ks, float(alpha), _lib.dtype_tag(q, "decode_qk"),
                                            _lib.stream_of(q)), "decode_qk")
    return out


def decode_pv(p, v_cache, kv_len_list, *, out: Optional[torch.Tensor] = None):
    """ctx[b,h,0,:] = sum_{j<kv_len[b]} p[b,h,0,j] v_cache[b,h,j,:]; ``[B,H,1,D]``."""
    _lib.require_gpu(p, "p")
    vs = _bhsd(v_cache, "v_cache")
    B, H, Smax, D = v_cache.shape
    if p.numel() != B * H * Smax or p.dtype != v_cache.dtype:
        raise RuntimeError("decode_pv: p must be [B,H,1,Smax] of v_cache's dtype")
    info = seq_info(kv_len_list, B, p.device)
    if out is None:
        out = torch.empty((B, H, 1, D), dtype=p.dtype, device=p.device)
    with _lib.device_guard(p):
        _lib.check(_lib.fn.en_decode_pv(p.data_ptr(), v_cache.data_ptr(), out.data_ptr(), info.lens.data_ptr(),
                                            B, H, Smax, D, *vs, _lib.dtype_tag(p, "decode_pv"), _lib.stream_of(p)),
                   "decode_pv")
    return out


def decode_attn(q, k_cache, v_cache, kv_len_list, *, scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                workspace: Optional[torch.Tensor] = None, split: bool = True):
    """ctx[b,h,0,:] = sum_j softmax_j(scale * <q[b,h,0,:], k_cache[b,h,j,:]>) v_cache[b,h,j,:] over the cached
    positions ``j < kv_len[b]``, in one pass over the caches: what ``decode_qk`` -> ``scale_mask_softmax`` ->
    ``decode_pv`` compute in three launches (and the reference by recomputing the whole square,
    energonai/model/attention.py:61-71,106-118).  ``[B,H,1,D]``; ``scale`` defaults to ``size_per_head ** -0.5``.
    A batch with fewer than 512 (batch, head) units shares each unit's keys between several workgroups and combines
    their partial results in a second small kernel; the fp32 buffer they pass through is ``workspace`` (any
    tensor of at least ``decode_attn_workspace_bytes`` bytes) or a temporary; ``split=False`` keeps one workgroup
    per unit."""
    _lib.require_gpu(q, "q", contiguous=False)
    ks = _bhsd(k_cache, "k_cache")
    vs = _bhsd(v_cache, "v_cache")
    B, H, Smax, D = k_cache.shape
    if v_cache.shape != k_cache.shape or v_cache.dtype != k_cache.dtype:
        raise RuntimeError("decode_attn: k_cache and v_cache must share shape and dtype")
    if q.numel() != B * H * D or q.dtype != k_cache.dtype:
        raise RuntimeError("decode_attn: q must be [B,H,1,D] of the caches' dtype")
    q_ = q.reshape(B, H, D).contiguous()
    info = seq_info(kv_len_list, B, q.device)
    if out is None:
        out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    else:
        _lib.require_gpu(out, "out")
        if out.numel() != B * H * D or out.dtype != q.dtype:
            raise RuntimeError("decode_attn: out must be a contiguous [B,H,1,D] tensor of q's dtype")
    arr = ctypes.c_int64 * 3
    scale = float(D) ** -0.5 if scale is None else float(scale)
    need = decode_attn_workspace_bytes(B, H, Smax, D) if split else 0
    if need and workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    ws_bytes = 0
    if workspace is not None and need:
        _lib.require_gpu(workspace, "workspace")
        ws_bytes = workspace.numel() * workspace.element_size()
    with _lib.device_guard(q):
        _lib.check(_lib.fn.en_decode_attn(q_.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
                                          info.lens.data_ptr(), B, H, Smax, D, arr(*ks), arr(*vs), scale,
                                          _lib.dtype_tag(q, "decode_attn"), _lib.ptr(workspace) if ws_bytes else None,
                                          ws_bytes, _lib.stream_of(q)), "decode_attn")
    return out


def decode_attn_workspace_bytes(batch_size: int, head_num: int, max_seq_len: int, size_per_head: int) -> int:
    """Bytes of the buffer through which ``decode_attn`` passes partial results when it shares a unit's keys between
    workgroups (0: this shape gets one workgroup per unit)."""
    return int(_lib.fn.en_decode_attn_workspace_bytes(int(batch_size), int(head_num), int(max_seq_len), int(size_per_head)))
