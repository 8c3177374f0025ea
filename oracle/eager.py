"""Torch-eager CPU restatement of the padding-removal hot path (test oracle).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the
CPU-baseline leg of the benchmark; never by the product.

Every function follows a reference file (path:line relative to the
reference checkout) and is written from its behaviour, not from its text.
All arithmetic that the reference does in fp32 is done here in fp32 (or in
float64 where a test asks for a tighter pin via ``acc_dtype``).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

NEG_INF = float("-inf")


def _as_len_list(seq_lens) -> list:
    if isinstance(seq_lens, torch.Tensor):
        return [int(v) for v in seq_lens.detach().cpu().tolist()]
    return [int(v) for v in seq_lens]


# ---------------------------------------------------------------------------
# offsets
# ---------------------------------------------------------------------------

def prefix_offsets(seq_lens, batch_size: int) -> torch.Tensor:
    """cu[b] = sum of lens before b, cu[B] = total.

    Restates the serial per-block loop of
    energonai/kernel/cuda_native/csrc/transpose_pad_fusion_kernel.cu:24-27,70-73.
    """
    lens = _as_len_list(seq_lens)[:batch_size]
    cu = [0]
    for v in lens:
        cu.append(cu[-1] + v)
    return torch.tensor(cu, dtype=torch.int32)


def ft_build_padding_offsets(seq_lens, batch_size: int, max_seq_len: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (valid_word_num[1], tmp_mask_offset[T]).

    transpose_pad_fusion_kernel.cu:112-131: for every valid token t of
    sequence b, offset = sum over earlier sequences of (max_seq_len - len).
    Closed form: repeat_interleave(exclusive_cumsum(S - len), len).
    """
    lens = torch.tensor(_as_len_list(seq_lens)[:batch_size], dtype=torch.int64)
    pad = max_seq_len - lens
    excl = torch.cumsum(pad, 0) - pad
    off = torch.repeat_interleave(excl, lens).to(torch.int32)
    valid = torch.tensor([int(lens.sum())], dtype=torch.int32)
    return valid, off


# ---------------------------------------------------------------------------
# pack / unpack (bit-exact data movement)
# ---------------------------------------------------------------------------

def depad(src: torch.Tensor, batch_size: int, seq_lens, left_padded: bool = False) -> torch.Tensor:
    """[B,S,hid] -> [1,T,hid] keeping only valid rows.

    energonai/kernel/cuda_native/transpose_pad.py:30-37 (right padded:
    rows 0:len of every sequence, concatenated).  ``left_padded`` keeps rows
    S-len:S instead (OPT batches are left padded, examples/opt/batch.py:12-24).
    """
    lens = _as_len_list(seq_lens)
    S = src.shape[1]
    parts = []
    for i in range(batch_size):
        n = lens[i]
        parts.append(src[i:i + 1, S - n:S, :] if left_padded else src[i:i + 1, 0:n, :])
    return torch.cat(parts, dim=1)


def repad(src: torch.Tensor, batch_size: int, max_seq_len: int, seq_lens, left_padded: bool = False) -> torch.Tensor:
    """[1,T,hid] -> [B,S,hid]: the inverse of :func:`depad`, padding rows zero.

    For right-padded batches this is what ft_rebuild_padding produces from the
    packed rows (csrc/transpose_pad_fusion_kernel.cu:176-199, caller
    examples/gpt/gpt.py:321-323); ``left_padded`` puts sequence b at rows S-len:S.
    """
    lens = _as_len_list(seq_lens)
    hid = src.shape[-1]
    rows = src.reshape(-1, hid)
    out = torch.zeros((batch_size, max_seq_len, hid), dtype=src.dtype)
    start = 0
    for i in range(batch_size):
        n = lens[i]
        if left_padded:
            out[i, max_seq_len - n:max_seq_len] = rows[start:start + n]
        else:
            out[i, 0:n] = rows[start:start + n]
        start += n
    return out


def transpose_pad(src: torch.Tensor, batch_size: int, max_seq_len: int, seq_lens,
                  head_num: int, size_per_head: int) -> torch.Tensor:
    """[1,T,H,Dk] -> zero-padded [B,H,S,Dk].

    transpose_pad_fusion_kernel.cu:58-84 and the wrapper's output shape
    (transpose_pad_fusion_wrapper.cpp:39-44).  Written the way the reference's
    own test states it (tests/test_kernel/test_transpose_pad_fusion_kernel.py:63-74):
    scatter the packed rows into a zero [B,S,H,Dk] tensor, then permute(0,2,1,3).
    """
    lens = _as_len_list(seq_lens)
    x = src.reshape(-1, head_num, size_per_head)
    padded = torch.zeros(batch_size, max_seq_len, head_num, size_per_head, dtype=src.dtype)
    t = 0
    for b in range(batch_size):
        n = lens[b]
        padded[b, :n] = x[t:t + n]
        t += n
    return padded.permute(0, 2, 1, 3).contiguous()


def transpose_depad(src: torch.Tensor, batch_size: int, sum_seq: int, max_seq_len: int, seq_lens,
                    head_num: int, size_per_head: int) -> torch.Tensor:
    """[B,H,S,D] -> [1,T,H,D] (valid rows only).

    transpose_pad_fusion_kernel.cu:8-35; wrapper output shape
    transpose_pad_fusion_wrapper.cpp:66-70.  Stated as the reference test does
    (test_transpose_pad_fusion_kernel.py:32-42,76-78): permute back, slice-copy
    the valid rows.
    """
    lens = _as_len_list(seq_lens)
    x = src.reshape(batch_size, head_num, max_seq_len, size_per_head).permute(0, 2, 1, 3)
    parts = [x[b, :lens[b]] for b in range(batch_size)]
    out = torch.cat(parts, dim=0).contiguous()
    assert out.shape[0] == int(sum_seq), (out.shape, int(sum_seq))
    return out.reshape(1, int(sum_seq), head_num, size_per_head)


def ft_remove_padding(src: torch.Tensor, tmp_mask_offset: torch.Tensor, valid_word_num: int,
                      hidden_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (tgt[1,valid,hid], mask_offset[valid]).

    transpose_pad_fusion_kernel.cu:142-156: tgt[t] = src[t + off[t]] over the
    flattened [B*S, hid] source; mask_offset is written as a copy of the
    temporary offsets.
    """
    v = int(valid_word_num)
    off = tmp_mask_offset.reshape(-1)[:v].to(torch.int64)
    rows = torch.arange(v, dtype=torch.int64) + off
    flat = src.reshape(-1, hidden_dim)
    return flat[rows].reshape(1, v, hidden_dim).contiguous(), off.to(torch.int32)


def ft_rebuild_padding(src: torch.Tensor, mask_offset: torch.Tensor, valid_word_num: int, hidden_dim: int,
                       batch_size: int, max_seq_len: int) -> torch.Tensor:
    """[1,valid,hid] -> zeros[B,S,hid] with valid rows filled.

    transpose_pad_fusion_kernel.cu:178-189 (scatter to row t + off[t]) into
    the wrapper's zero tensor (transpose_pad_fusion_wrapper.cpp:158).
    """
    v = int(valid_word_num)
    off = mask_offset.reshape(-1)[:v].to(torch.int64)
    rows = torch.arange(v, dtype=torch.int64) + off
    out = torch.zeros(batch_size * max_seq_len, hidden_dim, dtype=src.dtype)
    out[rows] = src.reshape(v, hidden_dim)
    return out.reshape(batch_size, max_seq_len, hidden_dim)


def ft_transpose_rebuild_padding(Q, K, V, q_buf, k_buf, v_buf, batch_size: int, seq_len: int, head_num: int,
                                 size_per_head: int, valid_word_num: int, mask_offset) -> None:
    """Q,K,V [valid,H,D] scattered into caller-owned [B,H,S,D] buffers in place.

    transpose_pad_fusion_kernel.cu:213-236: token t goes to
    (b, s) = divmod(t + off[t], S); the padding of the buffers is not touched.
    """
    v = int(valid_word_num)
    off = mask_offset.reshape(-1)[:v].to(torch.int64)
    pos = torch.arange(v, dtype=torch.int64) + off
    b = pos // seq_len
    s = pos % seq_len
    for src, dst in ((Q, q_buf), (K, k_buf), (V, v_buf)):
        x = src.reshape(v, head_num, size_per_head)
        d = dst.view(batch_size, head_num, seq_len, size_per_head)
        d[b, :, s, :] = x


def ft_transpose_remove_padding(src, valid_word_num: int, batch_size: int, seq_len: int, head_num: int,
                                size_per_head: int, mask_offset) -> torch.Tensor:
    """[B,H,S,D] -> [1,valid,H*D].

    transpose_pad_fusion_kernel.cu:268-289; output shape
    transpose_pad_fusion_wrapper.cpp:227-228.
    """
    v = int(valid_word_num)
    off = mask_offset.reshape(-1)[:v].to(torch.int64)
    pos = torch.arange(v, dtype=torch.int64) + off
    b = pos // seq_len
    s = pos % seq_len
    x = src.reshape(batch_size, head_num, seq_len, size_per_head)
    return x[b, :, s, :].reshape(1, v, head_num * size_per_head).contiguous()


# ---------------------------------------------------------------------------
# scale + mask + softmax
# ---------------------------------------------------------------------------

def visible_keys(q: int, q_len: int, k_len: int, causal: bool) -> int:
    """Number of leading keys query row q may see.

    Square case (q_len == k_len) reduces to the reference rule ``k <= q``
    (scale_mask_softmax_kernel.cu:19-22).  With fewer queries than keys the
    queries are the last q_len positions of the sequence (the reference's
    cached decode recomputes the full square and keeps the last rows,
    energonai/model/attention.py:61-71,106-118), so row q sees
    k <= q + (k_len - q_len).
    """
    if not causal:
        return k_len
    return max(0, min(k_len, q + (k_len - q_len) + 1))


def scale_mask_softmax(batch_size: int, batch_seq_len: int, head_num: int, src: torch.Tensor, seq_lens,
                       scale: float = 1.0, causal: bool = True, k_seq_len: Optional[int] = None,
                       q_lens=None, acc_dtype: torch.dtype = torch.float32,
                       out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Row softmax of [B,H,Sq,Sk] scores; returns a new tensor.

    Reference semantics (scale_mask_softmax_kernel.cu:11-42, defaults here):
    for each valid query row q < len[b] the row becomes
    softmax(src[..., :q+1]) followed by zeros; rows with q >= len[b] are left
    exactly as they were.  No scale is applied by the reference (scale=1.0).
    Extensions used by the configs: ``scale`` multiplies the scores first
    (examples/bert/bert.py:114), ``causal=False`` masks keys >= len[b] only
    (key-padding mask, energonai/model/model_factory.py:117-121 with a hard
    mask instead of -1e4), rectangular [Sq,Sk] with ``q_lens`` (see
    visible_keys).  Math in ``acc_dtype``; result cast to ``out_dtype``
    (default: src.dtype).
    """
    Sq = batch_seq_len
    Sk = Sq if k_seq_len is None else k_seq_len
    k_lens = _as_len_list(seq_lens)
    ql = [min(n, Sq) for n in k_lens] if q_lens is None else _as_len_list(q_lens)
    out_dtype = out_dtype or src.dtype
    x = src.reshape(batch_size, head_num, Sq, Sk)
    out = x.clone().to(out_dtype)
    for b in range(batch_size):
        for q in range(min(ql[b], Sq)):
            n = visible_keys(q, ql[b], k_lens[b], causal)
            row = torch.zeros(head_num, Sk, dtype=acc_dtype)
            if n > 0:
                row[:, :n] = torch.softmax(x[b, :, q, :n].to(acc_dtype) * scale, dim=-1)
            out[b, :, q, :] = row.to(out_dtype)
    return out.reshape(src.shape)


def scale_mask_softmax_additive(src: torch.Tensor, seq_lens, scale: float, causal: bool) -> torch.Tensor:
    """The eager form the reference models use: additive -1e4 masks, fp32 softmax.

    energonai/model/attention.py:105-116 and examples/gpt/gpt.py:114-123:
    x*scale -> where(causal, x, -1e4) -> + (1-mask)*-1e4 -> softmax(fp32).
    Square [B,H,S,S] only; used to bound the difference to the hard mask.
    """
    B, H, S, _ = src.shape
    lens = torch.tensor(_as_len_list(seq_lens))
    x = src.float() * scale
    if causal:
        tri = torch.tril(torch.ones(S, S, dtype=torch.bool)).view(1, 1, S, S)
        x = torch.where(tri, x, torch.tensor(-1e4))
    keymask = (torch.arange(S).view(1, S) < lens.view(B, 1)).float()
    x = x + (1.0 - keymask).view(B, 1, 1, S) * -10000.0
    return torch.softmax(x, -1, dtype=torch.float)


# ---------------------------------------------------------------------------
# LayerNorm forward (+ fused residual)
# ---------------------------------------------------------------------------

def layer_norm(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor, eps: float = 1e-5,
               residual: Optional[torch.Tensor] = None, acc_dtype: torch.dtype = torch.float32,
               out_dtype: Optional[torch.dtype] = None):
    """Returns (y, mean[n1], invvar[n1], pre_norm_sum).

    energonai/kernel/cuda_native/csrc/layer_norm_cuda_kernel.cu:243-279:
    biased variance over the last dim, invvar = rsqrt(var + eps),
    y = gamma * (x - mean) * invvar + beta, statistics in fp32; output dtype =
    gamma's dtype (layer_norm_cuda.cpp:93-94).  All math here in ``acc_dtype``
    with one rounding at the end (the reference rounds the normalised value
    to the output type before the affine step, kernel.cu:266; the parity
    target is the unrounded fp32 value).  ``residual`` is added to x first,
    in acc_dtype (examples/bert/bert.py:132).
    """
    n2 = gamma.numel()
    xs = x.reshape(-1, n2).to(acc_dtype)
    if residual is not None:
        xs = xs + residual.reshape(-1, n2).to(acc_dtype)
    mean = xs.mean(dim=-1)
    var = xs.var(dim=-1, unbiased=False)
    invvar = torch.rsqrt(var + eps)
    y = (xs - mean[:, None]) * invvar[:, None] * gamma.reshape(1, n2).to(acc_dtype) + beta.reshape(1, n2).to(acc_dtype)
    out_dtype = out_dtype or gamma.dtype
    return (y.to(out_dtype).reshape(x.shape), mean.to(torch.float32), invvar.to(torch.float32),
            xs.reshape(x.shape))


# ---------------------------------------------------------------------------
# attention contractions on the padded [B,H,S,*] layout
# ---------------------------------------------------------------------------

def attn_qk(q: torch.Tensor, k: torch.Tensor, acc_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """scores[b,h,i,j] = sum_d q[b,h,i,d] k[b,h,j,d]  (examples/bert/bert.py:110)."""
    return torch.matmul(q.to(acc_dtype), k.to(acc_dtype).transpose(-1, -2))


def attn_pv(p: torch.Tensor, v: torch.Tensor, acc_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """ctx[b,h,i,:] = sum_j p[b,h,i,j] v[b,h,j,:]  (examples/bert/bert.py:119)."""
    return torch.matmul(p.to(acc_dtype), v.to(acc_dtype))


# ---------------------------------------------------------------------------
# one transformer layer's hot path
# ---------------------------------------------------------------------------

def layer_unpadded(hidden_padded: torch.Tensor, qkv_packed: torch.Tensor, seq_lens, head_num: int,
                   size_per_head: int, gamma: torch.Tensor, beta: torch.Tensor, eps: float, scale: float,
                   causal: bool, left_padded: bool = False, dense_out: Optional[torch.Tensor] = None,
                   acc_dtype: torch.dtype = torch.float32, storage_dtype: Optional[torch.dtype] = None):
    """depad -> transpose_pad -> QK^T -> softmax -> PV -> transpose_depad -> residual + LN.

    Follows examples/bert/bert.py:54-62,91-134 with the projections left out:
    ``qkv_packed`` [1,T,H,3D] stands for the output of query_key_value,
    the attention output feeds the residual directly when H*D equals the
    LayerNorm width, otherwise ``dense_out`` [1,T,hid] stands for the output of
    the row-parallel dense.  ``storage_dtype`` rounds each intermediate to the
    dtype the kernels store (fp16 configs); None keeps everything in
    acc_dtype.  Returns a dict of every intermediate.
    """
    B, S, hid = hidden_padded.shape
    lens = _as_len_list(seq_lens)
    T = sum(lens)
    H, D = head_num, size_per_head
    rnd = (lambda t: t.to(storage_dtype).to(acc_dtype)) if storage_dtype is not None else (lambda t: t.to(acc_dtype))

    x = depad(hidden_padded, B, lens, left_padded=left_padded)
    qkv = transpose_pad(qkv_packed, B, S, lens, H, 3 * D)
    q, k, v = torch.chunk(qkv, 3, dim=-1)
    scores = rnd(attn_qk(q, k, acc_dtype))
    probs = rnd(scale_mask_softmax(B, S, H, scores, lens, scale=scale, causal=causal, acc_dtype=acc_dtype,
                                   out_dtype=acc_dtype))
    # rows of padded queries hold raw scores (reference quirk); they never reach the output
    ctx = rnd(attn_pv(probs, v, acc_dtype))
    ctx_packed = transpose_depad(ctx, B, T, S, lens, H, D)
    attn_out = ctx_packed.reshape(1, T, H * D) if dense_out is None else dense_out
    y, mean, invvar, _ = layer_norm(attn_out, gamma, beta, eps, residual=x, acc_dtype=acc_dtype,
                                    out_dtype=acc_dtype)
    return dict(x=x, qkv=qkv, scores=scores, probs=probs, ctx=ctx, ctx_packed=ctx_packed, y=y, mean=mean,
                invvar=invvar)


def layer_padded(hidden_padded: torch.Tensor, qkv_padded: torch.Tensor, seq_lens, head_num: int,
                 size_per_head: int, gamma: torch.Tensor, beta: torch.Tensor, eps: float, scale: float,
                 causal: bool, left_padded: bool = False, acc_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """The ordinary padded layer the reference models run (no padding removal).

    energonai/model/attention.py:101-124 + endecoder.py:48-70 shape, with the
    masks of model_factory.py:117-121 (additive -1e4) and the fp32 softmax.
    ``qkv_padded`` is [B,S,H,3D].  Returns LN(attn + hidden) as [B,S,hid]; only
    rows of valid tokens are meaningful.  Requires H*D == hid.
    """
    B, S, hid = hidden_padded.shape
    H, D = head_num, size_per_head
    lens = torch.tensor(_as_len_list(seq_lens))
    qkv = qkv_padded.to(acc_dtype).permute(0, 2, 1, 3)
    q, k, v = torch.chunk(qkv, 3, dim=-1)
    x = torch.matmul(q, k.transpose(-1, -2)) * scale
    pos = torch.arange(S)
    if left_padded:
        key_ok = pos.view(1, S) >= (S - lens).view(B, 1)
    else:
        key_ok = pos.view(1, S) < lens.view(B, 1)
    if causal:
        tri = torch.tril(torch.ones(S, S, dtype=torch.bool)).view(1, 1, S, S)
        x = torch.where(tri, x, torch.tensor(-1e4, dtype=acc_dtype))
    x = x + (~key_ok).to(acc_dtype).view(B, 1, 1, S) * -10000.0
    p = torch.softmax(x, -1)
    ctx = torch.matmul(p, v).permute(0, 2, 1, 3).reshape(B, S, H * D)
    y, _, _, _ = layer_norm(ctx, gamma, beta, eps, residual=hidden_padded, acc_dtype=acc_dtype,
                            out_dtype=acc_dtype)
    return y


def decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, kv_lens, scale: float,
                     acc_dtype: torch.dtype = torch.float32):
    """Single-query attention over a ragged cache.

    q [B,H,1,D]; caches [B,H,Smax,D]; the query is the last position, so it
    sees every cached key k < kv_len[b].  This is the last query row of the
    reference's concat-and-recompute cache (energonai/model/attention.py:61-71,
    106-118).  Returns (scores[B,H,1,Smax], probs, ctx[B,H,1,D]).
    """
    B, H, _, D = q.shape
    Smax = k_cache.shape[2]
    lens = _as_len_list(kv_lens)
    scores = attn_qk(q, k_cache, acc_dtype)
    probs = scale_mask_softmax(B, 1, H, scores, lens, scale=scale, causal=True, k_seq_len=Smax,
                               q_lens=[1] * B, acc_dtype=acc_dtype, out_dtype=acc_dtype)
    vz = v_cache.to(acc_dtype).clone()
    for b in range(B):
        vz[b, :, lens[b]:, :] = 0
    ctx = torch.matmul(probs, vz)
    return scores, probs, ctx
