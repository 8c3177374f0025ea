"""Pure-Python replay of the reference CUDA kernels' index arithmetic (test oracle).

TEST INFRASTRUCTURE ONLY.  Each function walks the reference launch grid
(blockIdx / threadIdx as plain loops) over flat Python lists, for tiny inputs,
so that the vectorised restatement in eager.py is pinned by something that
shares none of its code.
"""
from __future__ import annotations

import math
from typing import List, Sequence


def transpose_pad(src: Sequence[float], batch_size: int, seq_len: int, seq_lens: Sequence[int], head_num: int,
                  size_per_head: int) -> List[float]:
    """csrc/transpose_pad_fusion_kernel.cu:58-84 over grid B*H*S, one thread per element."""
    dst = [None] * (batch_size * head_num * seq_len * size_per_head)
    for block in range(batch_size * head_num * seq_len):
        batch_index = block // (head_num * seq_len)
        head_index = (block % (head_num * seq_len)) // seq_len
        seq_index = block % seq_len
        sum_len = 0
        for i in range(batch_index):
            sum_len += seq_lens[i]
        for idx in range(size_per_head):
            if seq_index >= seq_lens[batch_index]:
                dst[block * size_per_head + idx] = 0.0
            else:
                dst[block * size_per_head + idx] = src[(sum_len + seq_index) * (head_num * size_per_head)
                                                       + head_index * size_per_head + idx]
    return dst


def transpose_depad(src: Sequence[float], batch_size: int, seq_len: int, seq_lens: Sequence[int], head_num: int,
                    size_per_head: int) -> List[float]:
    """csrc/transpose_pad_fusion_kernel.cu:8-35; dst starts as zeros (wrapper.cpp:70)."""
    total = sum(seq_lens[:batch_size])
    dst = [0.0] * (total * head_num * size_per_head)
    for block in range(batch_size * head_num * seq_len):
        batch_index = block // (head_num * seq_len)
        head_index = (block % (head_num * seq_len)) // seq_len
        seq_index = block % seq_len
        if seq_index >= seq_lens[batch_index]:
            continue
        sum_len = 0
        for i in range(batch_index):
            sum_len += seq_lens[i]
        for idx in range(size_per_head):
            dst[(sum_len + seq_index) * (head_num * size_per_head) + head_index * size_per_head + idx] = \
                src[block * size_per_head + idx]
    return dst


def build_offsets(seq_lens: Sequence[int], batch_size: int, max_seq_len: int):
    """csrc/transpose_pad_fusion_kernel.cu:112-131 (the <<<1,1>>> serial kernel)."""
    off = []
    total = 0
    cum = 0
    for i in range(batch_size):
        n = seq_lens[i]
        for _ in range(n):
            off.append(cum)
        cum += max_seq_len - n
        total += n
    return total, off


def remove_padding(src: Sequence[float], off: Sequence[int], m: int, n: int) -> List[float]:
    """csrc/transpose_pad_fusion_kernel.cu:142-156: tgt[bid] = src[bid + off[bid]]."""
    tgt = [None] * (m * n)
    for bid in range(m):
        s = bid + off[bid]
        for i in range(n):
            tgt[bid * n + i] = src[s * n + i]
    return tgt


def rebuild_padding(src: Sequence[float], off: Sequence[int], m: int, n: int, rows_out: int) -> List[float]:
    """csrc/transpose_pad_fusion_kernel.cu:178-189 into a zero buffer (wrapper.cpp:158)."""
    tgt = [0.0] * (rows_out * n)
    for bid in range(m):
        t = bid + off[bid]
        for i in range(n):
            tgt[t * n + i] = src[bid * n + i]
    return tgt


def transpose_rebuild_padding(Q: Sequence[float], buf: List[float], seq_len: int, head_num: int,
                              size_per_head: int, off: Sequence[int], valid: int) -> None:
    """csrc/transpose_pad_fusion_kernel.cu:213-236 for one of the three tensors, in place."""
    bdim = head_num * size_per_head
    for bid in range(valid):
        for tid in range(bdim):
            tb = (bid + off[bid]) // seq_len
            ts = (bid + off[bid]) % seq_len
            th = tid // size_per_head
            td = tid % size_per_head
            buf[tb * head_num * seq_len * size_per_head + th * seq_len * size_per_head + ts * size_per_head + td] = \
                Q[bid * bdim + tid]


def transpose_remove_padding(src: Sequence[float], seq_len: int, head_num: int, size_per_head: int,
                             off: Sequence[int], valid: int) -> List[float]:
    """csrc/transpose_pad_fusion_kernel.cu:268-289."""
    bdim = head_num * size_per_head
    dst = [None] * (valid * bdim)
    for bid in range(valid):
        sb = (bid + off[bid]) // seq_len
        ss = (bid + off[bid]) % seq_len
        for tid in range(bdim):
            h = tid // size_per_head
            d = tid % size_per_head
            dst[bid * bdim + tid] = src[sb * head_num * seq_len * size_per_head + h * seq_len * size_per_head
                                        + ss * size_per_head + d]
    return dst


def softmax_reference_kernel(corr: List[float], real_seq_len: Sequence[int], batch_size: int, head_num: int,
                             batch_seq_len: int) -> None:
    """csrc/scale_mask_softmax_kernel.cu:11-42 over grid (B, H*S), block S threads; in place.

    -inf is the reference's -1e8 (csrc/common.h:15).
    """
    NEG = -100000000.0
    S = batch_seq_len
    grid_y = head_num * S
    for bx in range(batch_size):
        for by in range(grid_y):
            qpos = by % S
            if qpos >= real_seq_len[bx]:
                continue
            base = (bx * grid_y + by) * S
            vals = [corr[base + t] for t in range(S)]
            masked = [t > qpos for t in range(S)]
            mx = max(NEG if masked[t] else vals[t] for t in range(S))
            ex = [0.0 if masked[t] else math.exp(vals[t] - mx) for t in range(S)]
            sm = sum(ex)
            for t in range(S):
                corr[base + t] = ex[t] / sm


def layer_norm_rows(x: Sequence[float], n1: int, n2: int, gamma: Sequence[float], beta: Sequence[float],
                    eps: float):
    """csrc/layer_norm_cuda_kernel.cu:14-22,243-279 with the serial Welford update per row.

    Returns (y, mean, invvar) as Python lists; arithmetic in Python floats
    (float64), so it pins the definition, not fp32 rounding.
    """
    y = [0.0] * (n1 * n2)
    means, invvars = [], []
    for i1 in range(n1):
        count = 0.0
        mu = 0.0
        m2 = 0.0
        for i in range(n2):
            curr = x[i1 * n2 + i]
            count += 1.0
            delta = curr - mu
            mu = mu + delta / count
            m2 = m2 + delta * (curr - mu)
        sigma2 = m2 / n2
        inv = 1.0 / math.sqrt(sigma2 + eps)
        for i in range(n2):
            y[i1 * n2 + i] = gamma[i] * (inv * (x[i1 * n2 + i] - mu)) + beta[i]
        means.append(mu)
        invvars.append(inv)
    return y, means, invvars
