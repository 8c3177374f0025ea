"""The five benchmark / parity workloads and their seeded synthetic inputs.

Shapes follow the layer sizes of the reference model factories
(energonai/model/model_factory.py:256-354: hidden, heads) with the padding-removal
call pattern of examples/bert/bert.py:91-134.  Lengths come from
``torch.Generator().manual_seed(20240 + i)`` and activations from
``manual_seed(1000 + i)``, both on the CPU, so a CPU run and a GPU run see the
same bits.  Only valid tokens are drawn; padding is zero.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch


@dataclass(frozen=True)
class Workload:
    index: int
    name: str
    title: str
    dtype: torch.dtype
    batch: int
    seq: int            # bucket (padded) length; for decode the cache capacity
    heads: int          # local heads on this GPU
    head_dim: int
    hidden: int         # LayerNorm width
    len_lo: int
    len_hi: int
    causal: bool
    left_padded: bool
    decode: bool = False

    @property
    def scale(self) -> float:
        return float(self.head_dim) ** -0.5

    @property
    def attn_width(self) -> int:
        return self.heads * self.head_dim


WORKLOADS = (
    Workload(0, "c1", "BERT-base layer, fp32", torch.float32, 8, 128, 12, 64, 768, 16, 128, False, False),
    Workload(1, "c2", "OPT-125M layer, TP=1, fp16", torch.float16, 32, 512, 12, 64, 768, 64, 512, True, True),
    Workload(2, "c3", "OPT-30B layer, TP=1, fp16", torch.float16, 16, 1024, 56, 128, 7168, 128, 1024, True, True),
    Workload(3, "c4", "GPT-3 175B layer, one TP=8 share, fp16", torch.float16, 16, 2048, 12, 128, 12288, 256, 2048,
             True, True),
    Workload(4, "c5", "OPT-66B cached decode, fp16", torch.float16, 64, 2048, 72, 128, 9216, 1, 2048, True, False,
             decode=True),
)
BY_NAME = {w.name: w for w in WORKLOADS}

EPS = 1e-5


def make_lens(w: Workload) -> torch.Tensor:
    g = torch.Generator().manual_seed(20240 + w.index)
    return torch.randint(w.len_lo, w.len_hi + 1, (w.batch,), generator=g, dtype=torch.int32)


def _pad_rows(packed: torch.Tensor, lens, S: int, left: bool) -> torch.Tensor:
    """[T, W] -> zero-padded [B, S, W]."""
    B = len(lens)
    out = torch.zeros(B, S, packed.shape[1], dtype=packed.dtype)
    t = 0
    for b, n in enumerate(lens):
        if left:
            out[b, S - n:] = packed[t:t + n]
        else:
            out[b, :n] = packed[t:t + n]
        t += n
    return out


def make_inputs(w: Workload, device="cpu", dtype: Optional[torch.dtype] = None,
                lens: Optional[torch.Tensor] = None) -> Dict[str, object]:
    """Inputs of one prefill layer (c1-c4).  Tensors are drawn in fp32 on the CPU,
    cast to ``dtype`` (default: the workload's) and moved to ``device``."""
    if w.decode:
        raise ValueError("use make_decode_inputs for the decode workload")
    dtype = dtype or w.dtype
    lens = make_lens(w) if lens is None else lens.to(torch.int32).cpu()
    lens_list = [int(v) for v in lens]
    T = sum(lens_list)
    g = torch.Generator().manual_seed(1000 + w.index)
    x = torch.randn(T, w.hidden, generator=g)
    qkv = torch.randn(T, w.heads * 3 * w.head_dim, generator=g)
    dense = torch.randn(T, w.hidden, generator=g) if w.attn_width != w.hidden else None
    gamma = 1.0 + 0.02 * torch.randn(w.hidden, generator=g)
    beta = 0.02 * torch.randn(w.hidden, generator=g)
    hidden_padded = _pad_rows(x.to(dtype), lens_list, w.seq, w.left_padded)
    out = dict(
        lens=lens, lens_list=lens_list, total=T,
        hidden_padded=hidden_padded.to(device),
        qkv_packed=qkv.to(dtype).reshape(1, T, w.heads, 3 * w.head_dim).to(device),
        dense_out=None if dense is None else dense.to(dtype).reshape(1, T, w.hidden).to(device),
        gamma=gamma.to(dtype).to(device), beta=beta.to(dtype).to(device),
    )
    return out


def make_decode_inputs(w: Workload, device="cpu", dtype: Optional[torch.dtype] = None,
                       lens: Optional[torch.Tensor] = None, cache_on_device: bool = False) -> Dict[str, object]:
    """Inputs of one decode step (c5): one query per sequence and a ragged cache
    [B,H,Smax,D].  With ``cache_on_device`` the two caches (2.4 GB each at full
    size) are drawn by a seeded generator on ``device`` instead of the CPU; all
    other tensors are still drawn on the CPU."""
    dtype = dtype or w.dtype
    lens = make_lens(w) if lens is None else lens.to(torch.int32).cpu()
    lens_list = [int(v) for v in lens]
    g = torch.Generator().manual_seed(1000 + w.index)
    B, H, D, S = w.batch, w.heads, w.head_dim, w.seq
    q = torch.randn(B, H, 1, D, generator=g)
    residual = torch.randn(1, B, w.hidden, generator=g)
    dense = torch.randn(1, B, w.hidden, generator=g)
    gamma = 1.0 + 0.02 * torch.randn(w.hidden, generator=g)
    beta = 0.02 * torch.randn(w.hidden, generator=g)
    if cache_on_device:
        gd = torch.Generator(device=device).manual_seed(2000 + w.index)
        k_cache = torch.randn(B, H, S, D, generator=gd, device=device, dtype=dtype)
        v_cache = torch.randn(B, H, S, D, generator=gd, device=device, dtype=dtype)
    else:
        k_cache = torch.randn(B, H, S, D, generator=g).to(dtype).to(device)
        v_cache = torch.randn(B, H, S, D, generator=g).to(dtype).to(device)
    return dict(
        lens=lens, lens_list=lens_list, total=B, kv_total=sum(lens_list),
        q=q.to(dtype).to(device), k_cache=k_cache, v_cache=v_cache,
        residual=residual.to(dtype).to(device), dense_out=dense.to(dtype).to(device),
        gamma=gamma.to(dtype).to(device), beta=beta.to(dtype).to(device),
    )


def algorithmic_bytes(w: Workload, lens_list) -> Dict[str, float]:
    """Bytes each kernel must move at minimum (e = element size): the roofline numerators."""
    e = torch.empty(0, dtype=w.dtype).element_size()
    H, D, S, hid, B = w.heads, w.head_dim, w.seq, w.hidden, w.batch
    if w.decode:
        kv = sum(lens_list)
        return dict(decode_qk=H * kv * D * e + H * kv * e, decode_pv=H * kv * D * e + H * kv * e,
                    scale_mask_softmax=2 * H * kv * e, layernorm_residual=3 * B * hid * e,
                    decode_attn=2 * H * kv * D * e + 2 * B * H * D * e)    # K and V once; q in, ctx out
    T = sum(lens_list)
    vis = sum(n * (n + 1) // 2 for n in lens_list) if w.causal else sum(n * n for n in lens_list)
    return dict(
        depad=2 * T * hid * e,
        transpose_pad=T * H * 3 * D * e + B * S * H * 3 * D * e,
        transpose_depad=2 * T * H * D * e,
        scale_mask_softmax=H * e * vis + H * e * T * S,
        scale_mask_softmax_no_tail=2 * H * e * vis,   # the form in the step: the visible prefix in, the same out
        layernorm_residual=3 * T * hid * e,
        attn_qk=H * e * vis + 2 * T * H * D * e,
        attn_pv=H * e * vis + 2 * T * H * D * e,
    )


def algorithmic_flops(w: Workload, lens_list) -> float:
    """FLOPs of one contraction (QK^T and PV cost the same) over the visible region only."""
    H, D = w.heads, w.head_dim
    if w.decode:
        return 2.0 * H * D * sum(lens_list)
    vis = sum(n * (n + 1) // 2 for n in lens_list) if w.causal else sum(n * n for n in lens_list)
    return 2.0 * H * D * vis
