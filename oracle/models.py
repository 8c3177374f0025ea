"""Torch-eager restatement (CPU, fp32) of the reference's model layers on PADDED batches.

TEST INFRASTRUCTURE ONLY, like the rest of this package.  Each function follows the
reference forward it cites with ``disable_past_cache=True`` (every position recomputed);
the reference's cached decode returns, for the newest position, the last row of that
full recomputation (energonai/model/attention.py:61-71,126-135), which is how the
incremental path of the product is checked.

Weights are passed as plain dicts of fp32 tensors named like the module attributes.

Pinning: ``mha_forward`` is checked in tests/test_oracle_models.py against
``torch.nn.functional.multi_head_attention_forward`` (library routine; the k, v, q order
of the fused projection is taken from attention.py:74 and enters that check as a
permutation of the weight thirds), ``mlp_forward`` / ``block_forward`` against
compositions of library ``linear`` / ``layer_norm`` calls written in the other order of
evaluation.  The reference has no test for these modules: by its own tests PARITY UNPINNED.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch
import torch.nn.functional as F


def additive_mask(valid: torch.Tensor) -> torch.Tensor:
    """[B,S] 0/1 validity -> the [B,1,1,S] additive mask of energonai/model/model_factory.py:117-121."""
    m = valid.to(torch.float32).view(valid.shape[0], -1).unsqueeze(1).unsqueeze(2)
    return (1.0 - m) * -10000.0


def mha_forward(hidden: torch.Tensor, p: Dict[str, torch.Tensor], num_heads: int, is_decoder: bool,
                attention_mask: Optional[torch.Tensor] = None, fused_qkv: bool = True) -> torch.Tensor:
    """energonai/model/attention.py:56-136 without the past cache."""
    B, S, hid = hidden.shape
    D = hid // num_heads
    x = hidden.float()
    if fused_qkv:
        kvq = F.linear(x, p["query_key_value.weight"], p.get("query_key_value.bias"))
        k, v, q = torch.chunk(kvq, 3, dim=-1)                         # attention.py:74
    else:
        q = F.linear(x, p["query_.weight"], p.get("query_.bias"))
        k = F.linear(x, p["key_.weight"], p.get("key_.bias"))
        v = F.linear(x, p["value_.weight"], p.get("value_.bias"))

    def split(t):                                                     # attention.py:46-49
        return t.reshape(B, S, num_heads, D).permute(0, 2, 1, 3)

    q, k, v = split(q), split(k), split(v)
    q = q * (D ** -0.5)                                               # attention.py:103
    scores = torch.matmul(q, k.transpose(-1, -2))
    if is_decoder:                                                    # attention.py:108-110
        causal = torch.tril(torch.ones(S, S, dtype=torch.bool)).view(1, 1, S, S)
        scores = torch.where(causal, scores, torch.tensor(-1e4))
    if attention_mask is not None:                                    # attention.py:112-113
        scores = scores + attention_mask.float()
    probs = torch.softmax(scores, -1, dtype=torch.float)              # attention.py:115
    ctx = torch.matmul(probs, v).transpose(1, 2).reshape(B, S, hid)   # attention.py:117-123
    return F.linear(ctx, p["dense.weight"], p["dense.bias"])


def mlp_forward(hidden: torch.Tensor, p: Dict[str, torch.Tensor], activation: Callable) -> torch.Tensor:
    """energonai/model/mlp.py:30-35."""
    h = F.linear(hidden.float(), p["dense_1.weight"], p.get("dense_1.bias"))
    return F.linear(activation(h), p["dense_2.weight"], p.get("dense_2.bias"))


def block_forward(hidden: torch.Tensor, p: Dict[str, torch.Tensor], num_heads: int, eps: float,
                  apply_post_layernorm: bool, is_decoder: bool, attention_mask: Optional[torch.Tensor],
                  activation: Callable = F.gelu, fused_qkv: bool = True) -> torch.Tensor:
    """energonai/model/endecoder.py:48-70 (LayerNorm1D taken as the textbook LayerNorm)."""
    hid = hidden.shape[-1]
    x = hidden.float()
    sub = lambda prefix: {k[len(prefix):]: v for k, v in p.items() if k.startswith(prefix)}
    if not apply_post_layernorm:
        residual = x
    h = F.layer_norm(x, (hid,), p["norm1.weight"], p["norm1.bias"], eps)
    if apply_post_layernorm:
        residual = h
    h = residual + mha_forward(h, sub("attn."), num_heads, is_decoder, attention_mask, fused_qkv)
    if not apply_post_layernorm:
        residual = h
    h = F.layer_norm(h, (hid,), p["norm2.weight"], p["norm2.bias"], eps)
    if apply_post_layernorm:
        residual = h
    return residual + mlp_forward(h, sub("mlp."), activation)
