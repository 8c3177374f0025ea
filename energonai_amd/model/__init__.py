"""Attention / MLP / block modules with the constructor and ``forward`` signatures of the
reference's ``energonai.model`` layers (energonai/model/attention.py:9-136, mlp.py:7-51,
endecoder.py:11-70), routed through the padding-removal kernels of this package.

At tensor-parallel size 1 the reference's ``Linear1D_Col`` / ``Linear1D_Row`` are plain
linear layers, so ``torch.nn.Linear`` (a library GEMM) stands in for them with the same
attribute names; ``LayerNorm1D`` becomes the fused LayerNorm of ``energonai_amd.kernel``.
"""
from .gemm import gemm_tuning, set_gemm_tuning
from .kv_cache import KVCache, PagedKVCache
from .attention import MultiHeadAttention1D
from .mlp import MLP1D
from .endecoder import Block1D
from .stack import PackedStack

__all__ = ["KVCache", "PagedKVCache", "MultiHeadAttention1D", "MLP1D", "Block1D", "PackedStack", "set_gemm_tuning", "gemm_tuning"]
