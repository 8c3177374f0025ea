"""Drop-in for the reference's ``energonai.kernel`` package (energonai/kernel/__init__.py:1-10).

Same names, same positional signatures; every function runs hand-written
gfx950 kernels through the C ABI of libenergon_hip.so.  ``attn_qk`` /
``attn_pv`` / ``decode_qk`` / ``decode_pv`` are additions: the reference
callers use ``torch.matmul`` for the two contractions.  ``attn_fused`` and
``attn_fused_packed`` run the contractions and the softmax in one kernel, ``decode_attn``
does the same for the single-query step of cached decode (``decode_attn_paged``, ``kv_pages_fill`` and
``kv_pages_append`` for caches kept in pages of a shared pool);
``attn_qk_varlen`` / ``attn_pv_varlen`` are the two contractions on packed tokens
(no ``transpose_pad`` / ``transpose_depad`` around them), optionally with the scores in
the packed causal layout that ``scale_mask_softmax_packed`` works on.
"""
from .cuda_native import transpose_pad, transpose_depad, depad, repad, scale_mask_softmax
from .cuda_native import (ft_build_padding_offsets, ft_remove_padding, ft_rebuild_padding,
                          ft_transpose_remove_padding, ft_transpose_rebuild_padding)
from .cuda_native import linear, find_algo
from .cuda_native import LayerNorm, layer_norm_forward
from .attention import (attn_qk, attn_pv, attn_fused, attn_fused_packed, attn_fused_varlen, decode_qk, decode_pv, decode_attn,
                        decode_attn_workspace_bytes, decode_attn_paged, kv_pages_fill, kv_pages_append,
                        kv_cache_fill, kv_cache_append, attn_qk_varlen, attn_pv_varlen, scale_mask_softmax_packed,
                        packed_scores_elems)

__all__ = [
    "transpose_pad", "transpose_depad", "depad", "scale_mask_softmax", "ft_build_padding_offsets",
    "ft_remove_padding", "ft_rebuild_padding", "ft_transpose_remove_padding", "ft_transpose_rebuild_padding",
    "linear", "find_algo", "LayerNorm", "layer_norm_forward", "attn_qk", "attn_pv", "attn_fused",
    "attn_fused_packed", "attn_fused_varlen", "decode_qk", "decode_pv", "decode_attn", "decode_attn_workspace_bytes", "decode_attn_paged",
    "kv_pages_fill", "kv_pages_append", "kv_cache_fill", "kv_cache_append", "repad",
    "attn_qk_varlen", "attn_pv_varlen", "scale_mask_softmax_packed", "packed_scores_elems",
]
