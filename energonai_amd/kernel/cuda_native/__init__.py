"""Mirror of energonai/kernel/cuda_native/__init__.py:1-5 (the subpackage name
is kept so ``...kernel.cuda_native.LayerNorm`` resolves as in the reference)."""
from .transpose_pad import transpose_pad, transpose_depad, depad, repad
from .transpose_pad import (ft_build_padding_offsets, ft_remove_padding, ft_rebuild_padding,
                            ft_transpose_remove_padding, ft_transpose_rebuild_padding)
from .scale_mask_softmax import scale_mask_softmax
from .layer_norm import MixedFusedLayerNorm as LayerNorm
from .layer_norm import MixedFusedLayerNorm, layer_norm_forward
from .linear_func import linear, find_algo
