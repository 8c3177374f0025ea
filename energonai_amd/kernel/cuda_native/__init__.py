"""The subpackage name of the reference is kept so that ``...kernel.cuda_native.LayerNorm`` and the other
public names resolve as they do there (energonai/kernel/cuda_native/__init__.py:1-5)."""
from . import layer_norm as _ln
from . import linear_func as _lin
from . import scale_mask_softmax as _sm
from . import transpose_pad as _tp

# packing / unpacking
transpose_pad, transpose_depad = _tp.transpose_pad, _tp.transpose_depad
depad, repad = _tp.depad, _tp.repad
ft_build_padding_offsets = _tp.ft_build_padding_offsets
ft_remove_padding, ft_rebuild_padding = _tp.ft_remove_padding, _tp.ft_rebuild_padding
ft_transpose_remove_padding = _tp.ft_transpose_remove_padding
ft_transpose_rebuild_padding = _tp.ft_transpose_rebuild_padding

# softmax, LayerNorm, projection GEMM
scale_mask_softmax = _sm.scale_mask_softmax
MixedFusedLayerNorm = LayerNorm = _ln.MixedFusedLayerNorm
layer_norm_forward = _ln.layer_norm_forward
linear, find_algo = _lin.linear, _lin.find_algo
