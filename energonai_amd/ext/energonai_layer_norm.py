"""Same forward entry as the reference's ``energonai_layer_norm`` extension
(csrc/layer_norm_cuda.cpp:137-141).  ``backward_affine`` is not provided:
the path is inference only."""
from ..kernel.cuda_native.layer_norm import layer_norm_forward as _fwd


def forward_affine(input, normalized_shape, gamma, beta, epsilon):
    out, mean, invvar = _fwd(input, gamma, beta, normalized_shape, epsilon, return_stats=True)
    return [out, mean, invvar]


def backward_affine(*args, **kwargs):
    raise RuntimeError("energonai_layer_norm.backward_affine: inference-only build, backward is not implemented")
