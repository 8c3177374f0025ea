"""Stand-ins for the reference's compiled extension modules.

The reference's Python wrappers load four pybind11 modules by name
(``importlib.import_module("energonai_transpose_pad")`` etc.,
energonai/kernel/cuda_native/transpose_pad.py:4-7, scale_mask_softmax.py:4-7,
layer_norm.py:53-58, linear_func.py:5-8; names fixed in setup.py:132-147).
The modules in this package expose the same ``*_wrapper`` / ``forward_affine``
functions on top of libenergon_hip.so, so the reference's own
``energonai/kernel`` package runs unmodified once they are importable under
those names: call :func:`install` before ``import energonai.kernel``.
"""
import importlib
import sys

_NAMES = ("energonai_transpose_pad", "energonai_scale_mask", "energonai_layer_norm", "energonai_linear_func")


def install() -> None:
    """Registers the stand-ins in ``sys.modules`` under the reference's extension names."""
    for name in _NAMES:
        sys.modules.setdefault(name, importlib.import_module(f"{__name__}.{name}"))
