"""energonai_amd: MI355X (gfx950) implementation of EnergonAI's per-layer
padding-removal hot path behind the reference's ``energonai.kernel`` API.

    from energonai_amd.kernel import transpose_pad, transpose_depad, depad, scale_mask_softmax
    from energonai_amd.kernel.cuda_native import LayerNorm

Host code is Python on PyTorch-ROCm (tensors, allocator, streams); all compute
runs in hand-written HIP kernels behind the C ABI of ``libenergon_hip.so``
(``include/energon_hip.h``).  There is no CPU fallback: importing
``energonai_amd.kernel`` without the built library raises RuntimeError.
"""
__version__ = "0.1.0"

__all__ = ["__version__"]
