"""ctypes binding of libenergon_hip.so (the C ABI declared in include/energon_hip.h).

The library is the only compute path: there is no CPU or torch fallback.  If
the shared object has not been built, loading raises RuntimeError with the
reference's wording ("... requires cuda extensions",
energonai/kernel/cuda_native/transpose_pad.py:4-7).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

import torch

LIB_NAME = "libenergon_hip.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

EN_F32, EN_F16, EN_BF16 = 0, 1, 2
_DTYPE_TAG = {torch.float32: EN_F32, torch.float16: EN_F16, torch.bfloat16: EN_BF16}

# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "en_version": (c_int, []),
    "en_source_hash": (c_char_p, []),
    "en_status_string": (c_char_p, [c_int]),
    "en_last_hip_error": (c_int, []),
    "en_last_hip_error_string": (c_char_p, []),
    "en_prefix_sum": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "en_depad": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_int, c_void_p]),
    "en_repad": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_int, c_void_p]),
    "en_transpose_pad": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "en_transpose_pad_heads": (c_int, [c_void_p, c_void_p, c_void_p] + [c_int] * 8 + [c_void_p]),
    "en_kv_append": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_int64] * 5 + [c_int, c_void_p, c_void_p]),
    "en_transpose_depad": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "en_ft_build_offsets": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "en_ft_remove_padding": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_void_p]),
    "en_ft_rebuild_padding": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_void_p]),
    "en_ft_transpose_rebuild": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p, c_int, c_void_p]),
    "en_ft_transpose_remove": (c_int, [c_void_p, c_void_p] + [c_int] * 5 + [c_void_p, c_int, c_void_p]),
    "en_scale_mask_softmax": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                      c_int, c_void_p]),
    "en_layernorm_fwd": (c_int, [c_void_p] * 9 + [c_int64, c_int64, c_float, c_int, c_int, c_void_p]),
    "en_padding_offsets": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "en_attn_qk": (c_int, [c_void_p] * 5 + [c_int] * 5 + [c_int64] * 6 + [c_float, c_int, c_int, c_void_p, c_void_p,
                           c_int, c_void_p, c_void_p]),
    "en_attn_pv": (c_int, [c_void_p] * 5 + [c_int] * 5 + [c_int64] * 6 + [c_int, c_int, c_int, c_void_p, c_void_p,
                           c_int, c_void_p, c_void_p]),
    "en_attn_tile_table_elems": (c_int64, [c_int] * 4),
    "en_attn_tile_table": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "en_attn_fused_query_tile": (c_int, [c_int] * 5),
    "en_packed_scores_elems": (c_int64, [c_int] * 4),
    "en_scale_mask_softmax_packed": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_int, c_void_p]),
    "en_decode_qk": (c_int, [c_void_p] * 4 + [c_int] * 4 + [c_int64] * 3 + [c_float, c_int, c_void_p]),
    "en_decode_pv": (c_int, [c_void_p] * 4 + [c_int] * 4 + [c_int64] * 3 + [c_int, c_void_p]),
    "en_decode_attn": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_void_p, c_void_p, c_float, c_int, c_void_p, c_int64, c_void_p]),
    "en_decode_attn_workspace_bytes": (c_int64, [c_int] * 4),
    "en_decode_attn_paged": (c_int, [c_void_p] * 6 + [c_int] * 6 + [c_void_p, c_void_p, c_float, c_int, c_void_p, c_int64, c_void_p]),
    "en_kv_append_paged": (c_int, [c_void_p] * 6 + [c_int] * 6 + [c_int64, c_int64, c_void_p, c_int, c_void_p, c_void_p]),
    "en_kv_fill_paged": (c_int, [c_void_p] * 4 + [c_int] * 9 + [c_void_p, c_int, c_void_p, c_void_p]),
    "en_attn_fused": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_void_p] * 6 + [c_float, c_int, c_int, c_void_p, c_int, c_void_p]),
    "en_padding_removal_layer": (c_int, [c_void_p] * 13 + [c_int] * 4 + [c_int64, c_int64, c_float, c_float] + [c_int] * 3 + [c_void_p, c_int, c_void_p, c_void_p]),
    "en_padding_removal_layer_noalloc": (c_int, [c_void_p] * 7 + [c_int] * 5 + [c_int64, c_int64, c_float, c_float] +
                                         [c_int] * 5 + [c_void_p]),
    "en_copy_bytes": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "en_stream_yardstick": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "en_prefix_yardstick": (c_int, [c_void_p, c_void_p, c_void_p] + [c_int] * 7 + [c_void_p]),
}

LINEAR_LIB_NAME = "libenergon_linear.so"
LINEAR_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LINEAR_LIB_NAME)
LINEAR_SIGNATURES = {
    "en_linear": (c_int, [c_void_p] * 4 + [c_int64] * 3 + [c_int] * 3 + [c_void_p, c_int64, c_void_p]),
    "en_linear_algo_count": (c_int, [c_int64] * 3 + [c_int] * 3 + [c_int64]),
    "en_linear_status_string": (ctypes.c_char_p, [c_int]),
    "en_linear_source_hash": (ctypes.c_char_p, []),
}

_lib = None
_linear_lib = None


def _refuse_stale(lib, symbol: str, expected: str, path: str) -> None:
    """A library compiled from other sources than the ones beside it would make every test and measurement
    speak for code that is not in the tree."""
    fn_ = getattr(lib, symbol)
    fn_.restype = c_char_p
    fn_.argtypes = []
    built = fn_().decode()
    if built != expected:
        raise RuntimeError(f"energonai_amd requires cuda extensions: {path} was built from other sources "
                           f"(library {built}, tree {expected}); run `python -m energonai_amd.build`")


def load_linear() -> ctypes.CDLL:
    """Loads the hipBLASLt front end once; raises RuntimeError if it is not built."""
    global _linear_lib
    if _linear_lib is None:
        if not os.path.exists(LINEAR_LIB_PATH):
            raise RuntimeError(f"energonai_linear_func requires cuda extensions: {LINEAR_LIB_NAME} is not built "
                               f"(run `python -m energonai_amd.build`)")
        try:
            lib = ctypes.CDLL(LINEAR_LIB_PATH)
        except OSError as exc:
            raise RuntimeError(f"energonai_linear_func requires cuda extensions: cannot load {LINEAR_LIB_PATH}: {exc}") from exc
        from . import build
        _refuse_stale(lib, "en_linear_source_hash", build.linear_source_hash(), LINEAR_LIB_PATH)
        for name, (restype, argtypes) in LINEAR_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _linear_lib = lib
    return _linear_lib


def load() -> ctypes.CDLL:
    """Loads the shared library once; raises RuntimeError if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"energonai_amd requires cuda extensions: {LIB_NAME} is not built "
                f"(run `python -m energonai_amd.build`)")
        try:
            lib = ctypes.CDLL(LIB_PATH)
        except OSError as exc:
            raise RuntimeError(f"energonai_amd requires cuda extensions: cannot load {LIB_PATH}: {exc}") from exc
        from . import build
        _refuse_stale(lib, "en_source_hash", build.source_hash(), LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(status: int, op: str) -> None:
    """Turns a non-zero en_status into RuntimeError naming the op."""
    if status == 0:
        return
    lib = load()
    msg = lib.en_status_string(status).decode()
    if status == -6:
        msg += f": {lib.en_last_hip_error_string().decode()} (hipError {lib.en_last_hip_error()})"
    raise RuntimeError(f"{op}: {msg}")


def dtype_tag(t: torch.Tensor, op: str) -> int:
    try:
        return _DTYPE_TAG[t.dtype]
    except KeyError:
        raise RuntimeError(f"{op}: Datatype not implemented ({t.dtype}); expected float32, float16 or bfloat16") from None


def require_gpu(t: torch.Tensor, name: str, contiguous: bool = True) -> None:
    """The reference's CHECK_CUDA / CHECK_CONTIGUOUS (csrc/transpose_pad_fusion_wrapper.cpp:19-31)."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if contiguous and not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def stream_of(t: torch.Tensor) -> int:
    """Raw handle of torch's current stream on t's device (kernels launch there, never on the default stream)."""
    return torch._C._cuda_getCurrentRawStream(t.device.index)


class _NoGuard:
    __slots__ = ()

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(t: torch.Tensor):
    """Context that makes t's device current for the launch; free when it already is."""
    if t.device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(t.device)


class _Fns:
    """Attribute access to the bound entry points: ``fn.en_depad(...)``; loads the library on first use."""

    def __getattr__(self, name):
        f = getattr(load(), name)
        setattr(self, name, f)
        return f


fn = _Fns()
