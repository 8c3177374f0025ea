"""Same symbol table as the reference's ``energonai_scale_mask`` extension
(csrc/scale_mask_softmax_wrapper.cpp:46-49)."""
import importlib

# the package re-exports a function of the same name, which hides the module from a plain "from ... import"
_k = importlib.import_module("energonai_amd.kernel.cuda_native.scale_mask_softmax")


def scale_mask_softmax_wrapper(batch_size, batch_seq_len, head_num, correlation, real_seq_len):
    return _k.scale_mask_softmax(batch_size, batch_seq_len, head_num, correlation, real_seq_len)
