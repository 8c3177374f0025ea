"""Same symbol table as the reference's ``energonai_scale_mask`` extension
(csrc/scale_mask_softmax_wrapper.cpp:46-49)."""
from ..kernel.cuda_native import scale_mask_softmax as _k


def scale_mask_softmax_wrapper(batch_size, batch_seq_len, head_num, correlation, real_seq_len):
    return _k.scale_mask_softmax(batch_size, batch_seq_len, head_num, correlation, real_seq_len)
