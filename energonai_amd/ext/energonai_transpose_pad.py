"""Same symbol table as the reference's ``energonai_transpose_pad`` extension
(csrc/transpose_pad_fusion_wrapper.cpp:246-263)."""
import importlib

# the package re-exports a function of the same name, which hides the module from a plain "from ... import"
_k = importlib.import_module("energonai_amd.kernel.cuda_native.transpose_pad")


def transpose_pad_wrapper(src, batch_size, max_seq_len, seq_len_list, head_num, size_per_head):
    return _k.transpose_pad(src, batch_size, max_seq_len, seq_len_list, head_num, size_per_head)


def transpose_depad_wrapper(src, batch_size, sum_seq, max_seq_len, seq_len_list, head_num, size_per_head):
    return _k.transpose_depad(src, batch_size, sum_seq, max_seq_len, seq_len_list, head_num, size_per_head)


def ft_build_padding_offsets_wrapper(sequence_length, batch_size, max_seq_len, valid_word_num, tmp_mask_offset):
    return _k.ft_build_padding_offsets(sequence_length, batch_size, max_seq_len, valid_word_num, tmp_mask_offset)


def ft_remove_padding_wrapper(src, tmp_mask_offset, mask_offset, valid_word_num, hidden_dim):
    return _k.ft_remove_padding(src, tmp_mask_offset, mask_offset, valid_word_num, hidden_dim)


def ft_rebuild_padding_wrapper(src, mask_offset, valid_word_num, hidden_dim, batch_size, max_seq_len):
    return _k.ft_rebuild_padding(src, mask_offset, valid_word_num, hidden_dim, batch_size, max_seq_len)


def ft_transpose_rebuild_padding_wrapper(Q, K, V, q_buf, k_buf, v_buf, batch_size, seq_len, head_num, size_per_head,
                                         valid_word_num, mask_offset):
    return _k.ft_transpose_rebuild_padding(Q, K, V, q_buf, k_buf, v_buf, batch_size, seq_len, head_num,
                                           size_per_head, valid_word_num, mask_offset)


def ft_transpose_remove_padding_wrapper(src, valid_word_num, batch_size, seq_len, head_num, size_per_head,
                                        mask_offset):
    return _k.ft_transpose_remove_padding(src, valid_word_num, batch_size, seq_len, head_num, size_per_head,
                                          mask_offset)
