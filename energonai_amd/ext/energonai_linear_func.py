"""Same symbol table as the reference's ``energonai_linear_func`` extension
(csrc/linear_wrapper.cpp:133-140), on the hipBLASLt front end.  The reference's
algorithm ids are cuBLAS constants (-1..23 and 99..115); here the two ranges
collapse onto hipBLASLt's candidate list for the problem, so any id outside it
falls back to the first candidate."""
from ..kernel.cuda_native import linear_func as _lf


def mlp_gemm(tensor1, tensor2, algo=-1):
    return _lf.linear(tensor1, tensor2, algo)


def get_start_algo():
    return -1


def get_end_algo():
    return 23


def get_start_algo_t_op():
    return 99


def get_end_algo_t_op():
    return 115
