/* C ABI of libenergon_linear.so: the projection GEMM either side of the padding-removal path
 * on hipBLASLt.  Separate from energon_hip.h because it is the only piece that links a
 * library besides the HIP runtime.  Device pointers only; nothing is allocated or freed on
 * the device (hipBLASLt scratch comes in through `workspace`); launches go to `stream`. */
#ifndef ENERGON_LINEAR_H_
#define ENERGON_LINEAR_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum en_linear_activation { EN_LINEAR_ACT_NONE = 0, EN_LINEAR_ACT_RELU = 1, EN_LINEAR_ACT_GELU_TANH = 2 };

enum en_linear_status {
  EN_LINEAR_ERR_ARG = -1,
  EN_LINEAR_ERR_DTYPE = -2,
  EN_LINEAR_ERR_HIP = -3,
  EN_LINEAR_ERR_BLAS = -4,
  EN_LINEAR_ERR_NO_ALGO = -5
};

/* y[rows,dout] = act(x[rows,din] * w[dout,din]^T + bias[dout]); bias may be NULL.
 * Replaces mlp_gemm (energonai/kernel/cuda_native/csrc/linear_wrapper.cpp:82-111; Python
 * wrapper cuda_native/linear_func.py:11-32), which has neither bias nor activation: the
 * callers add them as separate ops (energonai/model/mlp.py:30-35).  dtype: 0 fp32, 1 fp16,
 * 2 bf16 (as en_dtype), fp32 accumulation.  `algo` indexes hipBLASLt's ranked candidate
 * list for this problem (-1 = first choice), the counterpart of the reference's cuBLAS
 * algorithm id.  GELU is hipBLASLt's epilogue form (tanh approximation). */
int en_linear(const void *x, const void *w, const void *bias, void *y, int64_t rows, int64_t din, int64_t dout,
              int activation, int dtype, int algo, void *workspace, int64_t workspace_bytes, void *stream);

/* Number of candidates `algo` may index for this problem, or a negative en_linear_status.
 * What find_algo (cuda_native/linear_func.py:35-92) loops over. */
int en_linear_algo_count(int64_t rows, int64_t din, int64_t dout, int has_bias, int activation, int dtype,
                         int64_t workspace_bytes);

const char *en_linear_status_string(int status);

/* Digest of the source files this library was compiled from (set by the build); see en_source_hash. */
const char *en_linear_source_hash(void);

#ifdef __cplusplus
}
#endif

#endif /* ENERGON_LINEAR_H_ */
