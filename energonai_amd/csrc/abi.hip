// Library bookkeeping (version, status strings, HIP error record), the prefix
// sum that turns sequence lengths into offsets once per batch, and the plain
// 128-bit copy used as the bandwidth yardstick.
#include "common.hip.h"

namespace en {

static thread_local int g_last_hip_error = 0;

int record_hip_error(hipError_t e) {
  g_last_hip_error = (int)e;
  return EN_ERR_HIP;
}

// ---------------------------------------------------------------------------
// prefix sum over up to 65536 lengths: one workgroup, 256 lanes each summing a
// contiguous chunk, then a scan of the 256 partial sums in LDS.
// ---------------------------------------------------------------------------
template <typename LenT>
__global__ __launch_bounds__(kBlock) void prefix_sum_kernel(const LenT *__restrict__ lens, int batch,
                                                            int32_t *__restrict__ cu, int32_t *__restrict__ lens32) {
  __shared__ int32_t s_part[kBlock];
  const int tid = threadIdx.x;
  const int per = (batch + kBlock - 1) / kBlock;
  const int lo = tid * per;
  const int hi = min(batch, lo + per);
  int32_t sum = 0;
  for (int i = lo; i < hi; ++i) sum += (int32_t)lens[i];
  s_part[tid] = sum;
  __syncthreads();
  // Hillis-Steele inclusive scan over 256 partials
  for (int off = 1; off < kBlock; off <<= 1) {
    int32_t v = (tid >= off) ? s_part[tid - off] : 0;
    __syncthreads();
    s_part[tid] += v;
    __syncthreads();
  }
  int32_t run = (tid == 0) ? 0 : s_part[tid - 1];
  for (int i = lo; i < hi; ++i) {
    const int32_t n = (int32_t)lens[i];
    cu[i] = run;
    if (lens32) lens32[i] = n;
    run += n;
  }
  if (tid == kBlock - 1) cu[batch] = s_part[kBlock - 1];
}

// ---------------------------------------------------------------------------
// plain copy: each lane moves 4 x 16 bytes per iteration, grid-stride.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                      int64_t nvec) {
  constexpr int U = 4;
  const int64_t stride = (int64_t)gridDim.x * kBlock * U;
  for (int64_t base = ((int64_t)blockIdx.x * U) * kBlock + threadIdx.x; base < nvec; base += stride) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + (int64_t)u * kBlock;
      if (i < nvec) v[u] = src[i];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + (int64_t)u * kBlock;
      if (i < nvec) dst[i] = v[u];
    }
  }
}

}  // namespace en

extern "C" {

int en_version(void) { return 300; }

#ifndef EN_SOURCE_HASH
#define EN_SOURCE_HASH "unknown"
#endif
const char *en_source_hash(void) { return EN_SOURCE_HASH; }

const char *en_status_string(int status) {
  switch (status) {
    case EN_OK: return "ok";
    case EN_ERR_NULL: return "a required pointer is NULL";
    case EN_ERR_SHAPE: return "an extent is out of range for this entry point";
    case EN_ERR_DTYPE: return "dtype or element size not supported by this entry point";
    case EN_ERR_ALIGN: return "pointer or stride not aligned to the element size";
    case EN_ERR_UNSUPPORTED: return "no kernel in this build for the requested shape";
    case EN_ERR_HIP: return "HIP runtime error (see en_last_hip_error_string)";
    case EN_ERR_SCRATCH: return "the call needs more than the library's static scratch array holds (EN_LAYER_SCRATCH_BYTES)";
    default: return "unknown status";
  }
}

int en_last_hip_error(void) { return en::g_last_hip_error; }

const char *en_last_hip_error_string(void) { return hipGetErrorString((hipError_t)en::g_last_hip_error); }

int en_prefix_sum(const void *seq_lens, int lens_are_i64, int batch, int32_t *cu_seqlens, int32_t *lens32_out,
                  en_stream_t stream) {
  if (!seq_lens || !cu_seqlens) return EN_ERR_NULL;
  if (batch < 1 || batch > 65536) return EN_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (lens_are_i64)
    en::prefix_sum_kernel<int64_t><<<1, en::kBlock, 0, s>>>((const int64_t *)seq_lens, batch, cu_seqlens, lens32_out);
  else
    en::prefix_sum_kernel<int32_t><<<1, en::kBlock, 0, s>>>((const int32_t *)seq_lens, batch, cu_seqlens, lens32_out);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_copy_bytes(const void *src, void *dst, int64_t nbytes, en_stream_t stream) {
  if (!src || !dst) return EN_ERR_NULL;
  if (nbytes < 0 || (nbytes % 16) != 0) return EN_ERR_SHAPE;
  if (!en::aligned_to(src, 16) || !en::aligned_to(dst, 16)) return EN_ERR_ALIGN;
  if (nbytes == 0) return EN_OK;
  const int64_t nvec = nbytes / 16;
  const int64_t want = en::ceil_div(nvec, (int64_t)en::kBlock * 4);
  const int grid = (int)(want < 256 * 16 ? want : 256 * 16);
  en::copy_kernel<<<grid, en::kBlock, 0, (hipStream_t)stream>>>((const uint4 *)src, (uint4 *)dst, nvec);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // extern "C"
