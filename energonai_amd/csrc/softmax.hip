// scale + mask + softmax over the rows of a [B,H,Sq,Sk] score tensor, in place.
//
// Single pass: a row is read once into VGPRs (128-bit loads, only the visible
// prefix is fetched), max and sum are reduced across the lanes that share the
// row with DPP row operations, and the whole row (probabilities, then the zero
// tail) is written back once.  LPR lanes share a row (8..64, so short rows do
// not idle most of a wave) and each lane holds VPL vectors of it.  Rows of
// padded queries exit without touching memory.  Rows too long for registers,
// or not 16-byte aligned, take the three-pass workgroup-per-row kernel.
#include "common.hip.h"

#include <math.h>

namespace en {

struct SoftmaxArgs {
  void *src;
  const int32_t *k_lens;
  const int32_t *q_lens;
  int B, H, Sq, Sk;
  float scale;
  int causal;
  int64_t nrows;
};

__device__ __forceinline__ int visible_keys(int q, int ql, int kl, int Sk, int causal) {
  int n = causal ? min(kl, q + (kl - ql) + 1) : kl;
  n = max(n, 0);
  return min(n, Sk);
}

template <int DT, int VPL, int LPR>
__global__ __launch_bounds__(kBlock) void softmax_rows_kernel(SoftmaxArgs a) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  constexpr int EPV = 16 / E::kSize;          // elements per 128-bit vector
  constexpr int ROWS_PER_WAVE = kWave / LPR;
  constexpr int ROWS_PER_BLOCK = ROWS_PER_WAVE * (kBlock / kWave);

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int sub = lane / LPR;
  const int l = lane % LPR;
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + wave * ROWS_PER_WAVE + sub;

  bool active = row < a.nrows;
  int n = 0;
  if (active) {
    const int q = (int)(row % a.Sq);
    const int b = (int)((row / a.Sq) / a.H);
    const int kl = a.k_lens[b];
    const int ql = a.q_lens ? a.q_lens[b] : min(kl, a.Sq);
    active = q < ql;
    n = visible_keys(q, ql, kl, a.Sk, a.causal);
  }
  if (__ballot(active) == 0ull) return;  // whole wave has nothing to do

  T *rowp = reinterpret_cast<T *>(a.src) + row * a.Sk;
  float x[VPL][EPV];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e0 = (l + LPR * j) * EPV;
    if (active && e0 < n) {
      const Pack<T, EPV> pk = load_pack<T, EPV>(rowp + e0);
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float v = (e0 + e < n) ? E::to_float(pk.v[e]) * a.scale : -INFINITY;
        x[j][e] = v;
        m = fmaxf(m, v);
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[j][e] = -INFINITY;
    }
  }
  m = group_allreduce<OpMax, LPR>(m);
  const float msafe = (m == -INFINITY) ? 0.f : m;  // nothing visible: all zeros, no NaN
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j)
#pragma unroll
    for (int e = 0; e < EPV; ++e) {
      const float ex = __expf(x[j][e] - msafe);
      x[j][e] = ex;
      s += ex;
    }
  s = group_allreduce<OpSum, LPR>(s);
  const float inv = s > 0.f ? 1.0f / s : 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e0 = (l + LPR * j) * EPV;
    if (active && e0 < a.Sk) {
      Pack<T, EPV> pk;
#pragma unroll
      for (int e = 0; e < EPV; ++e) pk.v[e] = E::from_float(x[j][e] * inv);
      store_pack<T, EPV>(rowp + e0, pk);
    }
  }
}

// Any Sk, any alignment: one workgroup per row, three strided passes.
template <int DT>
__global__ __launch_bounds__(kBlock) void softmax_generic_kernel(SoftmaxArgs a) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  __shared__ float s_max[kBlock / kWave];
  __shared__ float s_sum[kBlock / kWave];
  const int64_t row = blockIdx.x;
  const int q = (int)(row % a.Sq);
  const int b = (int)((row / a.Sq) / a.H);
  const int kl = a.k_lens[b];
  const int ql = a.q_lens ? a.q_lens[b] : min(kl, a.Sq);
  if (q >= ql) return;
  const int n = visible_keys(q, ql, kl, a.Sk, a.causal);
  T *rowp = reinterpret_cast<T *>(a.src) + row * a.Sk;
  float m = -INFINITY;
  for (int i = threadIdx.x; i < n; i += kBlock) m = fmaxf(m, E::to_float(rowp[i]) * a.scale);
  m = block_allreduce<OpMax, kBlock / kWave>(m, s_max);
  const float msafe = (m == -INFINITY) ? 0.f : m;
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += kBlock) s += __expf(E::to_float(rowp[i]) * a.scale - msafe);
  s = block_allreduce<OpSum, kBlock / kWave>(s, s_sum);
  const float inv = s > 0.f ? 1.0f / s : 0.f;
  for (int i = threadIdx.x; i < a.Sk; i += kBlock) {
    const float p = (i < n) ? __expf(E::to_float(rowp[i]) * a.scale - msafe) * inv : 0.f;
    rowp[i] = E::from_float(p);
  }
}

template <int DT, int VPL, int LPR>
static void launch_rows(const SoftmaxArgs &a, hipStream_t s) {
  constexpr int ROWS_PER_BLOCK = (kWave / LPR) * (kBlock / kWave);
  const int64_t blocks = ceil_div(a.nrows, ROWS_PER_BLOCK);
  softmax_rows_kernel<DT, VPL, LPR><<<(unsigned)blocks, kBlock, 0, s>>>(a);
}

template <int DT>
static int dispatch(const SoftmaxArgs &a, hipStream_t s) {
  constexpr int EPV = 16 / Elem<DT>::kSize;
  const bool vec_ok = (a.Sk % EPV) == 0 && aligned_to(a.src, 16);
  const int64_t nvec = vec_ok ? a.Sk / EPV : 0;
  if (a.nrows > (int64_t)INT32_MAX) return EN_ERR_SHAPE;
  if (!vec_ok || nvec > 64 * 16) {
    softmax_generic_kernel<DT><<<(unsigned)a.nrows, kBlock, 0, s>>>(a);
  } else if (nvec <= 8) launch_rows<DT, 1, 8>(a, s);
  else if (nvec <= 16) launch_rows<DT, 1, 16>(a, s);
  else if (nvec <= 32) launch_rows<DT, 1, 32>(a, s);
  else if (nvec <= 64) launch_rows<DT, 1, 64>(a, s);
  else if (nvec <= 128) launch_rows<DT, 2, 64>(a, s);
  else if (nvec <= 256) launch_rows<DT, 4, 64>(a, s);
  else if (nvec <= 512) launch_rows<DT, 8, 64>(a, s);
  else launch_rows<DT, 16, 64>(a, s);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // namespace en

extern "C" int en_scale_mask_softmax(void *src, const int32_t *k_lens, const int32_t *q_lens, int batch, int head_num,
                                     int q_seq_len, int k_seq_len, float scale, int causal, int dtype,
                                     en_stream_t stream) {
  using namespace en;
  if (!src || !k_lens) return EN_ERR_NULL;
  if (batch < 1 || head_num < 1 || q_seq_len < 1 || k_seq_len < 1) return EN_ERR_SHAPE;
  const int es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  if (!aligned_to(src, es)) return EN_ERR_ALIGN;
  SoftmaxArgs a{src, k_lens, q_lens, batch, head_num, q_seq_len, k_seq_len, scale, causal ? 1 : 0,
                (int64_t)batch * head_num * q_seq_len};
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return dispatch<EN_F32>(a, s);
    case EN_F16: return dispatch<EN_F16>(a, s);
    default: return dispatch<EN_BF16>(a, s);
  }
}
