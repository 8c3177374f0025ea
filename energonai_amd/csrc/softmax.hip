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

#ifndef EN_SOFTMAX_LPR_A
#define EN_SOFTMAX_LPR_A 16  // lanes per row for rows of 33..128 vectors
#endif

namespace en {

struct SoftmaxArgs {
  void *src;
  const int32_t *k_lens;
  const int32_t *q_lens;
  int B, H, Sq, Sk;
  float scale;
  int causal;
  int tail_shift; // < 0: zero the whole tail of a row; s: only up to the extent of its 2^s-row query tile
  int rows_per_batch;  // H * Sq
  float inv_sq;        // 1 / Sq
};

__device__ __forceinline__ int visible_keys(int q, int ql, int kl, int Sk, int causal) {
  int n = causal ? min(kl, q + (kl - ql) + 1) : kl;
  n = max(n, 0);
  return min(n, Sk);
}

// Per-row geometry: n visible keys, lim = one past the last element to write.
struct RowInfo {
  bool active;
  int n, lim;
};

// r % d for 0 <= r < 2^24 without an integer division: float quotient, one correction step.
__device__ __forceinline__ int small_mod(int r, int d, float inv_d) {
  int q = (int)((float)r * inv_d);
  int m = r - q * d;
  if (m < 0) m += d;
  if (m >= d) m -= d;
  return m;
}

// r = row index inside batch b (head-major: r = h * Sq + q); kl/ql are the batch's lengths.
__device__ __forceinline__ RowInfo row_info(const SoftmaxArgs &a, int r, int kl, int ql) {
  RowInfo ri{false, 0, 0};
  if (r >= a.rows_per_batch) return ri;
  const int q = small_mod(r, a.Sq, a.inv_sq);
  if (q >= ql) return ri;
  ri.active = true;
  ri.n = visible_keys(q, ql, kl, a.Sk, a.causal);
  ri.lim = a.Sk;
  if (a.tail_shift >= 0) {  // the consumer reads a row only up to what the last row of its query tile sees
    const int q_last = min(((q >> a.tail_shift) + 1) << a.tail_shift, ql) - 1;
    ri.lim = visible_keys(q_last, ql, kl, a.Sk, a.causal);
  }
  return ri;
}

// One wave per workgroup: rows differ in length, and a wave that is done frees its slot at once instead of
// waiting for the longest row among four waves (c3, tile-bounded form: 214 us with 256 threads, 163 us with 64).
constexpr int kRowsBlock = kWave;

// LPR lanes share a row, each lane holds VPL vectors of it, and every lane
// group works on R consecutive rows at once: all R*VPL loads are issued before
// the first reduction, so one wave keeps R rows of traffic in flight and the
// R independent reduction chains interleave.
template <int DT, int VPL, int LPR, int R>
__global__ __launch_bounds__(kRowsBlock) void softmax_rows_kernel(SoftmaxArgs a) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  constexpr int EPV = 16 / E::kSize;          // elements per 128-bit vector
  constexpr int GROUPS_PER_WAVE = kWave / LPR;
  constexpr int GROUPS_PER_BLOCK = GROUPS_PER_WAVE * (kRowsBlock / kWave);

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int sub = lane / LPR;
  const int l = lane % LPR;
  const int b = blockIdx.y;
  const int kl = a.k_lens[b];
  const int ql = min(a.q_lens ? a.q_lens[b] : min(kl, a.Sq), a.Sq);
  const int row0 = (blockIdx.x * GROUPS_PER_BLOCK + wave * GROUPS_PER_WAVE + sub) * R;  // inside the batch

  RowInfo ri[R];
  bool any = false;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    ri[i] = row_info(a, row0 + i, kl, ql);
    any |= ri[i].active;
  }
  if (__ballot(any) == 0ull) return;  // whole wave has nothing to do

  T *base = reinterpret_cast<T *>(a.src) + (int64_t)b * a.rows_per_batch * a.Sk;
  uint4 raw[R][VPL];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const T *rowp = base + (int64_t)(row0 + i) * a.Sk;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e0 = (l + LPR * j) * EPV;
      raw[i][j] = make_uint4(E::kNegInfWord, E::kNegInfWord, E::kNegInfWord, E::kNegInfWord);   // not visible: -inf
      if (ri[i].active && e0 < ri[i].n) raw[i][j] = load16<false>(rowp + e0);
    }
  }

  constexpr float kLog2e = 1.4426950408889634f;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = ri[i].n;
    // A vector step is skipped when no lane of the wave holds a visible key in it (one scalar branch); in a
    // step that runs, vectors past a row's prefix hold -inf from the load above and need no masking, so only
    // the one vector of a row that straddles the end of the prefix is masked element by element.  -inf stays
    // -inf through the scaling (the scale is positive) and exp2 turns it into the zero it must become.
    float x[VPL][EPV];
    bool any[VPL];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e0 = (l + LPR * j) * EPV;
      any[j] = __builtin_amdgcn_ballot_w64(e0 < n) != 0ull;
      if (any[j]) {
        const Pack<T, EPV> pk = __builtin_bit_cast(Pack<T, EPV>, raw[i][j]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) x[j][e] = E::to_float(pk.v[e]);
        const int nv = n - e0;                      // visible elements of this vector
        if (nv > 0 && nv < EPV) {
#pragma unroll
          for (int e = 1; e < EPV; ++e)
            if (e >= nv) x[j][e] = -INFINITY;
        }
#pragma unroll
        for (int e = 0; e < EPV; ++e) m = fmaxf(m, x[j][e]);
      }
    }
    m = group_allreduce<OpMax, LPR>(m);
    // exp(scale * (x - m)) = exp2(x * c - m * c), c = scale * log2(e) > 0 (other scales take the generic kernel)
    const float c = a.scale * kLog2e;
    const float moff = (m == -INFINITY) ? 0.f : -m * c;  // nothing visible: all zeros, no NaN
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      if (any[j]) {
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          const float ex = __builtin_amdgcn_exp2f(fmaf(x[j][e], c, moff));
          x[j][e] = ex;
          s += ex;
        }
      }
    }
    s = group_allreduce<OpSum, LPR>(s);
    const float inv = s > 0.f ? 1.0f / s : 0.f;
    T *rowp = base + (int64_t)(row0 + i) * a.Sk;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e0 = (l + LPR * j) * EPV;
      uint4 out = make_uint4(0u, 0u, 0u, 0u);
      if (any[j]) {                                 // masked elements are exact zeros by now
        Pack<T, EPV> pk;
#pragma unroll
        for (int e = 0; e < EPV; ++e) pk.v[e] = E::from_float(x[j][e] * inv);
        out = __builtin_bit_cast(uint4, pk);
      }
      if (ri[i].active && e0 < ri[i].lim) store16<false>(rowp + e0, out);
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
  const int b = blockIdx.y;
  const int kl = a.k_lens[b];
  const int ql = min(a.q_lens ? a.q_lens[b] : min(kl, a.Sq), a.Sq);
  const RowInfo ri = row_info(a, (int)blockIdx.x, kl, ql);
  if (!ri.active) return;
  const int n = ri.n;
  T *rowp = reinterpret_cast<T *>(a.src) + ((int64_t)b * a.rows_per_batch + blockIdx.x) * a.Sk;
  float m = -INFINITY;
  for (int i = threadIdx.x; i < n; i += kBlock) m = fmaxf(m, E::to_float(rowp[i]) * a.scale);
  m = block_allreduce<OpMax, kBlock / kWave>(m, s_max);
  const float msafe = (m == -INFINITY) ? 0.f : m;
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += kBlock) s += __expf(E::to_float(rowp[i]) * a.scale - msafe);
  s = block_allreduce<OpSum, kBlock / kWave>(s, s_sum);
  const float inv = s > 0.f ? 1.0f / s : 0.f;
  // The contraction that wrote the scores stored whole 16-byte vectors, and the one that reads the probabilities
  // loads whole vectors as far as the row can see, with no mask inside a vector: like the register kernel, clear
  // the vector that straddles the end of what is written, or its raw scores would be multiplied with real V rows.
  constexpr int EPV = 16 / E::kSize;
  const int lim = min((ri.lim + EPV - 1) / EPV * EPV, a.Sk);
  for (int i = threadIdx.x; i < lim; i += kBlock) {
    const float p = (i < n) ? __expf(E::to_float(rowp[i]) * a.scale - msafe) * inv : 0.f;
    rowp[i] = E::from_float(p);
  }
}

template <int DT, int VPL, int LPR, int R>
static void launch_rows(const SoftmaxArgs &a, hipStream_t s) {
  constexpr int ROWS_PER_BLOCK = (kWave / LPR) * (kRowsBlock / kWave) * R;
  const dim3 grid((unsigned)ceil_div(a.rows_per_batch, ROWS_PER_BLOCK), (unsigned)a.B, 1);
  softmax_rows_kernel<DT, VPL, LPR, R><<<grid, kRowsBlock, 0, s>>>(a);
}

template <int DT>
static int dispatch(const SoftmaxArgs &a, hipStream_t s) {
  constexpr int EPV = 16 / Elem<DT>::kSize;
  const bool vec_ok = (a.Sk % EPV) == 0 && aligned_to(a.src, 16);
  const int64_t nvec = vec_ok ? a.Sk / EPV : 0;
  if (!vec_ok || nvec > 64 * 16 || !(a.scale > 0.f)) {
    softmax_generic_kernel<DT><<<dim3((unsigned)a.rows_per_batch, (unsigned)a.B, 1), kBlock, 0, s>>>(a);
  }
  // Few lanes per row for short rows: a causal row uses on average half of its sequence, so narrow
  // lane groups keep more lanes busy and a wave skips the vector steps none of its rows reach.
  else if (nvec <= 8) launch_rows<DT, 1, 8, 1>(a, s);
  else if (nvec <= 16) launch_rows<DT, 1, 16, 1>(a, s);
  else if (nvec <= 32) launch_rows<DT, 2, 16, 1>(a, s);
  else if (nvec <= 64) launch_rows<DT, 4, EN_SOFTMAX_LPR_A, 1>(a, s);
  else if (nvec <= 128) launch_rows<DT, 8, EN_SOFTMAX_LPR_A, 1>(a, s);
  else if (nvec <= 256) launch_rows<DT, 4, 64, 1>(a, s);
  else if (nvec <= 512) launch_rows<DT, 8, 64, 1>(a, s);
  else launch_rows<DT, 16, 64, 1>(a, s);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // namespace en

extern "C" int en_scale_mask_softmax(void *src, const int32_t *k_lens, const int32_t *q_lens, int batch, int head_num,
                                     int q_seq_len, int k_seq_len, float scale, int causal, int tail_rows,
                                     int dtype, en_stream_t stream) {
  using namespace en;
  if (!src || !k_lens) return EN_ERR_NULL;
  if (batch < 1 || head_num < 1 || q_seq_len < 1 || k_seq_len < 1 || tail_rows < 0) return EN_ERR_SHAPE;
  if (tail_rows & (tail_rows - 1)) return EN_ERR_SHAPE;  // query tile must be a power of two
  int tail_shift = -1;
  for (int t = tail_rows; t > 0; t >>= 1) ++tail_shift;
  const int es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  if (!aligned_to(src, es)) return EN_ERR_ALIGN;
  if (batch > 65535 || (int64_t)head_num * q_seq_len >= (1 << 24)) return EN_ERR_SHAPE;
  SoftmaxArgs a{src, k_lens, q_lens, batch, head_num, q_seq_len, k_seq_len, scale, causal ? 1 : 0, tail_shift,
                head_num * q_seq_len, 1.0f / (float)q_seq_len};
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return dispatch<EN_F32>(a, s);
    case EN_F16: return dispatch<EN_F16>(a, s);
    default: return dispatch<EN_BF16>(a, s);
  }
}
