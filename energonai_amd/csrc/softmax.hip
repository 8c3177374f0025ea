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
  int tail_shift; // < 0: zero the whole tail of a row; s: only up to the extent of its 2^s-row query tile
  int rows_per_batch;  // H * Sq
  float inv_sq;        // 1 / Sq
  int packed;          // rows are the packed causal prefixes of common.hip.h instead of Sk elements apart
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
// a score tensor at least this large is read and written with the non-temporal policy (1.9 GB of scores, 1024-key
// rows: 157 -> 146 us; on tensors that fit the 256 MB memory-side cache the policy costs time)
constexpr int64_t kStreamSoftmaxBytes = 512ll << 20;

// The work of one lane group: LPR lanes share a row, each lane holds VPL vectors of it, and the group works on
// R rows at once: all R*VPL loads are issued before the first reduction, so one wave keeps R rows of traffic in
// flight and the R independent reduction chains interleave.  rowp[i] is row i's first element, ri[i] its
// geometry, l the lane's index inside its group.  Rows whose write extent lies past the LPR*VPL vectors the
// registers hold get the rest of their zero tail from a store loop (TAIL_LOOP).
template <int DT, int VPL, int LPR, int R, bool STREAM, bool TAIL_LOOP>
__device__ __forceinline__ void softmax_lane_group(const SoftmaxArgs &a, typename Elem<DT>::T *const (&rowp)[R],
                                                   const RowInfo (&ri)[R], int l) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  constexpr int EPV = 16 / E::kSize;          // elements per 128-bit vector
  uint4 raw[R][VPL];
#pragma unroll
  for (int i = 0; i < R; ++i) {
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e0 = (l + LPR * j) * EPV;
      raw[i][j] = make_uint4(E::kNegInfWord, E::kNegInfWord, E::kNegInfWord, E::kNegInfWord);   // not visible: -inf
      if (ri[i].active && e0 < ri[i].n) raw[i][j] = load16<STREAM>(rowp[i] + e0);
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
      any[j] = __builtin_amdgcn_ballot_w64(ri[i].active && e0 < n) != 0ull;
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
      if (ri[i].active && e0 < ri[i].lim) store16<STREAM>(rowp[i] + e0, out);
    }
    if (TAIL_LOOP && ri[i].active) {
      for (int e0 = (l + LPR * VPL) * EPV; e0 < ri[i].lim; e0 += LPR * EPV)
        store16<STREAM>(rowp[i] + e0, make_uint4(0u, 0u, 0u, 0u));
    }
  }
}

// Rows of up to 64 * 16 vectors, one lane-group shape for the whole launch (chosen from the row length Sk).
template <int DT, int VPL, int LPR, int R>
__global__ __launch_bounds__(kRowsBlock) void softmax_rows_kernel(SoftmaxArgs a) {
  typedef typename Elem<DT>::T T;
  constexpr int GROUPS_PER_WAVE = kWave / LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int sub = lane / LPR;
  const int l = lane % LPR;
  const int b = blockIdx.y;
  const int kl = a.k_lens[b];
  const int ql = min(a.q_lens ? a.q_lens[b] : min(kl, a.Sq), a.Sq);
  const int row0 = (blockIdx.x * GROUPS_PER_WAVE + sub) * R;  // inside the batch

  RowInfo ri[R];
  T *rowp[R];
  bool any = false;
  T *base = reinterpret_cast<T *>(a.src) + (int64_t)b * a.rows_per_batch * a.Sk;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    ri[i] = row_info(a, row0 + i, kl, ql);
    rowp[i] = base + (int64_t)(row0 + i) * a.Sk;
    any |= ri[i].active;
  }
  if (__ballot(any) == 0ull) return;  // whole wave has nothing to do
  softmax_lane_group<DT, VPL, LPR, R, false, false>(a, rowp, ri, l);
}

// ---------------------------------------------------------------------------------------------------------
// Rows of up to 256 vectors (2048 16-bit or 1024 fp32 keys): the lane-group shape follows each row, not the
// bucket.  Under a causal mask a row sees from one key to the whole sequence, and sequences are shorter than
// the bucket; with one shape per launch most lanes of most waves hold nothing, and what a wave keeps in
// flight -- which is what hides the memory latency -- shrinks with them.  Here every lane holds four vectors and
// a row is given 4, 8, 16, 32 or 64 lanes by the number of keys it sees, so a wave of 64 lanes works on 16, 8,
// 4, 2 or 1 rows (times R) and moves about the same number of bytes whichever band its rows are in.
//
// The rows of one (batch, head) are cut into bands by what they see; band k holds rows that see more than
// cap(k-1) and at most cap(k) = 4 * 2^k vectors.  Under a causal mask what a row sees grows by one key per row,
// so a band is a range of rows; without one every row of a sequence sees the same keys and all of them fall
// into one band.  A workgroup (one wave) finds its batch's band layout from the two lengths with a few scalar
// operations, then its head, band and first row from its index; workgroups past the batch's count exit.  Bands
// are laid out from the longest rows to the shortest, so the heavy waves start first.
// ---------------------------------------------------------------------------------------------------------
constexpr int kBandVpl = 4;
constexpr int kBands = 5;

struct BandLayout {
  int first[kBands + 1];   // band k holds rows first[k] .. first[k+1]-1 (k = 0: the shortest rows)
  int blocks[kBands];      // workgroups band k needs per head
  int total;               // workgroups per head
};

// cap(k) in elements; the top band takes every longer row as well (rows are at most 256 vectors long here)
template <int EPV> __host__ __device__ constexpr int band_cap(int k) { return kBandVpl * EPV * (4 << k); }

template <int EPV, int R>
__device__ __forceinline__ BandLayout band_layout(const SoftmaxArgs &a, int kl, int ql) {
  BandLayout L;
  L.first[0] = 0;
  L.total = 0;
  const int vis_all = min(max(kl, 0), a.Sk);       // what every row sees without a causal mask
#pragma unroll
  for (int k = 0; k < kBands; ++k) {
    int end;
    if (k == kBands - 1) end = ql;
    else if (a.causal) end = min(max(band_cap<EPV>(k) - (kl - ql), 0), ql);   // row q sees q + (kl - ql) + 1 keys
    else end = vis_all <= band_cap<EPV>(k) ? ql : 0;
    end = max(end, L.first[k]);
    L.first[k + 1] = end;
    const int rows_per_wave = (16 >> k) * R;
    L.blocks[k] = (end - L.first[k] + rows_per_wave - 1) / rows_per_wave;
    L.total += L.blocks[k];
  }
  return L;
}

template <int DT, int K, int R, bool STREAM>
__device__ __forceinline__ void softmax_band_wave(const SoftmaxArgs &a, typename Elem<DT>::T *unit, int q0, int q_end,
                                                  int kl, int ql, int lane) {
  typedef typename Elem<DT>::T T;
  constexpr int LPR = 4 << K;
  const int sub = lane / LPR, l = lane % LPR;
  RowInfo ri[R];
  T *rowp[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int q = q0 + sub * R + i;
    ri[i] = RowInfo{false, 0, 0};
    constexpr int EPV = 16 / Elem<DT>::kSize;
    if (q < q_end) {
      ri[i].active = true;
      ri[i].n = visible_keys(q, ql, kl, a.Sk, a.causal);
      ri[i].lim = a.Sk;
      if (a.packed) {           // the row's slot ends with the vector that holds its last visible key
        ri[i].lim = (q / EPV + 1) * EPV;
      } else if (a.tail_shift >= 0) {  // the consumer reads a row only up to what the last row of its query tile sees
        const int q_last = min(((q >> a.tail_shift) + 1) << a.tail_shift, ql) - 1;
        ri[i].lim = visible_keys(q_last, ql, kl, a.Sk, a.causal);
      }
    }
    rowp[i] = unit + (a.packed ? packed_row_start<EPV * kPackedRowVectors>(q) : (int64_t)q * a.Sk);
  }
  softmax_lane_group<DT, kBandVpl, LPR, R, STREAM, true>(a, rowp, ri, l);
}

template <int DT, int R, bool STREAM>
__global__ __launch_bounds__(kWave) void softmax_bands_kernel(SoftmaxArgs a) {
  typedef typename Elem<DT>::T T;
  constexpr int EPV = 16 / Elem<DT>::kSize;
  // grid (workgroups per head, heads, batches): the workgroups a shorter sequence does not need are spread over
  // the heads, a few hundred at a time, instead of forming one long run of empty workgroups per batch, during
  // which the machine would drain
  const int b = blockIdx.z, h = blockIdx.y;
  int i = blockIdx.x;
  const int kl = min(a.k_lens[b], a.Sk);           // a key length past the row length means the whole row
  const int ql = min(a.q_lens ? a.q_lens[b] : min(kl, a.Sq), a.Sq);
  if (ql <= 0) return;
  const BandLayout L = band_layout<EPV, R>(a, kl, ql);
  if (i >= L.total) return;
  T *unit = reinterpret_cast<T *>(a.src) +
            ((int64_t)b * a.H + h) * (a.packed ? packed_row_start<EPV * kPackedRowVectors>(a.Sq) : (int64_t)a.Sq * a.Sk);
  const int lane = threadIdx.x;
  // longest rows first
  if (i < L.blocks[4]) return softmax_band_wave<DT, 4, R, STREAM>(a, unit, L.first[4] + i * 1 * R, L.first[5], kl, ql, lane);
  i -= L.blocks[4];
  if (i < L.blocks[3]) return softmax_band_wave<DT, 3, R, STREAM>(a, unit, L.first[3] + i * 2 * R, L.first[4], kl, ql, lane);
  i -= L.blocks[3];
  if (i < L.blocks[2]) return softmax_band_wave<DT, 2, R, STREAM>(a, unit, L.first[2] + i * 4 * R, L.first[3], kl, ql, lane);
  i -= L.blocks[2];
  if (i < L.blocks[1]) return softmax_band_wave<DT, 1, R, STREAM>(a, unit, L.first[1] + i * 8 * R, L.first[2], kl, ql, lane);
  i -= L.blocks[1];
  softmax_band_wave<DT, 0, R, STREAM>(a, unit, L.first[0] + i * 16 * R, L.first[1], kl, ql, lane);
}

// Upper bound, over all lengths a batch may have, of the workgroups one head needs (host side of band_layout).
template <int EPV, int R>
static int band_blocks_bound(const SoftmaxArgs &a, bool square_self_attention) {
  auto rows_per_wave = [](int k) { return (16 >> k) * R; };
  if (!a.causal) {
    // all rows of a sequence share one band; the widest band the row length allows needs the most workgroups
    int k = 0;
    while (k < kBands - 1 && band_cap<EPV>(k) < a.Sk) ++k;
    return (int)ceil_div(a.Sq, rows_per_wave(k));
  }
  if (square_self_attention) {
    // row q sees q + 1 keys: band k holds the rows cap(k-1) .. cap(k)-1, the top band whatever is left
    int total = 0, prev_cap = 0;
    for (int k = 0; k < kBands; ++k) {
      const int hi = (k == kBands - 1 || band_cap<EPV>(k) > a.Sq) ? a.Sq : band_cap<EPV>(k);
      if (hi > prev_cap) total += (int)ceil_div(hi - prev_cap, rows_per_wave(k));
      prev_cap = hi > prev_cap ? hi : prev_cap;
    }
    return total;
  }
  // Any shift between query and key positions (chunked prefill, decode): the Sq rows may fall into the bands in
  // many ways.  Each band takes at most its span of rows (the two outer ones are open-ended), rows in a higher band
  // need more workgroups, and every band that holds rows at all may end with a partly filled workgroup.
  int left = a.Sq;
  double blocks = 0.0;          // the most whole-and-fractional workgroups any split of the rows can need
  for (int k = kBands - 1; k >= 0 && left > 0; --k) {
    const int span = (k == 0 || k == kBands - 1) ? a.Sq : band_cap<EPV>(k) - band_cap<EPV>(k - 1);
    const int rows = span < left ? span : left;
    blocks += (double)rows / rows_per_wave(k);
    left -= rows;
  }
  const int bands_with_rows = a.Sq < kBands ? a.Sq : kBands;      // no more bands hold rows than there are rows
  return (int)(blocks + 0.999999) + bands_with_rows - 1;
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
  constexpr int ROWS_PER_BLOCK = (kWave / LPR) * R;
  const dim3 grid((unsigned)ceil_div(a.rows_per_batch, ROWS_PER_BLOCK), (unsigned)a.B, 1);
  softmax_rows_kernel<DT, VPL, LPR, R><<<grid, kRowsBlock, 0, s>>>(a);
}

template <int DT>
static int launch_bands(const SoftmaxArgs &a, hipStream_t s) {
  constexpr int EPV = 16 / Elem<DT>::kSize;
  constexpr int R = 1;   // rows per lane group; two at once were slower on every workload measured
  const bool square = a.q_lens == nullptr && a.Sq == a.Sk;      // q_len = k_len <= Sk: row q sees q + 1 keys
  const int64_t blocks = band_blocks_bound<EPV, R>(a, square);
  if (a.H > 65535 || a.B > 65535) return EN_ERR_SHAPE;
  const dim3 grid((unsigned)blocks, (unsigned)a.H, (unsigned)a.B);
  if (blocks > INT32_MAX) return EN_ERR_SHAPE;
  // a tensor too large to stay in the memory-side cache is read and written with the non-temporal policy
  const bool stream = (int64_t)a.B * a.rows_per_batch * a.Sk * Elem<DT>::kSize / (a.packed ? 2 : 1) >= kStreamSoftmaxBytes;
  if (stream) softmax_bands_kernel<DT, R, true><<<grid, kWave, 0, s>>>(a);
  else softmax_bands_kernel<DT, R, false><<<grid, kWave, 0, s>>>(a);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

template <int DT>
static int dispatch(const SoftmaxArgs &a, hipStream_t s) {
  constexpr int EPV = 16 / Elem<DT>::kSize;
  const bool vec_ok = (a.Sk % EPV) == 0 && aligned_to(a.src, 16);
  const int64_t nvec = vec_ok ? a.Sk / EPV : 0;
  if (!vec_ok || nvec > 64 * 16 || !(a.scale > 0.f)) {
    softmax_generic_kernel<DT><<<dim3((unsigned)a.rows_per_batch, (unsigned)a.B, 1), kBlock, 0, s>>>(a);
  }
  // Rows of up to 128 vectors (1024 16-bit keys): lane groups sized by what each row sees.  Measured against one
  // shape per launch: 512-key rows 18.7 -> 16.3 us, 1024-key rows 160 -> 142 us; with 2048-key rows the banded form
  // is slower (144 -> 183 us: two 512-byte pieces per instruction, a row pitch apart, instead of one 1024-byte piece),
  // so those keep 64 lanes per row.
  else if (nvec <= 128) return launch_bands<DT>(a, s);
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
                head_num * q_seq_len, 1.0f / (float)q_seq_len, 0};
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return dispatch<EN_F32>(a, s);
    case EN_F16: return dispatch<EN_F16>(a, s);
    default: return dispatch<EN_BF16>(a, s);
  }
}

extern "C" int64_t en_packed_scores_elems(int batch, int head_num, int seq_len, int dtype) {
  using namespace en;
  const int es = dtype_size(dtype);
  if (!es || batch < 1 || head_num < 1 || seq_len < 1) return 0;
  const int64_t unit = es == 4 ? packed_row_start<4 * kPackedRowVectors>(seq_len) : packed_row_start<8 * kPackedRowVectors>(seq_len);
  return (int64_t)batch * head_num * unit;
}

extern "C" int en_scale_mask_softmax_packed(void *scores, const int32_t *seq_lens, int batch, int head_num, int seq_len,
                                            float scale, int dtype, en_stream_t stream) {
  using namespace en;
  if (!scores || !seq_lens) return EN_ERR_NULL;
  if (batch < 1 || batch > 65535 || head_num < 1 || head_num > 65535 || seq_len < 1) return EN_ERR_SHAPE;
  const int es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  if (!aligned_to(scores, 16)) return EN_ERR_ALIGN;
  if (!(scale > 0.f)) return EN_ERR_UNSUPPORTED;
  const int epv = 16 / es;
  if (seq_len > kBandVpl * 64 * epv) return EN_ERR_UNSUPPORTED;     // rows of up to 256 vectors
  SoftmaxArgs a{scores, seq_lens, nullptr, batch, head_num, seq_len, seq_len, scale, 1, 0,
                head_num * seq_len, 1.0f / (float)seq_len, 1};
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return launch_bands<EN_F32>(a, s);
    case EN_F16: return launch_bands<EN_F16>(a, s);
    default: return launch_bands<EN_BF16>(a, s);
  }
}
