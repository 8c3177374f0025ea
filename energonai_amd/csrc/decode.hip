// Single-query attention contractions for cached decode: one new token per
// sequence against a ragged K/V cache.  Both are matrix-vector products whose
// cost is the K (or V) bytes streamed from HBM, so they are written as
// streaming reductions with 128-bit loads, one workgroup per (batch, head):
// LPK lanes cover one cached row of D elements, 256/LPK rows are in flight per
// step, four steps are unrolled so each lane keeps 64 bytes outstanding.
#include "common.hip.h"

namespace en {

struct DecodeArgs {
  const void *x;    // q [B,H,D] (QK) or p [B,H,Smax] (PV)
  const void *kv;   // cache [B,H,Smax,D], strided
  void *out;        // scores [B,H,Smax] (QK) or ctx [B,H,D] (PV)
  const int32_t *kv_lens;
  int H, Sk, D;
  int64_t sb, sh, ss;
  float alpha;
  int stream;       // the cache is too large to stay in the memory-side cache: read it with non-temporal loads
};

// A cache that cannot stay in the 256 MB memory-side cache between steps is streamed with
// non-temporal loads (measured on a 2.4 GB cache: QK 5.1 -> 5.8 TB/s, PV 5.6 -> 6.3 TB/s).
constexpr int64_t kStreamCacheBytes = 256ll << 20;
// ... and by workgroups of 1024 lanes per (batch, head): more rows of one cache in flight per workgroup
// (same cache: QK 5.8 -> 6.2 TB/s, PV 6.3 -> 6.8 TB/s over 256 lanes; 64 lanes: 4.1 / 4.5 TB/s)
constexpr int kStreamBlock = 1024;

template <int DT, int LPK, bool STREAM>
__global__ __launch_bounds__(STREAM ? kStreamBlock : kBlock) void decode_qk_kernel(DecodeArgs a) {
  constexpr int kBlock = STREAM ? kStreamBlock : en::kBlock;
  typedef Elem<DT> E;
  typedef typename E::T T;
  constexpr int EPV = 16 / E::kSize;
  constexpr int KPS = kBlock / LPK;  // keys per step
  constexpr int U = 4;
  const int h = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x;
  const int c = tid % LPK, slot = tid / LPK;
  const int kl = min(a.kv_lens[b], a.Sk);
  const T *q = reinterpret_cast<const T *>(a.x) + ((int64_t)b * a.H + h) * a.D;
  const T *kbase = reinterpret_cast<const T *>(a.kv) + (int64_t)b * a.sb + (int64_t)h * a.sh;
  T *srow = reinterpret_cast<T *>(a.out) + ((int64_t)b * a.H + h) * a.Sk;

  // head sizes that are not a power-of-two number of vectors (80, 96) run on the next power of two of
  // lanes per key; the lanes past the head load nothing and add zeros
  const bool cv = c * EPV < a.D;
  float qv[EPV];
  {
    Pack<T, EPV> pk;
#pragma unroll
    for (int e = 0; e < EPV; ++e) pk.v[e] = E::from_float(0.f);
    if (cv) pk = load_pack<T, EPV>(q + c * EPV);
#pragma unroll
    for (int e = 0; e < EPV; ++e) qv[e] = E::to_float(pk.v[e]) * a.alpha;
  }
  for (int k0 = 0; k0 < kl; k0 += KPS * U) {  // uniform trip count: all lanes reach the reductions
    Pack<T, EPV> kv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = k0 + u * KPS + slot;
      if (key < kl && cv) kv[u] = __builtin_bit_cast(Pack<T, EPV>, load16<STREAM>(kbase + (int64_t)key * a.ss + c * EPV));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = k0 + u * KPS + slot;
      float dot = 0.f;
      if (key < kl && cv) {
#pragma unroll
        for (int e = 0; e < EPV; ++e) dot += qv[e] * E::to_float(kv[u].v[e]);
      }
      dot = group_allreduce<OpSum, LPK>(dot);
      if (c == 0 && key < kl) srow[key] = E::from_float(dot);
    }
  }
}

template <int DT, int LPK, bool STREAM>
__global__ __launch_bounds__(STREAM ? kStreamBlock : kBlock) void decode_pv_kernel(DecodeArgs a) {
  constexpr int kBlock = STREAM ? kStreamBlock : en::kBlock;
  typedef Elem<DT> E;
  typedef typename E::T T;
  constexpr int EPV = 16 / E::kSize;
  constexpr int KPS = kBlock / LPK;
  constexpr int U = 4;
  __shared__ float s_acc[KPS][LPK * EPV + 1];
  const int h = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x;
  const int c = tid % LPK, slot = tid / LPK;
  const int kl = min(a.kv_lens[b], a.Sk);
  const T *prow = reinterpret_cast<const T *>(a.x) + ((int64_t)b * a.H + h) * a.Sk;
  const T *vbase = reinterpret_cast<const T *>(a.kv) + (int64_t)b * a.sb + (int64_t)h * a.sh;
  T *ctx = reinterpret_cast<T *>(a.out) + ((int64_t)b * a.H + h) * a.D;
  const bool cv = c * EPV < a.D;     // lanes past the head size idle (head sizes such as 80 and 96)

  float acc[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) acc[e] = 0.f;
  for (int k0 = slot; k0 < kl; k0 += KPS * U) {
    Pack<T, EPV> vv[U];
    float p[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = k0 + u * KPS;
      p[u] = 0.f;
      if (key < kl && cv) {
        vv[u] = __builtin_bit_cast(Pack<T, EPV>, load16<STREAM>(vbase + (int64_t)key * a.ss + c * EPV));
        p[u] = E::to_float(prow[key]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = k0 + u * KPS;
      if (key < kl && cv) {
#pragma unroll
        for (int e = 0; e < EPV; ++e) acc[e] += p[u] * E::to_float(vv[u].v[e]);
      }
    }
  }
#pragma unroll
  for (int e = 0; e < EPV; ++e) s_acc[slot][c * EPV + e] = acc[e];
  __syncthreads();
  for (int d = tid; d < a.D; d += kBlock) {
    float s = 0.f;
#pragma unroll 4
    for (int j = 0; j < KPS; ++j) s += s_acc[j][d];
    ctx[d] = E::from_float(s);
  }
}

template <int DT, template <int, int> class Launcher>
static int dispatch_lpk(const DecodeArgs &a, int batch, hipStream_t s) {
  constexpr int EPV = 16 / Elem<DT>::kSize;
  int lpk = 4;                                 // lanes per key: vectors in a head, rounded up to a power of two
  while (lpk * EPV < a.D) lpk *= 2;
  dim3 grid((unsigned)a.H, (unsigned)batch, 1);
  switch (lpk) {
    case 4: Launcher<DT, 4>::go(a, grid, s); break;
    case 8: Launcher<DT, 8>::go(a, grid, s); break;
    case 16: Launcher<DT, 16>::go(a, grid, s); break;
    case 32: Launcher<DT, 32>::go(a, grid, s); break;
    case 64: Launcher<DT, 64>::go(a, grid, s); break;
    default: return EN_ERR_UNSUPPORTED;
  }
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

template <int DT, int LPK> struct QkLauncher {
  static void go(const DecodeArgs &a, dim3 grid, hipStream_t s) {
    if (a.stream) decode_qk_kernel<DT, LPK, true><<<grid, kStreamBlock, 0, s>>>(a);
    else decode_qk_kernel<DT, LPK, false><<<grid, kBlock, 0, s>>>(a);
  }
};
template <int DT, int LPK> struct PvLauncher {
  static void go(const DecodeArgs &a, dim3 grid, hipStream_t s) {
    if (a.stream) decode_pv_kernel<DT, LPK, true><<<grid, kStreamBlock, 0, s>>>(a);
    else decode_pv_kernel<DT, LPK, false><<<grid, kBlock, 0, s>>>(a);
  }
};

static int64_t cache_bytes(int batch, int head_num, int k_seq_len, int size_per_head, int dtype) {
  return (int64_t)batch * head_num * k_seq_len * size_per_head * dtype_size(dtype);
}

static int check_decode(const void *x, const void *kv, const void *out, const int32_t *lens, int batch, int head_num,
                        int k_seq_len, int size_per_head, int64_t sb, int64_t sh, int64_t ss, int dtype) {
  if (!x || !kv || !out || !lens) return EN_ERR_NULL;
  if (batch < 1 || batch > 65535 || head_num < 1 || k_seq_len < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  const int es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  const int epv = 16 / es;
  if ((size_per_head % epv) != 0) return EN_ERR_UNSUPPORTED;
  if (!aligned_to(kv, 16) || (sb % epv) || (sh % epv) || (ss % epv)) return EN_ERR_ALIGN;
  return EN_OK;
}

}  // namespace en

namespace en {

// Appends one new K row and one new V row per (batch, head) to the caches at position
// kv_lens[b]; sequences whose cache is full are left alone and counted.  Bytes are moved as they are.
struct AppendArgs {
  const unsigned char *k_new, *v_new;
  unsigned char *k_cache, *v_cache;
  const int32_t *kv_lens;
  int H, Sk;
  int row_bytes;
  int64_t n_sb, n_sh;           // strides of the new rows, bytes
  int64_t c_sb, c_sh, c_ss;     // strides of the caches, bytes
  int32_t *overflow;            // counts the sequences that had no room (null: not counted)
};

template <typename Vec>
__global__ __launch_bounds__(kWave) void kv_append_kernel(AppendArgs a) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int pos = a.kv_lens[b];
  if (pos < 0 || pos >= a.Sk) {
    if (a.overflow && h == 0 && threadIdx.x == 0) atomicAdd(a.overflow, 1);
    return;
  }
  const int64_t src = (int64_t)b * a.n_sb + (int64_t)h * a.n_sh;
  const int64_t dst = (int64_t)b * a.c_sb + (int64_t)h * a.c_sh + (int64_t)pos * a.c_ss;
  for (int i = threadIdx.x * (int)sizeof(Vec); i < a.row_bytes; i += kWave * (int)sizeof(Vec)) {
    *reinterpret_cast<Vec *>(a.k_cache + dst + i) = *reinterpret_cast<const Vec *>(a.k_new + src + i);
    *reinterpret_cast<Vec *>(a.v_cache + dst + i) = *reinterpret_cast<const Vec *>(a.v_new + src + i);
  }
}

}  // namespace en

extern "C" {

int en_kv_append(const void *k_new, const void *v_new, void *k_cache, void *v_cache, const int32_t *kv_lens,
                 int batch, int head_num, int k_seq_len, int size_per_head, int64_t new_stride_b,
                 int64_t new_stride_h, int64_t cache_stride_b, int64_t cache_stride_h, int64_t cache_stride_s,
                 int elem_size, int32_t *overflow, en_stream_t stream) {
  using namespace en;
  if (!k_new || !v_new || !k_cache || !v_cache || !kv_lens) return EN_ERR_NULL;
  if (overflow && !aligned_to(overflow, 4)) return EN_ERR_ALIGN;
  if (elem_size != 2 && elem_size != 4) return EN_ERR_DTYPE;
  if (batch < 1 || head_num < 1 || k_seq_len < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  if (batch > 65535) return EN_ERR_SHAPE;
  if (new_stride_b < 0 || new_stride_h < 0 || cache_stride_b < 0 || cache_stride_h < 0 || cache_stride_s < 0)
    return EN_ERR_UNSUPPORTED;
  AppendArgs a{(const unsigned char *)k_new, (const unsigned char *)v_new, (unsigned char *)k_cache,
               (unsigned char *)v_cache, kv_lens, head_num, k_seq_len, size_per_head * elem_size,
               new_stride_b * elem_size, new_stride_h * elem_size, cache_stride_b * elem_size,
               cache_stride_h * elem_size, cache_stride_s * elem_size, overflow};
  const dim3 grid((unsigned)head_num, (unsigned)batch, 1);
  hipStream_t s = (hipStream_t)stream;
  const bool v16 = (a.row_bytes % 16 == 0) && aligned_to(k_new, 16) && aligned_to(v_new, 16) &&
                   aligned_to(k_cache, 16) && aligned_to(v_cache, 16) && a.n_sb % 16 == 0 && a.n_sh % 16 == 0 &&
                   a.c_sb % 16 == 0 && a.c_sh % 16 == 0 && a.c_ss % 16 == 0;
  if (v16) {
    kv_append_kernel<uint4><<<grid, kWave, 0, s>>>(a);
  } else if (elem_size == 4) {
    if (!aligned_to(k_new, 4) || !aligned_to(v_new, 4) || !aligned_to(k_cache, 4) || !aligned_to(v_cache, 4))
      return EN_ERR_ALIGN;
    kv_append_kernel<uint32_t><<<grid, kWave, 0, s>>>(a);
  } else {
    if (!aligned_to(k_new, 2) || !aligned_to(v_new, 2) || !aligned_to(k_cache, 2) || !aligned_to(v_cache, 2))
      return EN_ERR_ALIGN;
    kv_append_kernel<uint16_t><<<grid, kWave, 0, s>>>(a);
  }
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_decode_qk(const void *q, const void *k_cache, void *scores, const int32_t *kv_lens, int batch, int head_num,
                 int k_seq_len, int size_per_head, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                 float alpha, int dtype, en_stream_t stream) {
  using namespace en;
  int rc = check_decode(q, k_cache, scores, kv_lens, batch, head_num, k_seq_len, size_per_head, k_stride_b,
                        k_stride_h, k_stride_s, dtype);
  if (rc) return rc;
  if (!aligned_to(q, 16) || !aligned_to(scores, dtype_size(dtype))) return EN_ERR_ALIGN;
  DecodeArgs a{q, k_cache, scores, kv_lens, head_num, k_seq_len, size_per_head, k_stride_b, k_stride_h, k_stride_s,
               alpha, cache_bytes(batch, head_num, k_seq_len, size_per_head, dtype) >= kStreamCacheBytes};
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return dispatch_lpk<EN_F32, QkLauncher>(a, batch, s);
    case EN_F16: return dispatch_lpk<EN_F16, QkLauncher>(a, batch, s);
    default: return dispatch_lpk<EN_BF16, QkLauncher>(a, batch, s);
  }
}

int en_decode_pv(const void *p, const void *v_cache, void *ctx, const int32_t *kv_lens, int batch, int head_num,
                 int k_seq_len, int size_per_head, int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                 int dtype, en_stream_t stream) {
  using namespace en;
  int rc = check_decode(p, v_cache, ctx, kv_lens, batch, head_num, k_seq_len, size_per_head, v_stride_b, v_stride_h,
                        v_stride_s, dtype);
  if (rc) return rc;
  if (!aligned_to(p, dtype_size(dtype)) || !aligned_to(ctx, dtype_size(dtype))) return EN_ERR_ALIGN;
  DecodeArgs a{p, v_cache, ctx, kv_lens, head_num, k_seq_len, size_per_head, v_stride_b, v_stride_h, v_stride_s, 1.f,
               cache_bytes(batch, head_num, k_seq_len, size_per_head, dtype) >= kStreamCacheBytes};
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return dispatch_lpk<EN_F32, PvLauncher>(a, batch, s);
    case EN_F16: return dispatch_lpk<EN_F16, PvLauncher>(a, batch, s);
    default: return dispatch_lpk<EN_BF16, PvLauncher>(a, batch, s);
  }
}

}  // extern "C"
