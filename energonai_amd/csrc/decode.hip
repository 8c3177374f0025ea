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

// ---------------------------------------------------------------------------------------------------------------
// Single-pass decode attention: ctx = softmax(scale * q K^T) V for one query per sequence, K and V each read
// once, scores and probabilities never written.  One workgroup per (batch, head); LPK lanes cover one cached row
// (16 bytes each), so the workgroup's NT / LPK lane groups take NT / LPK keys per step.  Two stages of registers:
// the K and V pieces of the next step are in flight while this step's are worked on, and the kernel stays within
// 64 registers so that two 1024-lane workgroups share a CU (measured on 72 heads x 64 caches of up to 2048
// positions, 2.6 GB: 6.7 TB/s; four pieces per lane and stage at one workgroup per CU 5.9, one stage of four
// pieces as in the two-kernel forms 5.3; a third stage spills).  Each lane group carries its own running maximum, sum and
// output slice (online softmax, maximum and exponent in the log2 domain with the scale folded in); the groups are
// combined once, through LDS, at the end.  The sequences are taken longest first (rank computed inside each
// workgroup from the lengths, batches of up to kRankBatch): the launch then ends on its short units instead of on
// whatever the last batch index happens to hold.
// ---------------------------------------------------------------------------------------------------------------
struct DecodeAttnArgs {
  const void *q;      // [B,H,D]
  const void *k, *v;  // caches [B,H,Smax,D], strided
  void *ctx;          // [B,H,D]
  const int32_t *kv_lens;
  int B, H, Sk, D;
  int64_t k_sb, k_sh, k_ss, v_sb, v_sh, v_ss;
  float c_exp;        // scale * log2(e)
  int nsplit;         // workgroups that share one (batch, head) unit's keys (grid z); 1: none
  float *partial;     // nsplit > 1: [B*H][nsplit][D + 2] unnormalised output, maximum (log2 domain), sum
  // paged caches: k and v are pools of pages, page p of head h at p * k_sb + h * k_sh (k_sb is the page stride),
  // position s of sequence b in page page_table[b * max_pages + s / page] at row s % page
  const int32_t *page_table;
  int max_pages, lg_page, num_pages;
};

// Keys of one workgroup when nsplit share a unit: a multiple of 64, so that the keys of one wave (at most 16) never
// straddle a share or a page.  The combine kernel derives the same shares from the length.
__device__ __forceinline__ int split_share(int kl, int nsplit) {
  return nsplit > 1 ? ((kl + nsplit - 1) / nsplit + 63) & ~63 : kl;
}

constexpr int kRankBatch = 256;

template <int DT, int LPK, bool STREAM, bool BIG, bool PAGED = false>
__global__ __launch_bounds__(BIG ? kStreamBlock : kBlock, 8) void decode_attn_kernel(DecodeAttnArgs a) {
  constexpr int NT = BIG ? kStreamBlock : en::kBlock;
  typedef Elem<DT> E;
  typedef typename E::T T;
  constexpr int EPV = 16 / E::kSize;
  constexpr int G = NT / LPK;        // lane groups = keys per step
  constexpr int U = 1;               // keys per lane group and stage
  constexpr int W = LPK * EPV;       // channels the lanes of a group cover (>= D)
  __shared__ float s_m[G], s_l[G], s_w[G];
  __shared__ float s_acc[G][W + 1];
  __shared__ int s_len[kRankBatch];
  __shared__ int s_b;
  const int tid = threadIdx.x;
  const int h = blockIdx.x;
  int b = blockIdx.y;
  if (a.B <= kRankBatch && a.B > 1) {
    // batch index whose length ranks blockIdx.y-th (longest first, ties by index)
    if (tid < a.B) s_len[tid] = min(a.kv_lens[tid], a.Sk);
    __syncthreads();
    if (tid < a.B) {
      const int mine = s_len[tid];
      int rank = 0;
      for (int j = 0; j < a.B; ++j) {
        const int lj = s_len[j];
        rank += (lj > mine || (lj == mine && j < tid)) ? 1 : 0;
      }
      if (rank == (int)blockIdx.y) s_b = tid;
    }
    __syncthreads();
    b = s_b;
  }
  const int c = tid % LPK, g = tid / LPK;
  const int kl = max(min(a.kv_lens[b], a.Sk), 0);
  // with the keys of a unit split over nsplit workgroups this one takes [kbeg, kend); a share past the end has no
  // workgroup's worth of work and leaves no partial (the combine kernel derives the same shares from the length)
  const int share = split_share(kl, a.nsplit);
  const int kbeg = (int)blockIdx.z * share, kend = min(kl, kbeg + share);
  if (a.nsplit > 1 && kbeg >= kl) return;
  const T *q = reinterpret_cast<const T *>(a.q) + ((int64_t)b * a.H + h) * a.D;
  const T *kbase = reinterpret_cast<const T *>(a.k) + (PAGED ? 0 : (int64_t)b * a.k_sb) + (int64_t)h * a.k_sh;
  const T *vbase = reinterpret_cast<const T *>(a.v) + (PAGED ? 0 : (int64_t)b * a.v_sb) + (int64_t)h * a.v_sh;
  T *ctx = reinterpret_cast<T *>(a.ctx) + ((int64_t)b * a.H + h) * a.D;
  const bool cv = c * EPV < a.D;     // lanes past the head size idle (head sizes such as 80 and 96)

  float qv[EPV];
  {
    Pack<T, EPV> pk;
#pragma unroll
    for (int e = 0; e < EPV; ++e) pk.v[e] = E::from_float(0.f);
    if (cv) pk = load_pack<T, EPV>(q + c * EPV);
#pragma unroll
    for (int e = 0; e < EPV; ++e) qv[e] = E::to_float(pk.v[e]) * a.c_exp;
  }
  float m_run = -INFINITY, l_run = 0.f;
  float acc[EPV];
#pragma unroll
  for (int e = 0; e < EPV; ++e) acc[e] = 0.f;

  // Bounds-checked buffer loads: a row at or past the sequence's length (and a lane past the head size) reads
  // zeros without a branch, so the loads of the next stage can be issued ahead of this stage's arithmetic and the
  // compiler counts what is outstanding statically.
  const rsrc_t k_rsrc = make_rsrc(kbase, kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * E::kSize) : 0u);
  const rsrc_t v_rsrc = make_rsrc(vbase, kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * a.v_ss + a.D) * E::kSize) : 0u);
  const uint32_t k_row = (uint32_t)(a.k_ss * E::kSize), v_row = (uint32_t)(a.v_ss * E::kSize);
  const uint32_t col = cv ? (uint32_t)(c * 16) : kOutOfRange;
  constexpr int AUX = STREAM ? 2 : 0;
  // Paged caches: the keys of one wave (64 / LPK of them, first one a multiple of that) lie in one page, so the
  // page is a wave-uniform choice of buffer.  Each wave keeps the ids of 64 pages of the sequence in one register,
  // lane i the id of page tab0 + i, and takes the one it needs with a lane read; the register is filled again when
  // the walk leaves its range (every 64 pages).  An id outside the pool makes an empty buffer: zeros, no access.
  constexpr int KPW = kWave / LPK;                   // keys of one wave and step
  const int wkey = __builtin_amdgcn_readfirstlane(tid / kWave) * KPW;
  const uint32_t page_mask = PAGED ? (1u << a.lg_page) - 1u : 0u;
  const uint32_t k_page_bytes = PAGED ? (uint32_t)((((int64_t)page_mask) * a.k_ss + a.D) * E::kSize) : 0u;
  const uint32_t v_page_bytes = PAGED ? (uint32_t)((((int64_t)page_mask) * a.v_ss + a.D) * E::kSize) : 0u;
  int tab = -1, tab0 = 0;
  auto fill_tab = [&](int first_page) {
    tab0 = first_page;
    const int pi = first_page + (tid % kWave);
    tab = pi < a.max_pages ? a.page_table[(int64_t)b * a.max_pages + pi] : -1;
  };
  if constexpr (PAGED) fill_tab((kbeg + wkey) >> a.lg_page);
  auto load_stage = [&](uint4 (&kk)[U], uint4 (&vv)[U], int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = k0 + u * G + g;
      const uint32_t in = key < kend ? 0u : kOutOfRange;     // past the end: out of range whatever the stride
      if constexpr (PAGED) {
        const int pi = (k0 + u * G + wkey) >> a.lg_page;      // wave-uniform
        if (pi - tab0 >= kWave) fill_tab(pi);
        const int id = __builtin_amdgcn_readlane(tab, pi - tab0);
        const bool ok = (unsigned)id < (unsigned)a.num_pages;
        const rsrc_t kr = make_rsrc(kbase + (int64_t)id * a.k_sb, ok ? k_page_bytes : 0u);
        const rsrc_t vr = make_rsrc(vbase + (int64_t)id * a.v_sb, ok ? v_page_bytes : 0u);
        const uint32_t row = (uint32_t)key & page_mask;
        kk[u] = buffer_load16<AUX>(kr, row * k_row + col | in);
        vv[u] = buffer_load16<AUX>(vr, row * v_row + col | in);
      } else {
        kk[u] = buffer_load16<AUX>(k_rsrc, (uint32_t)key * k_row + col | in);
        vv[u] = buffer_load16<AUX>(v_rsrc, (uint32_t)key * v_row + col | in);
      }
    }
  };
  auto compute_stage = [&](const uint4 (&kk)[U], const uint4 (&vv)[U], int k0) {
    float sc[U];
    float m_new = m_run;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = k0 + u * G + g;
      const Pack<T, EPV> kp = __builtin_bit_cast(Pack<T, EPV>, kk[u]);
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < EPV; ++e) dot += qv[e] * E::to_float(kp.v[e]);
      dot = group_allreduce<OpSum, LPK>(dot);
      sc[u] = key < kend ? dot : -INFINITY;
      m_new = fmaxf(m_new, sc[u]);
    }
    if (m_new > -INFINITY) {            // this group has seen a key: (-inf) - (-inf) never reaches exp2
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);      // exp2(-inf) = 0 on the first key
      l_run *= alpha;
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc[e] *= alpha;
      m_run = m_new;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const Pack<T, EPV> vp = __builtin_bit_cast(Pack<T, EPV>, vv[u]);
        const float p = __builtin_amdgcn_exp2f(sc[u] - m_new);        // 0 for a key past the end
        l_run += p;
#pragma unroll
        for (int e = 0; e < EPV; ++e) acc[e] += p * E::to_float(vp.v[e]);
      }
    }
  };
  // NS stages of registers: while one is worked on, the loads of the others are in flight
  constexpr int STEP = G * U;
  constexpr int NS = 2;
  static_assert((2 * NS - 1) * STEP <= 4096, "the host check allows 4096 keys past the end");
  uint4 kr[NS][U], vr[NS][U];
#pragma unroll
  for (int st = 0; st < NS - 1; ++st) load_stage(kr[st], vr[st], kbeg + st * STEP);
  for (int k0 = kbeg; k0 < kend; k0 += NS * STEP) {   // uniform trip count: all lanes reach the reductions
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      load_stage(kr[(st + NS - 1) % NS], vr[(st + NS - 1) % NS], k0 + (st + NS - 1) * STEP);
      compute_stage(kr[st], vr[st], k0 + st * STEP);
    }
  }
  if (c == 0) { s_m[g] = m_run; s_l[g] = l_run; }
#pragma unroll
  for (int e = 0; e < EPV; ++e) s_acc[g][c * EPV + e] = acc[e];
  __syncthreads();
  float m_all = -INFINITY;
  for (int j = 0; j < G; ++j) m_all = fmaxf(m_all, s_m[j]);
  if (tid < G) s_w[tid] = s_m[tid] > -INFINITY ? __builtin_amdgcn_exp2f(s_m[tid] - m_all) : 0.f;
  __syncthreads();
  float *part = a.nsplit > 1 ? a.partial + (((int64_t)b * a.H + h) * a.nsplit + blockIdx.z) * (a.D + 2) : nullptr;
  for (int d = tid; d < a.D; d += NT) {
    float l = 0.f, o = 0.f;
#pragma unroll 4
    for (int j = 0; j < G; ++j) {
      l += s_l[j] * s_w[j];
      o += s_acc[j][d] * s_w[j];
    }
    if (part) {
      part[d] = o;
      if (d == 0) { part[a.D] = m_all; part[a.D + 1] = l; }
    } else {
      ctx[d] = E::from_float(l > 0.f ? o / l : 0.f);
    }
  }
}

// Combines the partial results of the workgroups that shared a unit's keys: one workgroup per (batch, head).
template <int DT>
__global__ __launch_bounds__(kBlock) void decode_attn_combine_kernel(DecodeAttnArgs a) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  const int unit = blockIdx.x, b = unit / a.H;
  const int kl = max(min(a.kv_lens[b], a.Sk), 0);
  const int share = split_share(kl, a.nsplit);
  const int nvalid = share > 0 ? (kl + share - 1) / share : 0;       // shares that had keys
  const float *part = a.partial + (int64_t)unit * a.nsplit * (a.D + 2);
  T *ctx = reinterpret_cast<T *>(a.ctx) + (int64_t)unit * a.D;
  float m_all = -INFINITY;
  for (int z = 0; z < nvalid; ++z) m_all = fmaxf(m_all, part[z * (a.D + 2) + a.D]);
  float l = 0.f;
  for (int z = 0; z < nvalid; ++z) {
    const float m = part[z * (a.D + 2) + a.D];
    l += m > -INFINITY ? part[z * (a.D + 2) + a.D + 1] * __builtin_amdgcn_exp2f(m - m_all) : 0.f;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  for (int d = threadIdx.x; d < a.D; d += kBlock) {
    float o = 0.f;
    for (int z = 0; z < nvalid; ++z) {
      const float m = part[z * (a.D + 2) + a.D];
      o += m > -INFINITY ? part[z * (a.D + 2) + d] * __builtin_amdgcn_exp2f(m - m_all) : 0.f;
    }
    ctx[d] = E::from_float(o * inv);
  }
}

template <int DT, int LPK, bool PAGED = false> struct AttnLauncher {
  // stream_cache: caches too large to stay in the memory-side cache between steps are read with non-temporal loads;
  // big: 1024-lane workgroups (large caches, and whenever a unit's keys are split: few units, long rows)
  static void go(const DecodeAttnArgs &a, dim3 grid, bool stream_cache, bool big, hipStream_t s) {
    if (stream_cache) decode_attn_kernel<DT, LPK, true, true, PAGED><<<grid, kStreamBlock, 0, s>>>(a);
    else if (big) decode_attn_kernel<DT, LPK, false, true, PAGED><<<grid, kStreamBlock, 0, s>>>(a);
    else decode_attn_kernel<DT, LPK, false, false, PAGED><<<grid, kBlock, 0, s>>>(a);
  }
};

template <int DT, bool PAGED = false>
static int dispatch_attn(const DecodeAttnArgs &a, bool stream_cache, hipStream_t s) {
  constexpr int EPV = 16 / Elem<DT>::kSize;
  int lpk = 4;
  while (lpk * EPV < a.D) lpk *= 2;
  dim3 grid((unsigned)a.H, (unsigned)a.B, (unsigned)a.nsplit);
  const bool big = stream_cache || a.nsplit > 1;
  switch (lpk) {
    case 4: AttnLauncher<DT, 4, PAGED>::go(a, grid, stream_cache, big, s); break;
    case 8: AttnLauncher<DT, 8, PAGED>::go(a, grid, stream_cache, big, s); break;
    case 16: AttnLauncher<DT, 16, PAGED>::go(a, grid, stream_cache, big, s); break;
    case 32: AttnLauncher<DT, 32, PAGED>::go(a, grid, stream_cache, big, s); break;
    case 64: AttnLauncher<DT, 64, PAGED>::go(a, grid, stream_cache, big, s); break;
    default: return EN_ERR_UNSUPPORTED;
  }
  EN_RETURN_IF_LAUNCH_FAILED();
  if (a.nsplit > 1) {
    decode_attn_combine_kernel<DT><<<(unsigned)(a.B * a.H), kBlock, 0, s>>>(a);
    EN_RETURN_IF_LAUNCH_FAILED();
  }
  return EN_OK;
}

// How many workgroups share one unit's keys: none while the units alone fill the chip's 512 slots of 1024 lanes;
// else enough for about two slots' worth per CU, each share at least 512 keys long (shorter shares cost more in
// workgroup start-up and in the combine pass than they win: 22 us instead of 25 for one sequence of 2048 keys).
static int decode_split(int batch, int head_num, int k_seq_len) {
  constexpr int kTargetWorkgroups = 1024, kMinShare = 512;
  const int64_t units = (int64_t)batch * head_num;
  if (units >= 512 || k_seq_len < 2 * kMinShare) return 1;
  int64_t n = (kTargetWorkgroups + units - 1) / units;
  if (n > k_seq_len / kMinShare) n = k_seq_len / kMinShare;
  if (n > 64) n = 64;
  return n < 1 ? 1 : (int)n;
}

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


// Paged caches: the same append, the row found through the page table.  A sequence whose next position has no page
// (position past max_pages * page, id outside the pool) is left alone and counted.
struct PagedAppendArgs {
  const unsigned char *k_new, *v_new;
  unsigned char *k_pool, *v_pool;
  const int32_t *kv_lens, *page_table;
  int H, max_pages, lg_page, num_pages;
  int row_bytes;
  int64_t n_sb, n_sh;           // strides of the new rows, bytes
  int64_t p_sp, p_sh, p_ss;     // page, head and row strides of the pools, bytes
  int32_t *overflow;
};

__global__ __launch_bounds__(kWave) void kv_append_paged_kernel(PagedAppendArgs a) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int pos = a.kv_lens[b];
  const int pi = pos >> a.lg_page;
  const int id = (pos >= 0 && pi < a.max_pages) ? a.page_table[(int64_t)b * a.max_pages + pi] : -1;
  if ((unsigned)id >= (unsigned)a.num_pages) {
    if (a.overflow && h == 0 && threadIdx.x == 0) atomicAdd(a.overflow, 1);
    return;
  }
  const int64_t src = (int64_t)b * a.n_sb + (int64_t)h * a.n_sh;
  const int64_t dst = (int64_t)id * a.p_sp + (int64_t)h * a.p_sh + (int64_t)(pos & ((1 << a.lg_page) - 1)) * a.p_ss;
  for (int i = threadIdx.x * 16; i < a.row_bytes; i += kWave * 16) {
    *reinterpret_cast<uint4 *>(a.k_pool + dst + i) = *reinterpret_cast<const uint4 *>(a.k_new + src + i);
    *reinterpret_cast<uint4 *>(a.v_pool + dst + i) = *reinterpret_cast<const uint4 *>(a.v_new + src + i);
  }
}

// Prefill into pages: the rows of sequence b, packed tokens cu[b] .. of a [T, src_head_rows, D] source of which heads
// src_head_first .. + H - 1 are taken, go to rows 0 .. len - 1 of the sequence's pages.
struct PagedFillArgs {
  const unsigned char *src;
  unsigned char *pool;
  const int32_t *cu, *page_table;
  int H, S, max_pages, lg_page, num_pages;
  int vecs_per_row;             // 16-byte vectors per head row
  int64_t s_row, s_head;        // source: bytes per token, bytes per head row
  int64_t head_first_bytes;
  int64_t p_sp, p_sh, p_ss;
  int32_t *overflow;
};

__global__ __launch_bounds__(kBlock) void kv_fill_paged_kernel(PagedFillArgs a) {
  constexpr int ROWS = 4;
  const int b = blockIdx.y;
  const int t0 = a.cu[b], len = min(a.cu[b + 1] - t0, a.S);
  const int per_row = a.H * a.vecs_per_row;
  for (int r = 0; r < ROWS; ++r) {
    const int s = blockIdx.x * ROWS + r;
    if (s >= len) return;
    const int pi = s >> a.lg_page;
    const int id = pi < a.max_pages ? a.page_table[(int64_t)b * a.max_pages + pi] : -1;
    if ((unsigned)id >= (unsigned)a.num_pages) {
      if (a.overflow && threadIdx.x == 0) atomicAdd(a.overflow, 1);
      continue;
    }
    const unsigned char *src = a.src + (int64_t)(t0 + s) * a.s_row + a.head_first_bytes;
    unsigned char *dst = a.pool + (int64_t)id * a.p_sp + (int64_t)(s & ((1 << a.lg_page) - 1)) * a.p_ss;
    for (int i = threadIdx.x; i < per_row; i += kBlock) {
      const int h = i / a.vecs_per_row, c = i - h * a.vecs_per_row;
      *reinterpret_cast<uint4 *>(dst + (int64_t)h * a.p_sh + c * 16) =
          *reinterpret_cast<const uint4 *>(src + (int64_t)h * a.s_head + c * 16);
    }
  }
}

static int log2_exact(int v) {
  int lg = 0;
  while ((1 << lg) < v) ++lg;
  return (1 << lg) == v ? lg : -1;
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

int64_t en_decode_attn_workspace_bytes(int batch, int head_num, int k_seq_len, int size_per_head) {
  using namespace en;
  if (batch < 1 || head_num < 1 || k_seq_len < 1 || size_per_head < 1) return 0;
  const int n = decode_split(batch, head_num, k_seq_len);
  return n > 1 ? (int64_t)batch * head_num * n * (size_per_head + 2) * (int64_t)sizeof(float) : 0;
}

int en_decode_attn(const void *q, const void *k_cache, const void *v_cache, void *ctx, const int32_t *kv_lens, int batch,
                   int head_num, int k_seq_len, int size_per_head, const int64_t *k_strides, const int64_t *v_strides,
                   float scale, int dtype, void *workspace, int64_t workspace_bytes, en_stream_t stream) {
  using namespace en;
  if (!k_strides || !v_strides || !v_cache) return EN_ERR_NULL;
  int rc = check_decode(q, k_cache, ctx, kv_lens, batch, head_num, k_seq_len, size_per_head, k_strides[0], k_strides[1],
                        k_strides[2], dtype);
  if (rc) return rc;
  const int es = dtype_size(dtype), epv = 16 / es;
  if (!aligned_to(v_cache, 16) || (v_strides[0] % epv) || (v_strides[1] % epv) || (v_strides[2] % epv)) return EN_ERR_ALIGN;
  if (!aligned_to(q, 16) || !aligned_to(ctx, es)) return EN_ERR_ALIGN;
  if (size_per_head > 64 * epv) return EN_ERR_UNSUPPORTED;
  // 32-bit byte offsets inside a (batch, head) unit, two stages of keys past the end included
  if (((int64_t)k_seq_len + 4096) * k_strides[2] * es >= (1ll << 31) || ((int64_t)k_seq_len + 4096) * v_strides[2] * es >= (1ll << 31))
    return EN_ERR_UNSUPPORTED;
  if (!(scale > 0.f)) return EN_ERR_UNSUPPORTED;     // the running maximum is kept in units of scale * log2(e)
  for (int i = 0; i < 3; ++i)
    if (k_strides[i] < 0 || v_strides[i] < 0) return EN_ERR_UNSUPPORTED;
  // a unit's keys are shared between workgroups only when the caller brought the room for their partial results
  const int64_t need = en_decode_attn_workspace_bytes(batch, head_num, k_seq_len, size_per_head);
  const bool split = need > 0 && workspace && workspace_bytes >= need && aligned_to(workspace, 4);
  DecodeAttnArgs a{q, k_cache, v_cache, ctx, kv_lens, batch, head_num, k_seq_len, size_per_head, k_strides[0], k_strides[1],
                   k_strides[2], v_strides[0], v_strides[1], v_strides[2], scale * 1.4426950408889634f,
                   split ? decode_split(batch, head_num, k_seq_len) : 1, static_cast<float *>(workspace)};
  const bool stream_cache = 2 * cache_bytes(batch, head_num, k_seq_len, size_per_head, dtype) >= kStreamCacheBytes;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return dispatch_attn<EN_F32>(a, stream_cache, s);
    case EN_F16: return dispatch_attn<EN_F16>(a, stream_cache, s);
    default: return dispatch_attn<EN_BF16>(a, stream_cache, s);
  }
}

int en_kv_append_paged(const void *k_new, const void *v_new, void *k_pool, void *v_pool, const int32_t *kv_lens,
                       const int32_t *page_table, int batch, int head_num, int max_pages_per_seq, int page_size,
                       int num_pages, int size_per_head, int64_t new_stride_b, int64_t new_stride_h,
                       const int64_t *pool_strides, int elem_size, int32_t *overflow, en_stream_t stream) {
  using namespace en;
  if (!k_new || !v_new || !k_pool || !v_pool || !kv_lens || !page_table || !pool_strides) return EN_ERR_NULL;
  if (overflow && !aligned_to(overflow, 4)) return EN_ERR_ALIGN;
  if (elem_size != 2 && elem_size != 4) return EN_ERR_DTYPE;
  if (batch < 1 || batch > 65535 || head_num < 1 || max_pages_per_seq < 1 || num_pages < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  const int lg = log2_exact(page_size);
  if (lg < 4) return EN_ERR_UNSUPPORTED;                                  // a power of two, at least 16
  if ((int64_t)max_pages_per_seq * page_size >= (1ll << 31)) return EN_ERR_SHAPE;
  if (new_stride_b < 0 || new_stride_h < 0 || pool_strides[0] < 0 || pool_strides[1] < 0 || pool_strides[2] < 0)
    return EN_ERR_UNSUPPORTED;
  PagedAppendArgs a{(const unsigned char *)k_new, (const unsigned char *)v_new, (unsigned char *)k_pool,
                    (unsigned char *)v_pool, kv_lens, page_table, head_num, max_pages_per_seq, lg, num_pages,
                    size_per_head * elem_size, new_stride_b * elem_size, new_stride_h * elem_size,
                    pool_strides[0] * elem_size, pool_strides[1] * elem_size, pool_strides[2] * elem_size, overflow};
  if ((a.row_bytes % 16) || !aligned_to(k_new, 16) || !aligned_to(v_new, 16) || !aligned_to(k_pool, 16) ||
      !aligned_to(v_pool, 16) || (a.n_sb % 16) || (a.n_sh % 16) || (a.p_sp % 16) || (a.p_sh % 16) || (a.p_ss % 16))
    return EN_ERR_ALIGN;
  kv_append_paged_kernel<<<dim3((unsigned)head_num, (unsigned)batch, 1), kWave, 0, (hipStream_t)stream>>>(a);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_kv_fill_paged(const void *src, void *pool, const int32_t *cu_seqlens, const int32_t *page_table, int batch,
                     int max_seq_len, int head_num, int size_per_head, int src_head_rows, int src_head_first,
                     int max_pages_per_seq, int page_size, int num_pages, const int64_t *pool_strides, int elem_size,
                     int32_t *overflow, en_stream_t stream) {
  using namespace en;
  if (!src || !pool || !cu_seqlens || !page_table || !pool_strides) return EN_ERR_NULL;
  if (overflow && !aligned_to(overflow, 4)) return EN_ERR_ALIGN;
  if (elem_size != 2 && elem_size != 4) return EN_ERR_DTYPE;
  if (batch < 1 || batch > 65535 || max_seq_len < 1 || head_num < 1 || size_per_head < 1 || max_pages_per_seq < 1 ||
      num_pages < 1)
    return EN_ERR_SHAPE;
  if (src_head_first < 0 || src_head_rows < src_head_first + head_num) return EN_ERR_SHAPE;
  const int lg = log2_exact(page_size);
  if (lg < 4) return EN_ERR_UNSUPPORTED;
  if ((int64_t)max_pages_per_seq * page_size >= (1ll << 31)) return EN_ERR_SHAPE;
  if (pool_strides[0] < 0 || pool_strides[1] < 0 || pool_strides[2] < 0) return EN_ERR_UNSUPPORTED;
  const int64_t row_bytes = (int64_t)size_per_head * elem_size;
  PagedFillArgs a{(const unsigned char *)src, (unsigned char *)pool, cu_seqlens, page_table, head_num, max_seq_len,
                  max_pages_per_seq, lg, num_pages, (int)(row_bytes / 16), (int64_t)src_head_rows * row_bytes, row_bytes,
                  (int64_t)src_head_first * row_bytes, pool_strides[0] * elem_size, pool_strides[1] * elem_size,
                  pool_strides[2] * elem_size, overflow};
  if ((row_bytes % 16) || !aligned_to(src, 16) || !aligned_to(pool, 16) || (a.p_sp % 16) || (a.p_sh % 16) || (a.p_ss % 16))
    return EN_ERR_ALIGN;
  const dim3 grid((unsigned)ceil_div(max_seq_len, 4), (unsigned)batch, 1);
  kv_fill_paged_kernel<<<grid, kBlock, 0, (hipStream_t)stream>>>(a);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_decode_attn_paged(const void *q, const void *k_pool, const void *v_pool, void *ctx, const int32_t *kv_lens,
                         const int32_t *page_table, int batch, int head_num, int max_pages_per_seq, int page_size,
                         int num_pages, int size_per_head, const int64_t *k_strides, const int64_t *v_strides, float scale,
                         int dtype, void *workspace, int64_t workspace_bytes, en_stream_t stream) {
  using namespace en;
  if (!k_strides || !v_strides || !v_pool || !page_table) return EN_ERR_NULL;
  if (max_pages_per_seq < 1 || num_pages < 1) return EN_ERR_SHAPE;
  const int lg = log2_exact(page_size);
  if (lg < 4) return EN_ERR_UNSUPPORTED;                                  // a power of two, at least 16: a wave's keys share a page
  if ((int64_t)max_pages_per_seq * page_size >= (1ll << 30)) return EN_ERR_SHAPE;
  const int k_seq_len = max_pages_per_seq * page_size;
  int rc = check_decode(q, k_pool, ctx, kv_lens, batch, head_num, k_seq_len, size_per_head, k_strides[0], k_strides[1],
                        k_strides[2], dtype);
  if (rc) return rc;
  const int es = dtype_size(dtype), epv = 16 / es;
  if (!aligned_to(v_pool, 16) || (v_strides[0] % epv) || (v_strides[1] % epv) || (v_strides[2] % epv)) return EN_ERR_ALIGN;
  if (!aligned_to(q, 16) || !aligned_to(ctx, es)) return EN_ERR_ALIGN;
  if (size_per_head > 64 * epv) return EN_ERR_UNSUPPORTED;
  // 32-bit byte offsets inside a page
  if ((int64_t)page_size * k_strides[2] * es >= (1ll << 31) || (int64_t)page_size * v_strides[2] * es >= (1ll << 31))
    return EN_ERR_UNSUPPORTED;
  if (!(scale > 0.f)) return EN_ERR_UNSUPPORTED;
  for (int i = 0; i < 3; ++i)
    if (k_strides[i] < 0 || v_strides[i] < 0) return EN_ERR_UNSUPPORTED;
  const int64_t need = en_decode_attn_workspace_bytes(batch, head_num, k_seq_len, size_per_head);
  const bool split = need > 0 && workspace && workspace_bytes >= need && aligned_to(workspace, 4);
  DecodeAttnArgs a{q, k_pool, v_pool, ctx, kv_lens, batch, head_num, k_seq_len, size_per_head, k_strides[0], k_strides[1],
                   k_strides[2], v_strides[0], v_strides[1], v_strides[2], scale * 1.4426950408889634f,
                   split ? decode_split(batch, head_num, k_seq_len) : 1, static_cast<float *>(workspace),
                   page_table, max_pages_per_seq, lg, num_pages};
  const bool stream_cache = 2 * cache_bytes(batch, head_num, k_seq_len, size_per_head, dtype) >= kStreamCacheBytes;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return dispatch_attn<EN_F32, true>(a, stream_cache, s);
    case EN_F16: return dispatch_attn<EN_F16, true>(a, stream_cache, s);
    default: return dispatch_attn<EN_BF16, true>(a, stream_cache, s);
  }
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
