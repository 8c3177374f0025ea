// Fused attention for the padded [B,H,S,*] layout and for the packed layout
// (all valid tokens back to back, no padding rows anywhere):
//
//   ctx = softmax(scale * Q K^T, causal / key-padding mask) V
//
// in one kernel, so the [B,H,Sq,Sk] score tensor never exists in HBM.  This is
// an addition to the reference's API (its callers run matmul, softmax, matmul,
// examples/bert/bert.py:108-119); the three separate ops stay available.
//
// Workgroup: 4 waves, one tile of 128 query rows of one (batch, head); wave w
// owns query rows 32w..32w+31 and every channel.  Per 64-key tile:
//
//   S^T = K Q^T      A = K rows from LDS, B = Q fragments held in registers.
//                    The 32x32 result gives each lane ONE query (its column)
//                    and 16 of the 32 keys, so row maxima and sums are
//                    per-lane reductions plus one exchange between the two
//                    lane groups.
//   online softmax   running max / sum per lane; exp2 with the scale folded in.
//   O^T += V^T P^T   A = V^T rows from LDS (V is staged transposed), B = the
//                    probabilities straight out of the S^T accumulators,
//                    rounded to the storage type: a lane's registers
//                    (j, i) hold keys 8j + 4g + i, and the A operand simply
//                    reads V^T at those same keys, so P never touches LDS.
//
// K/V tiles are fetched with bounds-checked 128-bit buffer loads one tile
// ahead and the barriers order LDS only, as in the unfused kernels.
#include "attn_common.hip.h"

namespace en {

struct FusedArgs {
  AttnArgs base;             // a_ptr = q, b_ptr = k, out = ctx; q_s* = q strides, k_s* = k strides
  const void *v;
  int64_t v_sb, v_sh, v_ss;
  int64_t c_sb, c_sh, c_ss;
  const int32_t *q_row0;     // packed layout: first row of batch b in q / ctx (else null)
  const int32_t *k_row0;     // packed layout: first row of batch b in k / v (else null)
  float scale;
};

template <int DT, int DP>
__global__ __launch_bounds__(kBlock, 2) void attn_fused_kernel(FusedArgs fa) {
  static_assert(DT != EN_F32, "the fused kernel is built for 16-bit storage");
  typedef Elem<DT> E;
  typedef typename E::T T;
  typedef Mma<DT> M;
  const AttnArgs &a = fa.base;
  constexpr int EPV = 8;
  constexpr int BK = 64;                         // keys per tile
  constexpr int KB = BK / 32;                    // 32-key MFMA blocks per tile
  constexpr int NVS = DP / 16;                   // MFMA steps over the head dim
  constexpr int DMT = DP / 32;                   // 32-channel MFMA tiles of the output
  constexpr int KPITCH = DP + EPV;               // LDS pitch of a K row
  constexpr int VPITCH = BK + EPV;               // LDS pitch of a V^T row
  constexpr int KVEC_ROW = DP / EPV;
  constexpr int KLOADS = BK * KVEC_ROW / kBlock;
  constexpr int NQUAD = BK / 4, NCHUNK = DP / EPV;
  constexpr int VUNITS = NQUAD * NCHUNK;         // (four keys, eight channels) units of a V tile
  constexpr int VLOADS = (VUNITS + kBlock - 1) / kBlock;
  constexpr float kLog2e = 1.4426950408889634f;
  static_assert(BK * KVEC_ROW % kBlock == 0, "K tile must divide over the block");
  __shared__ __attribute__((aligned(16))) T lds_k[BK * KPITCH];
  __shared__ __attribute__((aligned(16))) T lds_v[DP * VPITCH];

  int unit, qi;
  if (!map_block(a, unit, qi)) return;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
  const int q0 = qi * kQTile;
  if (q0 >= ql) return;
  const int nk = tile_key_extent(a, min(q0 + kQTile, ql) - 1, kl, ql);
  const int nkt = (nk + BK - 1) / BK;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int q = q0 + wave * 32 + r;              // this lane's query row
  const bool q_valid = q < ql;
  // keys this query may see: k < vis
  const int vis = q_valid ? (a.causal ? min(kl, q + (kl - ql) + 1) : kl) : 0;
  // smallest extent among the wave's 32 queries (wave-uniform): tiles below it need no masking
  const int q_first = q0 + wave * 32;
  const int vis_min = (q_first + 31 < ql) ? (a.causal ? min(kl, q_first + (kl - ql) + 1) : kl) : 0;

  // batch base: b * batch stride (padded layout) or first-row * row stride (packed layout)
  const int64_t qr = fa.q_row0 ? fa.q_row0[b] : 0, kr = fa.k_row0 ? fa.k_row0[b] : 0;
  const T *qbase = reinterpret_cast<const T *>(a.a_ptr) + (int64_t)b * a.q_sb + qr * a.q_ss + (int64_t)h * a.q_sh;
  const T *kbase = reinterpret_cast<const T *>(a.b_ptr) + (int64_t)b * a.k_sb + kr * a.k_ss + (int64_t)h * a.k_sh;
  const T *vbase = reinterpret_cast<const T *>(fa.v) + (int64_t)b * fa.v_sb + kr * fa.v_ss + (int64_t)h * fa.v_sh;
  T *cbase = reinterpret_cast<T *>(a.out) + (int64_t)b * fa.c_sb + qr * fa.c_ss + (int64_t)h * fa.c_sh;

  // Q fragments (B operand of S^T = K Q^T): this lane's query row, 8 channels per step
  uint4 qf[NVS];
  {
    const rsrc_t q_rsrc = make_rsrc(qbase, (uint32_t)(((int64_t)(ql - 1) * a.q_ss + a.D) * E::kSize));
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      const int d = M::k_of(vs, g, NVS);
      const uint32_t off = (uint32_t)(((int64_t)q * a.q_ss + d) * E::kSize);
      qf[vs] = buffer_load16(q_rsrc, (q_valid && d < a.D) ? off : kOutOfRange);
    }
  }

  const rsrc_t k_rsrc = make_rsrc(kbase, (uint32_t)(((int64_t)(max(kl, 1) - 1) * a.k_ss + a.D) * E::kSize));
  const rsrc_t v_rsrc = make_rsrc(vbase, (uint32_t)(((int64_t)(max(kl, 1) - 1) * fa.v_ss + a.D) * E::kSize));
  uint4 kreg[KLOADS];
  uint4 vreg[VLOADS][4];
  auto fetch = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / KVEC_ROW, c = v % KVEC_ROW;
      const int key = k0 + row;
      const uint32_t off = (uint32_t)(((int64_t)key * a.k_ss + c * EPV) * E::kSize);
      kreg[i] = buffer_load16(k_rsrc, (kt < nkt && key < kl && c * EPV < a.D) ? off : kOutOfRange);
    }
#pragma unroll
    for (int i = 0; i < VLOADS; ++i) {
      const int u = tid + i * kBlock;
      const int c = (u % 4) + 4 * (u / (4 * NQUAD));
      const int kq = (u / 4) % NQUAD;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int key = k0 + kq * 4 + x;
        const uint32_t off = (uint32_t)(((int64_t)key * fa.v_ss + c * EPV) * E::kSize);
        vreg[i][x] = buffer_load16(v_rsrc, (kt < nkt && u < VUNITS && key < kl && c * EPV < a.D) ? off : kOutOfRange);
      }
    }
  };
  fetch(0);

  floatx16 o[DMT];
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
    for (int x = 0; x < 16; ++x) o[mt][x] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float c_exp = fa.scale * kLog2e;

  for (int kt = 0; kt < nkt; ++kt) {
    const int k0 = kt * BK;
    // registers -> LDS: K as is, V transposed (four keys of one channel per 64-bit store)
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) {
      const int v = tid + i * kBlock;
      *reinterpret_cast<uint4 *>(&lds_k[(v / KVEC_ROW) * KPITCH + (v % KVEC_ROW) * EPV]) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VLOADS; ++i) {
      const int u = tid + i * kBlock;
      if (VUNITS % kBlock == 0 || u < VUNITS) {
        const int c = (u % 4) + 4 * (u / (4 * NQUAD));
        const int kq = (u / 4) % NQUAD;
        Pack<T, EPV> rows[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) rows[x] = __builtin_bit_cast(Pack<T, EPV>, vreg[i][x]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          Pack<T, 4> col;
#pragma unroll
          for (int x = 0; x < 4; ++x) col.v[x] = rows[x].v[e];
          store_pack<T, 4>(&lds_v[(c * EPV + e) * VPITCH + kq * 4], col);
        }
      }
    }
    lds_barrier();
    fetch(kt + 1);

    // ---- S^T = K Q^T for the tile's KB blocks of 32 keys
    floatx16 s[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
      for (int x = 0; x < 16; ++x) s[kb][x] = 0.f;
#pragma unroll
      for (int vs = 0; vs < NVS; ++vs) {
        const uint4 kf = *reinterpret_cast<const uint4 *>(&lds_k[(kb * 32 + r) * KPITCH + M::k_of(vs, g, NVS)]);
        M::step(kf, qf[vs], s[kb]);
      }
    }

    // ---- mask + online softmax; register 4j+i of block kb holds key k0 + 32kb + 8j + 4g + i
    float m_tile = -INFINITY;
    if (k0 + BK <= vis_min) {  // whole tile visible to every query of this wave: no masking work
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int x = 0; x < 16; ++x) m_tile = fmaxf(m_tile, s[kb][x]);
    } else {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          const int key = k0 + kb * 32 + 8 * (x >> 2) + 4 * g + (x & 3);
          const float v = (key < vis) ? s[kb][x] : -INFINITY;
          s[kb][x] = v;
          m_tile = fmaxf(m_tile, v);
        }
    }
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, kWave));   // the other half of this query's keys
    const float m_new = fmaxf(m_run, m_tile);
    const float moff = (m_new == -INFINITY) ? 0.f : -m_new * c_exp;
    const float alpha = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(fmaf(m_run, c_exp, moff));
    float l_tile = 0.f;
    uint4 pf[KB][2];                                           // B operands of the second MFMA
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      Pack<T, EPV> pk[2];
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const float p = (s[kb][x] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(fmaf(s[kb][x], c_exp, moff));
        const T pt = E::from_float(p);
        l_tile += E::to_float(pt);                             // sum what is actually multiplied
        pk[x >> 3].v[x & 7] = pt;                              // step t = x/8 takes registers j = 2t, 2t+1
      }
      pf[kb][0] = __builtin_bit_cast(uint4, pk[0]);
      pf[kb][1] = __builtin_bit_cast(uint4, pk[1]);
    }
    l_tile += __shfl_xor(l_tile, 32, kWave);
    l_run = l_run * alpha + l_tile;
    m_run = m_new;
#pragma unroll
    for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
      for (int x = 0; x < 16; ++x) o[mt][x] *= alpha;

    // ---- O^T += V^T P^T; the A operand reads V^T at the keys the B registers hold:
    //      elements 0..3 <-> keys 16t + 4g + 0..3, elements 4..7 <-> keys 16t + 8 + 4g + 0..3
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int kk = kb * 32 + 16 * t + 4 * g;
#pragma unroll
        for (int mt = 0; mt < DMT; ++mt) {
          const T *vrow = &lds_v[(mt * 32 + r) * VPITCH + kk];
          const uint2 lo = *reinterpret_cast<const uint2 *>(vrow);
          const uint2 hi = *reinterpret_cast<const uint2 *>(vrow + 8);
          M::step(make_uint4(lo.x, lo.y, hi.x, hi.y), pf[kb][t], o[mt]);
        }
      }
    lds_barrier();  // tiles are consumed before the next ones are written
  }

  // ---- normalise and store: register 4j+i of tile mt holds channel 32mt + 8j + 4g + i of this lane's query
  if (!q_valid) return;
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  T *crow = cbase + (int64_t)q * fa.c_ss;
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = mt * 32 + 8 * j + 4 * g;
      if (d < a.D) {
        Pack<T, 4> pk;
#pragma unroll
        for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(o[mt][4 * j + i] * inv);
        store_pack<T, 4>(crow + d, pk);
      }
    }
}

template <int DT>
static int launch_fused(FusedArgs &fa, hipStream_t s) {
  const AttnArgs &a = fa.base;
  const unsigned grid = (unsigned)(ceil_div(a.units, kXcds) * kXcds * a.ntq);
  if (a.D <= 64) attn_fused_kernel<DT, 64><<<grid, kBlock, 0, s>>>(fa);
  else attn_fused_kernel<DT, 128><<<grid, kBlock, 0, s>>>(fa);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // namespace en

extern "C" int en_attn_fused(const void *q, const void *k, const void *v, void *ctx, const int32_t *k_lens,
                             const int32_t *q_lens, int batch, int head_num, int q_seq_len, int k_seq_len,
                             int size_per_head, const int64_t *q_strides, const int64_t *k_strides,
                             const int64_t *v_strides, const int64_t *c_strides, const int32_t *q_row_offsets,
                             const int32_t *k_row_offsets, float scale, int causal, int dtype, en_stream_t stream) {
  using namespace en;
  if (!q || !k || !v || !ctx || !k_lens || !q_strides || !k_strides || !v_strides || !c_strides) return EN_ERR_NULL;
  if (batch < 1 || head_num < 1 || q_seq_len < 1 || k_seq_len < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  if (dtype != EN_F16 && dtype != EN_BF16) return EN_ERR_DTYPE;
  if (size_per_head > 128 || (size_per_head % 8) != 0) return EN_ERR_UNSUPPORTED;
  if (!(scale >= 0.f)) return EN_ERR_UNSUPPORTED;
  if ((int64_t)batch * head_num > INT32_MAX / 64) return EN_ERR_SHAPE;
  if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(v, 16) || !aligned_to(ctx, 8)) return EN_ERR_ALIGN;
  for (int i = 0; i < 3; ++i) {
    if ((q_strides[i] % 8) || (k_strides[i] % 8) || (v_strides[i] % 8) || (c_strides[i] % 4)) return EN_ERR_ALIGN;
    if (q_strides[i] < 0 || k_strides[i] < 0 || v_strides[i] < 0 || c_strides[i] < 0) return EN_ERR_UNSUPPORTED;
  }
  if ((int64_t)q_seq_len * q_strides[2] * 2 >= (1ll << 31) || (int64_t)k_seq_len * k_strides[2] * 2 >= (1ll << 31) ||
      (int64_t)k_seq_len * v_strides[2] * 2 >= (1ll << 31))
    return EN_ERR_UNSUPPORTED;
  FusedArgs fa{};
  AttnArgs &a = fa.base;
  a.a_ptr = q; a.b_ptr = k; a.out = ctx; a.k_lens = k_lens; a.q_lens = q_lens;
  a.B = batch; a.H = head_num; a.Sq = q_seq_len; a.Sk = k_seq_len; a.D = size_per_head;
  a.q_sb = q_strides[0]; a.q_sh = q_strides[1]; a.q_ss = q_strides[2];
  a.k_sb = k_strides[0]; a.k_sh = k_strides[1]; a.k_ss = k_strides[2];
  a.alpha = 1.f; a.causal = causal ? 1 : 0;
  a.ntq = (int)ceil_div(q_seq_len, kQTile);
  a.units = batch * head_num;
  fa.v = v;
  fa.v_sb = v_strides[0]; fa.v_sh = v_strides[1]; fa.v_ss = v_strides[2];
  fa.c_sb = c_strides[0]; fa.c_sh = c_strides[1]; fa.c_ss = c_strides[2];
  fa.q_row0 = q_row_offsets; fa.k_row0 = k_row_offsets;
  fa.scale = scale;
  hipStream_t s = (hipStream_t)stream;
  return dtype == EN_F16 ? launch_fused<EN_F16>(fa, s) : launch_fused<EN_BF16>(fa, s);
}
