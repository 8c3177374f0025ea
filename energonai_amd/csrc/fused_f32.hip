// Fused attention for fp32 storage and heads of up to 64 channels (the BERT-base shape of the reference's CPU
// path, examples/bert/bert.py:108-119 in fp32): ctx = softmax(scale * Q K^T, mask) V in one kernel, no score
// tensor.  The 16-bit kernels of fused.hip are built around 16-bit operand vectors (probabilities as 16-bit B
// operands, the transposing LDS read); here everything is fp32 on the 32x32x2 MFMA.
//
// Workgroup: 4 waves, one tile of 64 query rows of one (batch, head).  Wave (wq, wk): query rows 32 wq .. + 31 and
// the keys 32 wk .. + 31 of every 64-key tile, so the two waves of a query half split the keys between them, each
// with its own running maximum, sum and output (online softmax over its own keys only: no exchange per tile);
// the pair is combined once, through LDS, at the end.  Small problems are what this kernel is for (fp32 batches are
// short), and they are bound by the length of a workgroup's dependent chain: half the keys per wave halve it, and
// 64-row tiles give twice the workgroups of the 128-row tiles of the 16-bit kernels.
//
//   S^T = K Q^T      A = the wave's 32 K rows from LDS, B = Q fragments in registers; one query per lane.
//   online softmax   as in fused.hip (in-lane reductions, one exchange between the wave's halves, lazy rescale).
//   O^T += V^T P^T   B = the probabilities as they sit in the S^T accumulators (fp32, no conversion): the MFMA step
//                    for register (j, i) contracts over the two keys 8j + i and 8j + 4 + i that the lane's two
//                    halves hold; A = V at those keys, one channel per lane, read from the row-major V tile.
#include "fused_common.hip.h"

namespace en {

constexpr int kF32QTile = 64;

template <int DP>
__global__ __launch_bounds__(kBlock) void attn_fused_f32_kernel(FusedArgs fa) {
  typedef float T;
  typedef Mma<EN_F32> M;
  const AttnArgs &a = fa.base;
  constexpr int EPV = 4;
  constexpr int BK = 64;                         // keys per tile (32 per wave)
  constexpr int NVS = DP / M::KPV;               // 128-bit steps over the head dim
  constexpr int DMT = DP / 32;                   // 32-channel MFMA tiles of the output
  constexpr int KP = DP + 4;                     // LDS pitch of a K row: 16-byte fragment reads of 32 rows spread over the banks
  constexpr int VP = DP + 8;                     // LDS pitch of a V row: the wave's halves read rows four keys apart, 4 VP = 32 (mod 64) banks
  constexpr int VEC_ROW = DP / EPV;
  constexpr int LOADS = BK * VEC_ROW / kBlock;   // 128-bit loads per lane and tile, for each of K and V
  constexpr float kLog2e = 1.4426950408889634f;
  static_assert(DP == 64, "pitches and the combine area are laid out for 64 channels");
  __shared__ __attribute__((aligned(16))) float lds_k[BK * KP];
  __shared__ __attribute__((aligned(16))) float lds_v[BK * VP];

  const int unit = blockIdx.y, qi = blockIdx.x;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
  const int q0 = qi * kF32QTile;
  if (q0 >= ql) return;
  const int nk = tile_key_extent(a, min(q0 + kF32QTile, ql) - 1, kl, ql);
  const int nkt = (nk + BK - 1) / BK;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int wq = wave & 1, wk = wave >> 1;
  const int q_first = q0 + wq * 32;
  const int q_lane = q_first + r;
  // keys this lane's query may see, and the wave's smallest and largest such extent
  const int vis_l = (q_lane < ql) ? (a.causal ? min(kl, q_lane + (kl - ql) + 1) : kl) : 0;
  const int vis_min = (q_first + 31 < ql) ? (a.causal ? min(kl, q_first + (kl - ql) + 1) : kl) : 0;
  const int vis_max = (q_first < ql) ? (a.causal ? min(kl, min(q_first + 31, ql - 1) + (kl - ql) + 1) : kl) : 0;

  const int64_t qr = fa.q_row0 ? fa.q_row0[b] : 0, kr = fa.k_row0 ? fa.k_row0[b] : 0;
  const T *qbase = reinterpret_cast<const T *>(a.a_ptr) + (int64_t)b * a.q_sb + qr * a.q_ss + (int64_t)h * a.q_sh;
  const T *kbase = reinterpret_cast<const T *>(a.b_ptr) + (int64_t)b * a.k_sb + kr * a.k_ss + (int64_t)h * a.k_sh;
  const T *vbase = reinterpret_cast<const T *>(fa.v) + (int64_t)b * fa.v_sb + kr * fa.v_ss + (int64_t)h * fa.v_sh;
  T *cbase = reinterpret_cast<T *>(a.out) + (int64_t)b * fa.c_sb + qr * fa.c_ss + (int64_t)h * fa.c_sh;

  // Q fragments: this lane's query row, four channels per step (rows past the last valid one are never stored)
  uint4 qf[NVS];
  {
    const T *qrow = qbase + (int64_t)min(q_lane, ql - 1) * a.q_ss;
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      const int d = M::k_of(vs, g, NVS);
      qf[vs] = (d < a.D) ? *reinterpret_cast<const uint4 *>(qrow + d) : zero4();
    }
  }

  // K / V tiles come through registers (bounds-checked: rows at or past the last key and channels past the head
  // size read as zeros) a tile ahead of the one being worked on
  const rsrc_t k_rsrc = make_rsrc(kbase, kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * 4) : 0u);
  const rsrc_t v_rsrc = make_rsrc(vbase, kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * fa.v_ss + a.D) * 4) : 0u);
  uint4 kreg[LOADS], vreg[LOADS];
  auto fetch = [&](int kt) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / VEC_ROW, c = v % VEC_ROW;
      const int key = kt * BK + row;
      const bool in = key < kl && c * EPV < a.D;
      kreg[i] = buffer_load16(k_rsrc, in ? (uint32_t)(((int64_t)key * a.k_ss + c * EPV) * 4) : kOutOfRange);
      vreg[i] = buffer_load16(v_rsrc, in ? (uint32_t)(((int64_t)key * fa.v_ss + c * EPV) * 4) : kOutOfRange);
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
  const float lazy_gap = 8.0f / c_exp;

  for (int kt = 0; kt < nkt; ++kt) {
    __syncthreads();                              // every wave has left the previous tile
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / VEC_ROW, c = v % VEC_ROW;
      *reinterpret_cast<uint4 *>(&lds_k[row * KP + c * EPV]) = kreg[i];
      *reinterpret_cast<uint4 *>(&lds_v[row * VP + c * EPV]) = vreg[i];
    }
    __syncthreads();
    if (kt + 1 < nkt) fetch(kt + 1);

    const int k0 = kt * BK + wk * 32;             // first key of this wave's block
    if (k0 >= vis_max) continue;                  // wave-uniform: nothing for this wave's queries here

    // ---- S^T = K Q^T
    floatx16 s;
#pragma unroll
    for (int x = 0; x < 16; ++x) s[x] = 0.f;
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      const uint4 kf = *reinterpret_cast<const uint4 *>(&lds_k[(wk * 32 + r) * KP + M::k_of(vs, g, NVS)]);
      M::step(kf, qf[vs], s);
    }

    // ---- mask + online softmax; register 4j+i holds key k0 + 8j + 4g + i of this lane's query
    float m_tile = -INFINITY;
    if (k0 + 32 <= vis_min) {
#pragma unroll
      for (int x = 0; x < 16; ++x) m_tile = fmaxf(m_tile, s[x]);
    } else {
      const int lim = vis_l - k0 - 4 * g;
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const float v = (8 * (x >> 2) + (x & 3) < lim) ? s[x] : -INFINITY;
        s[x] = v;
        m_tile = fmaxf(m_tile, v);
      }
    }
    {
      float lo, hi;
      halves_of(m_tile, lo, hi);
      m_tile = fmaxf(lo, hi);
    }
    if (__builtin_amdgcn_ballot_w64(m_tile - lazy_gap > m_run) != 0) {
      const float m_new = fmaxf(m_run, m_tile);
      const float alpha = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run - m_new) * c_exp);
      l_run *= alpha;
#pragma unroll
      for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
        for (int x = 0; x < 16; ++x) o[mt][x] *= alpha;
      m_run = m_new;
    }
    const float moff = (m_run == -INFINITY) ? 0.f : -m_run * c_exp;
    float l_tile = 0.f;
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      s[x] = __builtin_amdgcn_exp2f(fmaf(s[x], c_exp, moff));       // exp2(-inf) = 0: masked keys
      l_tile += s[x];
    }
    {
      float lo, hi;
      halves_of(l_tile, lo, hi);
      l_run += lo + hi;
    }

    // ---- O^T += V^T P^T: step (j, i) contracts over keys 8j + i (lanes 0..31) and 8j + 4 + i (lanes 32..63)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float *vrow = &lds_v[(wk * 32 + 8 * j + 4 * g) * VP + r];
      const uint4 pb = make_uint4(__float_as_uint(s[4 * j]), __float_as_uint(s[4 * j + 1]), __float_as_uint(s[4 * j + 2]),
                                  __float_as_uint(s[4 * j + 3]));
#pragma unroll
      for (int mt = 0; mt < DMT; ++mt) {
        const uint4 va = make_uint4(__float_as_uint(vrow[mt * 32]), __float_as_uint(vrow[VP + mt * 32]),
                                    __float_as_uint(vrow[2 * VP + mt * 32]), __float_as_uint(vrow[3 * VP + mt * 32]));
        M::step(va, pb, o[mt]);
      }
    }
  }

  // ---- combine the two waves of a query half (they saw disjoint keys), then normalise and store.
  // Wave (wq, 1) leaves maximum, sum and output in LDS, value by value with the lane fastest; wave (wq, 0) merges.
  __syncthreads();
  float *comb = lds_v + wq * (2 + DMT * 16) * kWave;      // 2 x 34 x 64 floats: inside the V tile's 64 x 72
  if (wk == 1) {
    comb[lane] = m_run;
    comb[kWave + lane] = l_run;
#pragma unroll
    for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
      for (int x = 0; x < 16; ++x) comb[(2 + mt * 16 + x) * kWave + lane] = o[mt][x];
  }
  __syncthreads();
  if (wk == 1) return;
  {
    const float m1 = comb[lane], l1 = comb[kWave + lane];
    const float m = fmaxf(m_run, m1);
    const float w0 = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run - m) * c_exp);
    const float w1 = (m1 == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m1 - m) * c_exp);
    const float l = l_run * w0 + l1 * w1;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (q_lane >= ql) return;
    T *crow = cbase + (int64_t)q_lane * fa.c_ss;
#pragma unroll
    for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = mt * 32 + 8 * j + 4 * g;
        float4 v;
        v.x = (o[mt][4 * j + 0] * w0 + comb[(2 + mt * 16 + 4 * j + 0) * kWave + lane] * w1) * inv;
        v.y = (o[mt][4 * j + 1] * w0 + comb[(2 + mt * 16 + 4 * j + 1) * kWave + lane] * w1) * inv;
        v.z = (o[mt][4 * j + 2] * w0 + comb[(2 + mt * 16 + 4 * j + 2) * kWave + lane] * w1) * inv;
        v.w = (o[mt][4 * j + 3] * w0 + comb[(2 + mt * 16 + 4 * j + 3) * kWave + lane] * w1) * inv;
        if (d < a.D) {
          if (fa.c_vec16) *reinterpret_cast<float4 *>(crow + d) = v;
          else { crow[d] = v.x; crow[d + 1] = v.y; crow[d + 2] = v.z; crow[d + 3] = v.w; }
        }
      }
  }
}

int launch_fused_f32(FusedArgs &fa, hipStream_t s) {
  const AttnArgs &a = fa.base;
  if (a.units > 65535) return EN_ERR_SHAPE;
  const dim3 grid((unsigned)ceil_div(a.Sq, kF32QTile), (unsigned)a.units, 1);
  attn_fused_f32_kernel<64><<<grid, kBlock, 0, s>>>(fa);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // namespace en
