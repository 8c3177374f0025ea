// Fused attention with 64 queries per wave: the form of fused.hip for long sequences and heads of 65..128
// channels.
//
//   ctx = softmax(scale * Q K^T, causal / key-padding mask) V
//
// Workgroup: 4 waves, one tile of 256 query rows of one (batch, head); wave w owns query rows 64w..64w+63 as two
// blocks of 32 (lane r of either half of the wave holds query 32 qb + r of block qb) and every channel.  Against
// the 32-query wave of fused.hip every K fragment read from LDS feeds two MFMAs (one per query block) and so does
// every V^T fragment, every K / V tile fetched into LDS serves 256 queries instead of 128, and a tile costs one
// barrier per 64 MFMAs of a wave instead of two per 32: LDS fragment reads, tile loads and barriers per FLOP are
// all halved.  The price is registers: 128 accumulators for O^T (64 queries x 128 channels), 64 for the Q fragments,
// so the scores exist 32 keys at a time (32 registers for both query blocks) and a wave runs at two per SIMD.
//
// Per 64-key tile, for each of its two 32-key blocks kb:
//   S^T = K Q^T      A = the block's K rows from LDS (read once), B = Q fragments of block 0, then of block 1.
//   online softmax   one query per lane and block: in-lane reductions plus one exchange between the wave's halves;
//                    running maximum moved lazily (only when it grows by more than 2^8 after scaling).
//   O^T += V^T P^T   A = V^T by the transposing LDS read (read once), B = the probabilities straight out of the
//                    S^T accumulators of block 0, then of block 1.
//
// K and V each have two buffers and are a whole tile ahead (64 KB of LDS, two workgroups per CU): tile kt + 1 is
// sent for right behind the barrier that publishes tile kt, so a tile has the time of a whole tile's arithmetic
// to arrive and the loop has one barrier per tile.  Tiles, Q rows and the output tile all travel as whole rows
// (memory straight into LDS; output staged through LDS), with the XOR-swizzled slots of fused.hip.
#include "fused_common.hip.h"

namespace en {

#ifndef EN_WIDE_WPE
#define EN_WIDE_WPE 2
#endif
template <int DT>
__global__ __launch_bounds__(kBlock, EN_WIDE_WPE) void attn_fused_wide_kernel(FusedArgs fa) {
  static_assert(DT != EN_F32, "the fused kernel is built for 16-bit storage");
  typedef Elem<DT> E;
  typedef typename E::T T;
  typedef Mma<DT> M;
  const AttnArgs &a = fa.base;
  constexpr int DP = 128;
  constexpr int EPV = 8;
  constexpr int BK = 64;                         // keys per tile
  constexpr int KB = BK / 32;                    // 32-key blocks per tile
  constexpr int NVS = DP / 16;                   // MFMA steps over the head dim
  constexpr int DMT = DP / 32;                   // 32-channel MFMA tiles of the output
  constexpr int ROW = DP;                        // LDS pitch of a K or V row (elements)
  constexpr int ROWB = ROW * 2;                  // ... in bytes
  constexpr int KVEC_ROW = DP / EPV;             // 16-byte slots per row
  constexpr int KLOADS = BK * KVEC_ROW / kBlock; // direct-load instructions per wave and tile, for each of K and V
  constexpr int QB = 2;                          // 32-query blocks per wave
  constexpr float kLog2e = 1.4426950408889634f;
  __shared__ __attribute__((aligned(16))) T lds_k[2][BK * ROW];
  __shared__ __attribute__((aligned(16))) T lds_v[2][BK * ROW];

  int unit, qi;
  if (!map_block(a, unit, qi)) return;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
  const int q0 = qi * kWideQTile;
  if (q0 >= ql) return;
  const int nk = tile_key_extent(a, min(q0 + kWideQTile, ql) - 1, kl, ql);
  const int nkt = (nk + BK - 1) / BK;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  // largest extent among the wave's 64 queries and smallest among them (wave-uniform): key blocks from the
  // largest on hold nothing for this wave, key blocks below the smallest need no masking
  const int q_first = q0 + wave * 64;
  const int vis_min = (q_first + 63 < ql) ? (a.causal ? min(kl, q_first + (kl - ql) + 1) : kl) : 0;
  const int vis_max = (q_first < ql) ? (a.causal ? min(kl, min(q_first + 63, ql - 1) + (kl - ql) + 1) : kl) : 0;

  const int64_t qr = fa.q_row0 ? fa.q_row0[b] : 0, kr = fa.k_row0 ? fa.k_row0[b] : 0;
  const T *qbase = reinterpret_cast<const T *>(a.a_ptr) + (int64_t)b * a.q_sb + qr * a.q_ss + (int64_t)h * a.q_sh;
  const T *kbase = reinterpret_cast<const T *>(a.b_ptr) + (int64_t)b * a.k_sb + kr * a.k_ss + (int64_t)h * a.k_sh;
  const T *vbase = reinterpret_cast<const T *>(fa.v) + (int64_t)b * fa.v_sb + kr * fa.v_ss + (int64_t)h * fa.v_sh;
  T *cbase = reinterpret_cast<T *>(a.out) + (int64_t)b * fa.c_sb + qr * fa.c_ss + (int64_t)h * fa.c_sh;

  // ---- K / V tiles: as in fused.hip.  One direct load of a wave fills 1 KB of LDS (four rows of 16 slots); slot c
  // of K row r holds chunk c ^ (r & 15), slot c of V key k holds chunk c ^ 4 (k & 3).
  const uint32_t k_bytes = kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * E::kSize) : 0u;
  const uint32_t v_bytes = kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * fa.v_ss + a.D) * E::kSize) : 0u;
  const desc_t k_desc = make_desc(kbase, k_bytes);
  const desc_t v_desc = make_desc(vbase, v_bytes);
  const uint32_t k_row_bytes = (uint32_t)(a.k_ss * E::kSize), v_row_bytes = (uint32_t)(fa.v_ss * E::kSize);
  constexpr int RPL = kWave / KVEC_ROW;          // rows one direct load of a wave covers (4)
  uint32_t k_off, v_off;
  {
    const int ld_row = wave * RPL + lane / KVEC_ROW, ld_slot = lane % KVEC_ROW;
    const int k_c = ld_slot ^ (ld_row & 15);
    const int v_c = ld_slot ^ (4 * (ld_row & 3));
    k_off = (k_c * EPV < a.D) ? ld_row * k_row_bytes + k_c * EPV * E::kSize : kOutOfRange;
    v_off = (v_c * EPV < a.D) ? ld_row * v_row_bytes + v_c * EPV * E::kSize : kOutOfRange;
  }
  auto fetch_kv = [&](int buf) {
    const uint32_t k_lds = lds_address(lds_k[buf]) + wave * kWave * 16;
    const uint32_t v_lds = lds_address(lds_v[buf]) + wave * kWave * 16;
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) buffer_load16_to_lds(k_desc, k_lds + i * kBlock * 16, k_off + i * (kBlock / KVEC_ROW) * k_row_bytes);
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) buffer_load16_to_lds(v_desc, v_lds + i * kBlock * 16, v_off + i * (kBlock / KVEC_ROW) * v_row_bytes);
    k_off += BK * k_row_bytes;
    v_off += BK * v_row_bytes;
  };
  fetch_kv(0);

  // ---- Q fragments (B operand of S^T = K Q^T), held in registers: this lane's query row of each block, 8 channels
  // per step.  The wave's 64 rows come in as whole rows, memory straight into LDS, 32 rows at a time through a
  // region of its own in the buffers that are idle until the key loop starts (second K buffer: waves 0 and 1,
  // second V buffer: waves 2 and 3), chunks in the K tile's swizzled slots; each lane then reads its own row's chunks.
  uint4 qf[QB][NVS];
  {
    T *q_stage = (wave < 2 ? lds_k[1] : lds_v[1]) + (wave & 1) * 32 * ROW;
    const desc_t q_desc = make_desc(qbase, (uint32_t)(((int64_t)(ql - 1) * a.q_ss + a.D) * E::kSize));
    const int row = lane / KVEC_ROW, slot = lane % KVEC_ROW;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
      for (int n = 0; n < 32 / RPL; ++n) {
        const int rr = n * RPL + row;               // row of the block's 32
        const int c = slot ^ (rr & 15);
        const int qq = q_first + 32 * qb + rr;
        const uint32_t off = (uint32_t)(((int64_t)qq * a.q_ss + c * EPV) * E::kSize);
        buffer_load16_to_lds(q_desc, lds_address(q_stage) + n * kWave * 16, (qq < ql && c * EPV < a.D) ? off : kOutOfRange);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // the block's rows (and tile 0) have landed
#pragma unroll
      for (int vs = 0; vs < NVS; ++vs)
        qf[qb][vs] = *reinterpret_cast<const uint4 *>(&q_stage[r * ROW + (((2 * vs + g) ^ (r & 15)) * EPV)]);
      // the reads complete before the next block's rows (or, behind the loop's first barrier, tile 1) overwrite them
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
  }

  // fragment addresses (bytes into a tile buffer).  K: row 32 kb + r, chunk 2 vs + g.  V (transposing read): lane j
  // of a 16-lane group points at key j / 4 of the group's four keys and at channels 4 (j % 4) .. + 3 of the group's
  // sixteen; the read hands lane i of the group channel i of those sixteen at the four keys.
  const int ksw = r & 15;
  const int tj = lane & 15, tg = (lane >> 4) & 1;
  // byte offset of this lane's read for channel tile mt: v_frag ^ (64 mt) (bits 6 and 7 hold the swizzled tile index)
  const uint32_t v_frag = (uint32_t)((4 * g + (tj >> 2)) * ROWB + (2 * tg + ((tj >> 1) & 1)) * 16 + (tj & 1) * 8) ^ (uint32_t)(64 * (tj >> 2));

  floatx16 o[QB][DMT];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
      for (int x = 0; x < 16; ++x) o[qb][mt][x] = 0.f;
  float m_run[QB] = {-INFINITY, -INFINITY}, l_run[QB] = {0.f, 0.f};
  const float c_exp = fa.scale * kLog2e;
  const float lazy_gap = 8.0f / c_exp;

  for (int kt = 0; kt < nkt; ++kt) {
    // tile kt was sent for a whole tile ago; the barrier publishes every wave's share of it and tells that all
    // waves have left tile kt - 1, whose buffers the loads of tile kt + 1 now overwrite
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    fetch_kv((kt + 1) & 1);                      // past the end: out of range, zeros, no traffic
    const char *ksrc = reinterpret_cast<const char *>(lds_k[kt & 1]);
    const char *vsrc = reinterpret_cast<const char *>(lds_v[kt & 1]);

#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int k0 = kt * BK + kb * 32;
      if (k0 >= vis_max) break;                  // wave-uniform: later key blocks are masked for all of this wave's queries

      // ---- S^T = K Q^T for both query blocks; the K fragments are read a step ahead of the MFMAs
      floatx16 s[QB];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int x = 0; x < 16; ++x) s[qb][x] = 0.f;
      {
        const char *krow = ksrc + (kb * 32 + r) * ROWB;
        uint4 kf[2];
        kf[0] = *reinterpret_cast<const uint4 *>(krow + ((g ^ ksw) * 16));
#pragma unroll
        for (int vs = 0; vs < NVS; ++vs) {
          if (vs + 1 < NVS) kf[(vs + 1) & 1] = *reinterpret_cast<const uint4 *>(krow + (((2 * (vs + 1) + g) ^ ksw) * 16));
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) M::step(kf[vs & 1], qf[qb][vs], s[qb]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }

      // ---- mask + online softmax; register 4j+i of a block holds key k0 + 8j + 4g + i
      float m_tile[QB];
      if (k0 + 32 <= vis_min) {                  // whole key block visible to every query of this wave
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          float m = fmaxf(s[qb][0], s[qb][1]);
#pragma unroll
          for (int x = 2; x < 16; x += 2) m = fmaxf(fmaxf(m, s[qb][x]), s[qb][x + 1]);
          m_tile[qb] = m;
        }
      } else {
        const int l = lane_now();
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const int ql_ = q_first + 32 * qb + (l & 31);
          const int vis_l = (ql_ < ql) ? (a.causal ? min(kl, ql_ + (kl - ql) + 1) : kl) : 0;
          const int lim = vis_l - k0 - 4 * (l >> 5);   // register x is visible iff 8(x/4) + x%4 < lim
          float m = -INFINITY;
#pragma unroll
          for (int x = 0; x < 16; ++x) {
            const float v = (8 * (x >> 2) + (x & 3) < lim) ? s[qb][x] : -INFINITY;
            s[qb][x] = v;
            m = fmaxf(m, v);
          }
          m_tile[qb] = m;
        }
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {          // the other half of a query's keys sits in lane r + 32
        float lo, hi;
        halves_of(m_tile[qb], lo, hi);
        m_tile[qb] = fmaxf(lo, hi);
      }
      if (__builtin_amdgcn_ballot_w64(m_tile[0] - lazy_gap > m_run[0] || m_tile[1] - lazy_gap > m_run[1]) != 0) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const float m_new = fmaxf(m_run[qb], m_tile[qb]);
          const float alpha = (m_run[qb] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run[qb] - m_new) * c_exp);
          l_run[qb] *= alpha;
#pragma unroll
          for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
            for (int x = 0; x < 16; ++x) o[qb][mt][x] *= alpha;
          m_run[qb] = m_new;
        }
      }
      uint4 pf[QB][2];                           // B operands of the second MFMA: 16 keys per vector
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const float moff = (m_run[qb] == -INFINITY) ? 0.f : -m_run[qb] * c_exp;
        float l_tile = 0.f;
        Pack<T, EPV> pk[2];
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          const float p = __builtin_amdgcn_exp2f(fmaf(s[qb][x], c_exp, moff));   // exp2(-inf) = 0: masked keys
          l_tile += p;
          pk[x >> 3].v[x & 7] = E::from_float(p);
        }
        pf[qb][0] = __builtin_bit_cast(uint4, pk[0]);
        pf[qb][1] = __builtin_bit_cast(uint4, pk[1]);
        float lo, hi;
        halves_of(l_tile, lo, hi);
        l_run[qb] += lo + hi;
      }

      // ---- O^T += V^T P^T for both query blocks; the A operand reads V at the keys the B registers hold:
      //      elements 0..3 <-> keys 16 gi + 4g + 0..3, elements 4..7 <-> keys 16 gi + 8 + 4g + 0..3 of the block
      {
        const char *vblk = vsrc + kb * 32 * ROWB;
        auto load_va = [&](int idx) -> uint4 {    // idx = gi * DMT + mt
          const char *vt = vblk + (idx / DMT) * 16 * ROWB + (v_frag ^ (uint32_t)(64 * (idx % DMT)));
          const uint2 lo = lds_read_tr16(vt);
          const uint2 hi = lds_read_tr16(vt + 8 * ROWB);
          return make_uint4(lo.x, lo.y, hi.x, hi.y);
        };
        uint4 va[2];
        va[0] = load_va(0);
#pragma unroll
        for (int idx = 0; idx < 2 * DMT; ++idx) {
          if (idx + 1 < 2 * DMT) va[(idx + 1) & 1] = load_va(idx + 1);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) M::step(va[idx & 1], pf[qb][idx / DMT], o[qb][idx % DMT]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }
  // every wave has left the last tile before its buffers take the output
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  lds_barrier();

  // ---- normalise and store: register 4j+i of tile mt holds channel 32mt + 8j + 4g + i of this lane's query
  const int lane_e = lane_now(), r_e = lane_e & 31, g_e = lane_e >> 5;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float inv = l_run[qb] > 0.f ? 1.0f / l_run[qb] : 0.f;
    const int qblk = q_first + 32 * qb;
    if (fa.c_vec16) {
      // through LDS (each wave has 8 KB of the K buffers to itself) the block leaves as whole rows: 16 bytes per
      // lane, four rows per instruction.  Chunk c of row r sits in slot c ^ (r % 16).
      char *stage = reinterpret_cast<char *>(&lds_k[0][0]) + wave * 32 * ROWB;
#pragma unroll
      for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          Pack<T, 4> pk;
#pragma unroll
          for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(o[qb][mt][4 * j + i] * inv);
          const int c = 4 * mt + j;
          *reinterpret_cast<Pack<T, 4> *>(stage + r_e * ROWB + ((c ^ (r_e & 15)) * 16) + g_e * 8) = pk;
        }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes, before its lanes read each other's
#pragma unroll
      for (int i = 0; i < 32 / RPL; ++i) {
        const int row = i * RPL + lane_e / KVEC_ROW, c = lane_e % KVEC_ROW;
        const uint4 v = *reinterpret_cast<const uint4 *>(stage + row * ROWB + ((c ^ (row & 15)) * 16));
        const int qrow = qblk + row;
        if (qrow < ql && c * EPV < a.D) *reinterpret_cast<uint4 *>(cbase + (int64_t)qrow * fa.c_ss + c * EPV) = v;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the reads, before the next block's writes
    } else {
      const int q_e = qblk + r_e;
      if (q_e < ql) {
        T *crow = cbase + (int64_t)q_e * fa.c_ss;
#pragma unroll
        for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int d = mt * 32 + 8 * j + 4 * g_e;
            if (d < a.D) {
              Pack<T, 4> pk;
#pragma unroll
              for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(o[qb][mt][4 * j + i] * inv);
              store_pack<T, 4>(crow + d, pk);
            }
          }
      }
    }
  }
}

int launch_fused_wide(int dtype, FusedArgs &fa, hipStream_t s) {
  const AttnArgs &a = fa.base;
  const unsigned grid = (unsigned)(ceil_div(a.units, kXcds) * kXcds * a.ntq);
  if (dtype == EN_F16) attn_fused_wide_kernel<EN_F16><<<grid, kBlock, 0, s>>>(fa);
  else attn_fused_wide_kernel<EN_BF16><<<grid, kBlock, 0, s>>>(fa);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // namespace en
