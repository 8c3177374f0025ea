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
//   O^T += V^T P^T   A = V^T, read out of the row-major V tile with the LDS
//                    transposing read (four keys of one channel per lane and
//                    instruction), B = the probabilities straight out of the
//                    S^T accumulators, rounded to the storage type: a lane's
//                    registers (j, i) hold keys 8j + 4g + i, and the A operand
//                    simply reads V at those same keys, so P never touches LDS.
//
// K/V tiles travel from memory straight into LDS (bounds-checked loads that
// write LDS): no registers hold a tile in flight and no instruction copies
// one.  Rows keep their 16-byte chunks in XOR-swizzled slots so that both kinds
// of fragment read are free of bank conflicts.  K has two buffers and is a tile
// ahead; V has one buffer, is sent for at the top of its own tile and arrives
// behind the score and softmax work: 48 KB of LDS per workgroup, so that three
// workgroups fit a CU.  The barriers order LDS only, as in the unfused kernels.
//
// Everything that crosses the memory interface does so as whole rows: the K and
// V tiles, the workgroup's Q rows (loaded straight into the buffers that are
// idle before the key loop, each lane then reads its fragments from LDS) and the
// output tile (written to the K buffers behind the loop's last barrier, stored
// 16 bytes per lane).  A lane that fetches or stores pieces of a row of its own
// makes every instruction touch 32 rows, and the queue of the address unit then
// stands full and holds back the tile loads of every wave on the CU.
#include "fused_common.hip.h"

namespace en {

template <int DT, int DP>
__global__ __launch_bounds__(kBlock, 3) void attn_fused_kernel(FusedArgs fa) {
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
  constexpr int ROW = DP;                        // LDS pitch of a K or V row: tiles are written by direct loads, unpadded
  constexpr int KVEC_ROW = DP / EPV;             // 16-byte slots per row
  constexpr int KLOADS = BK * KVEC_ROW / kBlock; // direct-load instructions per wave and tile, for each of K and V
  constexpr float kLog2e = 1.4426950408889634f;
  static_assert(DP == 64 || DP == 128, "swizzles are written for 8 or 16 slots per row");
  static_assert(BK * KVEC_ROW % kBlock == 0, "tiles must divide over the block");
  __shared__ __attribute__((aligned(16))) T lds_k[2][BK * ROW];
  __shared__ __attribute__((aligned(16))) T lds_v[BK * ROW];

  int unit, qi;
  if (!map_block(a, unit, qi)) return;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
#ifdef EN_FUSED_START_ANCHORED
  const int q0 = qi * kQTile;
  if (q0 >= ql) return;
#else
  // The query tiles of a sequence are laid from its END: tile i of n covers rows ql - (n - i) * 128 .. and the ragged
  // tile is the first one (rows below 0 do not exist), whose walk over the keys is the shortest under a causal mask.
  // Laid from the start, the ragged tile would be the last one: a few rows holding a slot for the longest walk.
  const int ntl = (ql + kQTile - 1) / kQTile;
  if (qi >= ntl) return;
  const int q0 = ql - (ntl - qi) * kQTile;
#endif
  const int nk = tile_key_extent(a, min(q0 + kQTile, ql) - 1, kl, ql);
  const int nkt = (nk + BK - 1) / BK;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  // smallest and largest extent among the wave's 32 queries (wave-uniform): tiles below the
  // smallest need no masking, tiles from the largest on hold nothing for this wave
  const int q_first = q0 + wave * 32;
  const int vis_min = (q_first + 31 < ql) ? (a.causal ? min(kl, q_first + (kl - ql) + 1) : kl) : 0;
  const int vis_max = (q_first < ql && q_first + 31 >= 0) ? (a.causal ? min(kl, min(q_first + 31, ql - 1) + (kl - ql) + 1) : kl) : 0;

  // batch base: b * batch stride (padded layout) or first-row * row stride (packed layout)
  const int64_t qr = fa.q_row0 ? fa.q_row0[b] : 0, kr = fa.k_row0 ? fa.k_row0[b] : 0;
  const T *qbase = reinterpret_cast<const T *>(a.a_ptr) + (int64_t)b * a.q_sb + qr * a.q_ss + (int64_t)h * a.q_sh;
  const T *kbase = reinterpret_cast<const T *>(a.b_ptr) + (int64_t)b * a.k_sb + kr * a.k_ss + (int64_t)h * a.k_sh;
  const T *vbase = reinterpret_cast<const T *>(fa.v) + (int64_t)b * fa.v_sb + kr * fa.v_ss + (int64_t)h * fa.v_sh;
  T *cbase = reinterpret_cast<T *>(a.out) + (int64_t)b * fa.c_sb + qr * fa.c_ss + (int64_t)h * fa.c_sh;

  // Q fragments (B operand of S^T = K Q^T): this lane's query row, 8 channels per step.  The wave's 32 rows come in
  // as whole rows, memory straight into LDS (the second K buffer and the V buffer are idle until the key loop starts;
  // waves 0 and 1 take the one, waves 2 and 3 the other, 32 rows each), chunks in the K tile's swizzled slots, and
  // each lane then reads its own row's chunks: sixteen-byte pieces fetched by every lane from a row of its own
  // kept the address unit busy with 32 rows per instruction.
  uint4 qf[NVS];
  T *q_stage = (wave < 2 ? lds_k[1] : lds_v) + (wave & 1) * 32 * ROW;
  {
    const desc_t q_desc = make_desc(qbase, (uint32_t)(((int64_t)(ql - 1) * a.q_ss + a.D) * E::kSize));
    constexpr int RPLQ = kWave / KVEC_ROW;         // rows one direct load of a wave covers
    const int row = lane / KVEC_ROW, slot = lane % KVEC_ROW;
#pragma unroll
    for (int n = 0; n < 32 / RPLQ; ++n) {
      const int rr = n * RPLQ + row;               // row of the wave's 32
      const int c = slot ^ (DP == 128 ? (rr & 15) : ((rr >> 1) & 7));
      const int qq = q0 + wave * 32 + rr;
      const uint32_t off = (uint32_t)(((int64_t)qq * a.q_ss + c * EPV) * E::kSize);
      buffer_load16_to_lds(q_desc, lds_address(q_stage) + n * kWave * 16, ((unsigned)qq < (unsigned)ql && c * EPV < a.D) ? off : kOutOfRange);
    }
  }

  // K / V tiles: the descriptors end with the last valid key, so rows past it (and whole tiles past the last
  // one) arrive as zeros with no traffic and no branches.  One direct load of a wave fills 1 KB of LDS, lane i
  // the 16 bytes at 16 i: that is slot i % KVEC_ROW of tile row (64 / KVEC_ROW) * (4 n + wave) + i / KVEC_ROW
  // for the wave's n-th load.  Which 16-byte chunk of the row a slot holds is the lane's choice of offset:
  //   K: slot c of row r holds chunk c ^ kswz(r), kswz = r & 15 (16 slots) or (r >> 1) & 7 (8 slots): the
  //      128-bit fragment reads of 16 consecutive rows at one chunk then cover all 64 banks once;
  //   V: slot c of key k holds chunk c ^ vswz(k), vswz = 4 (k & 3) (16 slots) or 4 ((k >> 1) & 1) (8 slots):
  //      a transposing read takes 64 bytes from each of four consecutive keys, which the swizzle spreads over
  //      the four quarters of the banks.
  // Both swizzles depend on the row only through bits the lane's position fixes, so each lane keeps one byte
  // offset per operand and advances it by a tile per load; lanes whose chunk lies past the head size sit at an
  // offset that stays out of range.
  const uint32_t k_bytes = kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * E::kSize) : 0u;
  const uint32_t v_bytes = kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * fa.v_ss + a.D) * E::kSize) : 0u;
  const desc_t k_desc = make_desc(kbase, k_bytes);
  const desc_t v_desc = make_desc(vbase, v_bytes);
  const uint32_t k_row_bytes = (uint32_t)(a.k_ss * E::kSize), v_row_bytes = (uint32_t)(fa.v_ss * E::kSize);
  constexpr int RPL = kWave / KVEC_ROW;          // rows one direct load of a wave covers
  const int ld_row = wave * RPL + lane / KVEC_ROW, ld_slot = lane % KVEC_ROW;
  const int k_c = ld_slot ^ (DP == 128 ? (ld_row & 15) : ((ld_row >> 1) & 7));
  const int v_c = ld_slot ^ (DP == 128 ? 4 * (ld_row & 3) : 4 * ((ld_row >> 1) & 1));
  uint32_t k_off = (k_c * EPV < a.D) ? ld_row * k_row_bytes + k_c * EPV * E::kSize : kOutOfRange;
  uint32_t v_off = (v_c * EPV < a.D) ? ld_row * v_row_bytes + v_c * EPV * E::kSize : kOutOfRange;
  auto fetch_k = [&](T *kdst) {
    const uint32_t k_lds = lds_address(kdst) + wave * kWave * 16;
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) buffer_load16_to_lds(k_desc, k_lds + i * kBlock * 16, k_off + i * (kBlock / KVEC_ROW) * k_row_bytes);
    k_off += BK * k_row_bytes;
  };
  auto fetch_v = [&]() {
    const uint32_t v_lds = lds_address(lds_v) + wave * kWave * 16;
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) buffer_load16_to_lds(v_desc, v_lds + i * kBlock * 16, v_off + i * (kBlock / KVEC_ROW) * v_row_bytes);
    v_off += BK * v_row_bytes;
  };
  // fragment addresses.  K: row 32 kb + r, chunk 2 vs + g.  V (transposing read): lane j of a 16-lane group
  // points at key j / 4 of the group's four keys and at channels 4 (j % 4) .. + 3 of the group's sixteen; the
  // read hands lane i of the group channel i of those sixteen at the four keys.
  const int ksw = DP == 128 ? (r & 15) : ((r >> 1) & 7);
  const int tj = lane & 15, tg = (lane >> 4) & 1;     // position in the 16-lane group; which half of a 32-channel tile
  const int vsw = DP == 128 ? (tj >> 2) : ((tj >> 3) & 1);
  uint32_t v_frag[DMT];                                // byte offset of this lane's read for channel tile mt, keys 4g + 0..3
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
    v_frag[mt] = (uint32_t)((4 * g + (tj >> 2)) * ROW * E::kSize + (4 * (mt ^ vsw) + 2 * tg + ((tj >> 1) & 1)) * 16 + (tj & 1) * 8);

  floatx16 o[DMT];
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
    for (int x = 0; x < 16; ++x) o[mt][x] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float c_exp = fa.scale * kLog2e;
  // The running maximum is only moved (and the accumulators rescaled) when some query's new
  // maximum exceeds it by more than 2^8 after scaling: until then probabilities are formed
  // against the older, slightly smaller maximum and stay below 2^8, well inside the 16-bit
  // range, and the final division by the row sum cancels the common factor.
  const float lazy_gap = 8.0f / c_exp;

  // K tile kt is read out of buffer kt & 1 while K tile kt + 1 travels into the other one; V tile kt is sent for
  // at the top of iteration kt (its buffer was in use until the barrier that ended iteration kt - 1) and waited
  // for between the softmax and the second contraction.  Two barriers per tile.
  fetch_k(lds_k[0]);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  {  // the wave's own rows have landed; the barrier below also keeps the tiles of the key loop off them until all have read
    const int qsw = DP == 128 ? (r & 15) : ((r >> 1) & 7);
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs)
      qf[vs] = *reinterpret_cast<const uint4 *>(&q_stage[r * ROW + (((2 * vs + g) ^ qsw) * EPV)]);
  }
  lds_barrier();

  for (int kt = 0; kt < nkt; ++kt) {
    const int k0 = kt * BK;
    const T *ksrc = lds_k[kt & 1];
    fetch_v();                                   // V tile kt
    fetch_k(lds_k[(kt + 1) & 1]);                // K tile kt + 1 (past the end: out of range, zeros, no traffic)
    uint4 pf[KB * 2];                            // B operands of the second MFMA: the probabilities of this tile
    const bool live = k0 < vis_max;              // wave-uniform: later tiles are masked for all of this wave's queries

    if (live) {
      // ---- S^T = K Q^T; the K fragments are read from LDS a step ahead of the MFMAs
      floatx16 s[KB];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int x = 0; x < 16; ++x) s[kb][x] = 0.f;
      {
        uint4 kf[2][KB];                             // fragments of the step after the one the MFMAs work on
        auto load_step = [&](int vs, uint4 (&dst)[KB]) {
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
            dst[kb] = *reinterpret_cast<const uint4 *>(&ksrc[(kb * 32 + r) * ROW + (((2 * vs + g) ^ ksw) * EPV)]);
        };
        load_step(0, kf[0]);
#pragma unroll
        for (int vs = 0; vs < NVS; ++vs) {
          if (vs + 1 < NVS) load_step(vs + 1, kf[(vs + 1) & 1]);
          __builtin_amdgcn_sched_barrier(0);         // keep the reads of the next step ahead of these MFMAs
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) M::step(kf[vs & 1][kb], qf[vs], s[kb]);
          __builtin_amdgcn_sched_barrier(0);
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
        // this lane's query and the keys it may see (k < vis_l), counted afresh: only the tiles on the diagonal come here
        const int l = lane_now(), ql_ = q0 + wave * 32 + (l & 31);
        const int vis_l = ((unsigned)ql_ < (unsigned)ql) ? (a.causal ? min(kl, ql_ + (kl - ql) + 1) : kl) : 0;
        const int lim = vis_l - k0 - 4 * (l >> 5);   // register (kb, x) is visible iff 32kb + 8(x/4) + x%4 < lim
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int x = 0; x < 16; ++x) {
            const float v = (kb * 32 + 8 * (x >> 2) + (x & 3) < lim) ? s[kb][x] : -INFINITY;
            s[kb][x] = v;
            m_tile = fmaxf(m_tile, v);
          }
      }
      {  // the other half of this query's keys sits in lane r + 32
        float lo, hi;
        halves_of(m_tile, lo, hi);
        m_tile = fmaxf(lo, hi);
      }
      if (__builtin_amdgcn_ballot_w64(m_tile - lazy_gap > m_run) != 0) {   // -inf + gap stays -inf: the first tile moves it
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
      for (int kb = 0; kb < KB; ++kb) {
        Pack<T, EPV> pk[2];
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          // exp2(-inf) is 0, so masked keys need no special case
          const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][x], c_exp, moff));
          l_tile += p;
          pk[x >> 3].v[x & 7] = E::from_float(p);                // group t = x/8 takes registers j = 2t, 2t+1
        }
        pf[2 * kb] = __builtin_bit_cast(uint4, pk[0]);
        pf[2 * kb + 1] = __builtin_bit_cast(uint4, pk[1]);
      }
      {
        float lo, hi;
        halves_of(l_tile, lo, hi);
        l_tile = lo + hi;
      }
      l_run += l_tile;

    }

    // V tile kt was sent for before K tile kt + 1 and the loads complete in order: it has landed once only the
    // K loads are outstanding; the barrier publishes every wave's share
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(KLOADS) : "memory");
    lds_barrier();

    if (live) {
      // ---- O^T += V^T P^T; the A operand reads V at the keys the B registers hold:
      //      elements 0..3 <-> keys 16gi + 4g + 0..3, elements 4..7 <-> keys 16gi + 8 + 4g + 0..3
      constexpr int NG = KB * 2;                      // groups of 16 keys
      uint4 va[2][DMT];
      auto load_group = [&](int gi, uint4 (&dst)[DMT]) {
        const char *vt = reinterpret_cast<const char *>(lds_v) + gi * 16 * ROW * E::kSize;
#pragma unroll
        for (int mt = 0; mt < DMT; ++mt) {
          const uint2 lo = lds_read_tr16(vt + v_frag[mt]);                          // keys 16 gi + 4 g + 0..3
          const uint2 hi = lds_read_tr16(vt + v_frag[mt] + 8 * ROW * E::kSize);     // keys 16 gi + 8 + 4 g + 0..3
          dst[mt] = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
      };
      load_group(0, va[0]);
#pragma unroll
      for (int gi = 0; gi < NG; ++gi) {
        if (gi + 1 < NG) load_group(gi + 1, va[(gi + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < DMT; ++mt) M::step(va[gi & 1][mt], pf[gi], o[mt]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // K tile kt + 1 has landed once none of this wave's loads is outstanding; the barrier publishes it and
    // frees the V buffer and the other K buffer
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
  }

  // ---- normalise and store: register 4j+i of tile mt holds channel 32mt + 8j + 4g + i of this lane's query
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  const int lane_e = lane_now(), r_e = lane_e & 31, g_e = lane_e >> 5;
  if (fa.c_vec16) {
    // A lane holds 8-byte pieces of its own row, 32 rows per store instruction; through LDS (the K buffers are free
    // behind the loop's last barrier, each wave takes the 32 rows' worth that is its own, so no barrier is needed)
    // the wave's tile leaves as whole rows: 16 bytes per lane, 64 / KVEC_ROW rows per instruction.  Chunk c of row r
    // sits in slot c ^ (r % KVEC_ROW): writes and reads both spread over all banks.
    char *stage = reinterpret_cast<char *>(&lds_k[0][0]) + wave * 32 * ROW * E::kSize;
#pragma unroll
    for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        Pack<T, 4> pk;
#pragma unroll
        for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(o[mt][4 * j + i] * inv);
        const int c = 4 * mt + j;
        *reinterpret_cast<Pack<T, 4> *>(stage + r_e * ROW * E::kSize + ((c ^ (r_e & (KVEC_ROW - 1))) * 16) + g_e * 8) = pk;
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes, before its lanes read each other's
    constexpr int RPI = kWave / KVEC_ROW;              // rows per store instruction
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
      const int row = i * RPI + lane_e / KVEC_ROW, c = lane_e % KVEC_ROW;
      const uint4 v = *reinterpret_cast<const uint4 *>(stage + row * ROW * E::kSize + ((c ^ (row & (KVEC_ROW - 1))) * 16));
      const int qrow = q0 + wave * 32 + row;
      if ((unsigned)qrow < (unsigned)ql && c * EPV < a.D) *reinterpret_cast<uint4 *>(cbase + (int64_t)qrow * fa.c_ss + c * EPV) = v;
    }
    return;
  }
  const int q_e = q0 + wave * 32 + r_e;
  if ((unsigned)q_e >= (unsigned)ql) return;
  T *crow = cbase + (int64_t)q_e * fa.c_ss;
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = mt * 32 + 8 * j + 4 * g_e;
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

extern "C" int en_attn_fused_query_tile(int q_seq_len, int k_seq_len, int size_per_head, int causal, int dtype) {
  // The 256-row tile (64 queries per wave, fused_wide.hip) halves the LDS reads, tile loads and barriers per FLOP
  // but runs two waves per SIMD instead of three, and measures slower on every shape tried (uniform 1024-key
  // rows, 64 heads: 778 against 906 TFLOP/s; ragged batches lose more, having fewer and longer workgroups):
  // never chosen by itself.
  (void)q_seq_len; (void)k_seq_len; (void)size_per_head; (void)causal;
  return dtype == EN_F32 ? 64 : en::kQTile;     // fp32: the kernel of fused_f32.hip, 64-row tiles
}

extern "C" int en_attn_fused(const void *q, const void *k, const void *v, void *ctx, const int32_t *k_lens,
                             const int32_t *q_lens, int batch, int head_num, int q_seq_len, int k_seq_len,
                             int size_per_head, const int64_t *q_strides, const int64_t *k_strides,
                             const int64_t *v_strides, const int64_t *c_strides, const int32_t *q_row_offsets,
                             const int32_t *k_row_offsets, float scale, int causal, int dtype,
                             const int32_t *tile_table, int query_tile, en_stream_t stream) {
  using namespace en;
  if (!q || !k || !v || !ctx || !k_lens || !q_strides || !k_strides || !v_strides || !c_strides) return EN_ERR_NULL;
  if (batch < 1 || head_num < 1 || q_seq_len < 1 || k_seq_len < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  if (dtype != EN_F16 && dtype != EN_BF16 && dtype != EN_F32) return EN_ERR_DTYPE;
  const bool f32 = dtype == EN_F32;
  const int es = f32 ? 4 : 2, epv = 16 / es;
  if (size_per_head > 128 || (size_per_head % epv) != 0) return EN_ERR_UNSUPPORTED;
  if (f32 && size_per_head > 64) return EN_ERR_UNSUPPORTED;   // the fp32 kernel is built for heads of up to 64 channels
  if (!(scale > 0.f)) return EN_ERR_UNSUPPORTED;  // masked scores are -inf; -inf * 0 would not stay masked
  if (query_tile == 0) query_tile = en_attn_fused_query_tile(q_seq_len, k_seq_len, size_per_head, causal, dtype);
  if (f32 ? query_tile != 64 : (query_tile != kQTile && query_tile != kWideQTile)) return EN_ERR_UNSUPPORTED;
  if (query_tile == kWideQTile && size_per_head <= 64) return EN_ERR_UNSUPPORTED;   // the 64-query wave is built for 65..128 channels
  if ((int64_t)batch * head_num > INT32_MAX / 64) return EN_ERR_SHAPE;
  if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(v, 16) || !aligned_to(ctx, 4 * es)) return EN_ERR_ALIGN;
  for (int i = 0; i < 3; ++i) {
    if ((q_strides[i] % epv) || (k_strides[i] % epv) || (v_strides[i] % epv) || (c_strides[i] % 4)) return EN_ERR_ALIGN;
    if (q_strides[i] < 0 || k_strides[i] < 0 || v_strides[i] < 0 || c_strides[i] < 0) return EN_ERR_UNSUPPORTED;
  }
  // 32-bit byte offsets, advanced a tile at a time up to two tiles past the end
  if ((int64_t)q_seq_len * q_strides[2] * es >= (1ll << 31) || ((int64_t)k_seq_len + 256) * k_strides[2] * es >= (1ll << 31) ||
      ((int64_t)k_seq_len + 256) * v_strides[2] * es >= (1ll << 31))
    return EN_ERR_UNSUPPORTED;
  if (f32 && tile_table) return EN_ERR_UNSUPPORTED;            // the table lists 128- or 256-row tiles; the fp32 kernel has 64-row ones
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
  fa.c_vec16 = aligned_to(ctx, 16) && (c_strides[0] % epv) == 0 && (c_strides[1] % epv) == 0 && (c_strides[2] % epv) == 0;
  if (tile_table && q_lens) return EN_ERR_UNSUPPORTED;      // the table lists the query tiles of min(k_lens, q_seq_len) rows
  a.tile_table = tile_table;
  fa.scale = scale;
  hipStream_t s = (hipStream_t)stream;
  if (f32) return launch_fused_f32(fa, s);
  if (query_tile == kWideQTile) {
    a.ntq = (int)ceil_div(q_seq_len, kWideQTile);
    return launch_fused_wide(dtype, fa, s);
  }
  return dtype == EN_F16 ? launch_fused<EN_F16>(fa, s) : launch_fused<EN_BF16>(fa, s);
}
