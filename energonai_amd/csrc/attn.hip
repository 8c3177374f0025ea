// The two attention contractions on the padded [B,H,S,*] layout, restricted to
// the region softmax actually uses (valid query rows, visible keys):
//
//   scores = alpha * Q K^T      (attn_qk_strip_kernel; attn_qk_kernel for fp32 / unaligned rows)
//   ctx    = P V                (attn_pv_strip_kernel; attn_pv_kernel for fp32 / unaligned rows)
//
// All run on the 32x32 MFMA of gfx950 (32x32x16 for fp16/bf16, 32x32x2 for
// fp32) with fp32 accumulation over a 128-query tile per workgroup of four
// waves.  The strip kernels give each wave 32 queries and share only the K (or
// V^T) tile through LDS, one barrier per tile; the general kernels arrange the
// waves 2x2 over the tile and stage both operands and the result through LDS.
// In both, the streamed operand arrives by coalesced 128-bit loads and the
// next tile is prefetched into registers while the current one is multiplied.
//
// The MFMA result layout has lanes running along the N operand and registers
// along M, so the operands are assigned to make the registers run along the
// contiguous output dimension: QK^T computes (K)(Q)^T so that each lane owns
// four consecutive keys of one query row, PV computes (V^T)(P)^T so that each
// lane owns four consecutive channels of one query row.
//
// Work is laid out per (batch, head) "unit".  Workgroups are dealt to the eight
// XCDs round-robin by the hardware, so workgroup id -> (unit, query tile) is
// chosen such that all query tiles of a unit land on the same XCD and reuse
// that unit's K/V through one L2; within a unit the longest (bottom) causal
// query tiles are issued first.
#include "attn_common.hip.h"

namespace en {

// ===========================================================================
// scores = alpha * Q K^T
// ===========================================================================
template <int DT, int DP, bool VEC, bool STREAM>
__global__ __launch_bounds__(kBlock) void attn_qk_kernel(AttnArgs a) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  typedef Mma<DT> M;
  constexpr int EPV = M::EPV;
  constexpr int BN = (DT == EN_F32) ? 64 : 128;  // keys per tile
  constexpr int MT = BN / 64;                    // 32-key MFMA tiles per wave
  constexpr int NT = 2;                          // 32-query MFMA tiles per wave
  constexpr int NVS = DP / M::KPV;               // vector steps over the head dim
  constexpr int KPITCH = DP + EPV;               // LDS pitch of a K row, elements
  constexpr int CPITCH = BN + EPV;               // LDS pitch of a score row, elements
  constexpr int KVEC_ROW = DP / EPV;             // 128-bit vectors per K row
  constexpr int KLOADS = BN * KVEC_ROW / kBlock; // K vectors each lane stages per tile
  constexpr int CVEC_ROW = BN / EPV;
  constexpr int CSTORES = kQTile * CVEC_ROW / kBlock;
  constexpr int LDS_ELEMS = (BN * KPITCH > kQTile * CPITCH) ? BN * KPITCH : kQTile * CPITCH;
  static_assert(BN * KVEC_ROW % kBlock == 0 && kQTile * CVEC_ROW % kBlock == 0, "tile must divide over the block");
  __shared__ __attribute__((aligned(16))) T lds[LDS_ELEMS];

  int unit, qi;
  if (!map_block(a, unit, qi)) return;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
  const int q0 = qi * kQTile;
  if (q0 >= ql) return;
  const int nk = tile_key_extent(a, min(q0 + kQTile, ql) - 1, kl, ql);
  if (nk <= 0) return;
  const int nkt = (nk + BN - 1) / BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int wq = wave & 1, wk = wave >> 1;

  const T *qbase = reinterpret_cast<const T *>(a.a_ptr) + q_unit_offset(a, b, h);
  const T *kbase = reinterpret_cast<const T *>(a.b_ptr) + k_unit_offset(a, b, h);
  T *sbase = reinterpret_cast<T *>(a.out) + ((int64_t)unit * a.Sq) * a.Sk;

  // Q fragments stay in registers for the whole key loop.
  uint4 qf[NT][NVS];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int row = min(q0 + wq * 64 + nt * 32 + r, ql - 1);    // rows past the last valid one are never stored
    const T *qrow = qbase + (int64_t)row * a.q_ss;
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      const int d = M::k_of(vs, g, NVS);
      qf[nt][vs] = (d < a.D) ? *reinterpret_cast<const uint4 *>(qrow + d) : zero4();
    }
  }

  // K rows >= kl and channels >= D read as zero through the bounds check; a fetch past the
  // last tile is all out of range and costs no traffic, so the loop body has no branches.
  const rsrc_t k_rsrc = make_rsrc(kbase, (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * E::kSize));
  const rsrc_t s_rsrc = make_rsrc(sbase, (uint32_t)((int64_t)ql * a.Sk * E::kSize));
  uint4 kreg[KLOADS];
  auto fetch_k = [&](int kt) {
    const int k0 = kt * BN;
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / KVEC_ROW, c = v % KVEC_ROW;
      const int key = k0 + row;
      const uint32_t off = (uint32_t)(((int64_t)key * a.k_ss + c * EPV) * E::kSize);
      kreg[i] = buffer_load16(k_rsrc, (kt < nkt && key < kl && c * EPV < a.D) ? off : kOutOfRange);
    }
  };
  fetch_k(0);
  if constexpr (VEC) {
    // Out-of-range (dropped) stores that put the queue of outstanding memory operations into the same
    // shape on loop entry as on the back edge -- K loads, then score stores -- so the wait for the K
    // tile at the top of the loop is "all but the last CSTORES operations" and never drains the stores.
    asm volatile("" ::: "memory");  // keep the loads ahead of the stores in issue order
#pragma unroll
    for (int i = 0; i < CSTORES; ++i) buffer_store16(s_rsrc, kOutOfRange + 16u * i, zero4());  // distinct: not merged
    asm volatile("" ::: "memory");
  }

  for (int kt = 0; kt < nkt; ++kt) {
    const int k0 = kt * BN;
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / KVEC_ROW, c = v % KVEC_ROW;
      *reinterpret_cast<uint4 *>(&lds[row * KPITCH + c * EPV]) = kreg[i];
    }
    lds_barrier();
    fetch_k(kt + 1);

    floatx16 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int x = 0; x < 16; ++x) acc[mt][nt][x] = 0.f;

#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      uint4 kf[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        kf[mt] = *reinterpret_cast<const uint4 *>(&lds[(wk * (BN / 2) + mt * 32 + r) * KPITCH + M::k_of(vs, g, NVS)]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) M::step(kf[mt], qf[nt][vs], acc[mt][nt]);
    }
    lds_barrier();  // every wave is done reading K before the tile is reused for scores

    // accumulators -> LDS as a row-major [query][key] tile
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          Pack<T, 4> pk;
#pragma unroll
          for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(acc[mt][nt][4 * j + i] * a.alpha);
          const int qrow = wq * 64 + nt * 32 + r;
          const int kcol = wk * (BN / 2) + mt * 32 + 8 * j + 4 * g;
          store_pack<T, 4>(&lds[qrow * CPITCH + kcol], pk);
        }
    lds_barrier();

    // LDS -> HBM, whole rows of the tile as 128-bit stores
#pragma unroll
    for (int i = 0; i < CSTORES; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / CVEC_ROW, c = v % CVEC_ROW;
      const int q = q0 + row, k = k0 + c * EPV;
      const T *sp = &lds[row * CPITCH + c * EPV];
      // only vectors holding a key this row may see are written: nothing downstream reads the rest
      const int k_end = min(a.causal ? min(kl, q + (kl - ql) + 1) : kl, a.Sk);
      if constexpr (VEC) {  // rows >= ql fall outside the resource and are dropped by the bounds check
        const uint32_t off = (uint32_t)(((int64_t)q * a.Sk + k) * E::kSize);
        buffer_store16<STREAM ? 2 : 0>(s_rsrc, (k < k_end) ? off : kOutOfRange, *reinterpret_cast<const uint4 *>(sp));
      } else if (q < ql && k < k_end) {
        T *gp = sbase + (int64_t)q * a.Sk + k;
#pragma unroll
        for (int e = 0; e < EPV; ++e)
          if (k + e < a.Sk) gp[e] = sp[e];
      }
    }
    lds_barrier();  // scores leave LDS before the next K tile lands
  }
}

// ===========================================================================
// scores = alpha * Q K^T, 16-bit operands with 16-byte aligned score rows.
//
// Wave w of the workgroup owns queries 32w..32w+31 of a 128-query tile and computes
// S^T = K Q^T for 64 keys at a time: Q fragments stay in registers, K tiles are shared
// through LDS, double-buffered and fetched one tile ahead, which leaves ONE barrier per
// tile.  The 32x64 result of a wave is turned into row-major order through a strip of LDS
// that belongs to that wave alone (no workgroup barrier: a wave's LDS operations complete
// in order) and leaves as whole 128-byte row segments.  The loads of the next K tile and
// the stores of this tile are issued in the same iteration, before the only wait on the
// loads, so the stores are never waited for.
// ===========================================================================
template <int DT, int DP, bool STREAM>
__global__ __launch_bounds__(kBlock, 3) void attn_qk_strip_kernel(AttnArgs a) {
  static_assert(DT != EN_F32, "16-bit storage only");
  typedef Elem<DT> E;
  typedef typename E::T T;
  typedef Mma<DT> M;
  constexpr int EPV = 8;
  constexpr int BK = 64;                         // keys per tile
  constexpr int KB = BK / 32;                    // 32-key MFMA blocks per tile
  constexpr int NVS = DP / 16;                   // MFMA steps over the head dim
  constexpr int KPITCH = DP + EPV;               // LDS pitch of a K row
  constexpr int CPITCH = BK + EPV;               // LDS pitch of a score row in a wave's strip
  constexpr int KVEC_ROW = DP / EPV;
  constexpr int KLOADS = BK * KVEC_ROW / kBlock;
  constexpr int CVEC_ROW = BK / EPV;             // 128-bit vectors per score row of a tile
  constexpr int CSTORES = 32 * CVEC_ROW / kWave; // vectors each lane stores per tile
  static_assert(BK * KVEC_ROW % kBlock == 0, "K tile must divide over the block");
  constexpr bool DMA = (DP == 128);              // K tiles go from memory straight into LDS
  constexpr int KP = DMA ? DP : KPITCH;
  __shared__ __attribute__((aligned(16))) T lds_k[2][BK * KP];
  __shared__ __attribute__((aligned(16))) T lds_c[kBlock / kWave][32 * CPITCH];

  int unit, qi;
  if (!map_block(a, unit, qi)) return;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
  const int q0 = qi * kQTile;
  if (q0 >= ql) return;
  const int nk = tile_key_extent(a, min(q0 + kQTile, ql) - 1, kl, ql);
  if (nk <= 0) return;
  const int nkt = (nk + BK - 1) / BK;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int qw = q0 + wave * 32;                 // first query of this wave
  const int q = qw + r;                          // query whose scores this lane accumulates

  const T *qbase = reinterpret_cast<const T *>(a.a_ptr) + q_unit_offset(a, b, h);
  const T *kbase = reinterpret_cast<const T *>(a.b_ptr) + k_unit_offset(a, b, h);
  T *sbase = reinterpret_cast<T *>(a.out) + score_unit_offset<EPV>(a, unit);

  // Q fragments (B operand): this lane's query row, 8 channels per step; rows >= ql read as zero.  With direct loads
  // the wave's 32 rows come in as whole rows, memory straight into LDS (the second K buffer for waves 0 and 1, the
  // score strips, idle until the first tile's scores exist, for waves 2 and 3; 8 KB each), chunks in the K tile's
  // swizzled slots, and each lane then reads its own row's chunks from there: sixteen-byte pieces fetched by every
  // lane from a row of its own kept the address unit busy with 32 rows per instruction.
  uint4 qf[NVS];
  static_assert(!DMA || sizeof(lds_c) >= 2 * 32 * DP * sizeof(T), "two waves stage their Q rows in the score strips");
  T *q_stage = (wave < 2 ? lds_k[1] : &lds_c[0][0]) + (wave & 1) * 32 * DP;
  if constexpr (DMA) {
    const desc_t q_desc = make_desc(qbase, (uint32_t)(((int64_t)(ql - 1) * a.q_ss + a.D) * E::kSize));
    constexpr int RPLQ = kWave / KVEC_ROW;         // rows one direct load of a wave covers
#pragma unroll
    for (int n = 0; n < 32 / RPLQ; ++n) {
      const int rr = n * RPLQ + lane / KVEC_ROW;   // row of the wave's 32
      const int c = (lane % KVEC_ROW) ^ (rr & (KVEC_ROW - 1));
      const uint32_t off = (uint32_t)(((int64_t)(qw + rr) * a.q_ss + c * EPV) * E::kSize);
      buffer_load16_to_lds(q_desc, lds_address(q_stage) + n * kWave * 16, (qw + rr < ql && c * EPV < a.D) ? off : kOutOfRange);
    }
  } else {
    const rsrc_t q_rsrc = make_rsrc(qbase, (uint32_t)(((int64_t)(ql - 1) * a.q_ss + a.D) * E::kSize));
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      const int d = M::k_of(vs, g, NVS);
      const uint32_t off = (uint32_t)(((int64_t)q * a.q_ss + d) * E::kSize);
      qf[vs] = buffer_load16(q_rsrc, (q < ql && d < a.D) ? off : kOutOfRange);
    }
  }

  // K rows past the last valid key read as zeros through the bounds check (no traffic, no branches);
  // lanes whose channel chunk lies past the head size sit at an offset that stays out of range
  const rsrc_t k_rsrc = make_rsrc(kbase, (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * E::kSize));
  const rsrc_t s_rsrc = make_rsrc(sbase, (uint32_t)(score_row_offset<EPV>(a, ql) * E::kSize));   // rows >= ql are dropped
  const uint32_t k_row_bytes = (uint32_t)(a.k_ss * E::kSize);
  // direct loads: one instruction of a wave fills 1 KB of LDS, lane i the 16 bytes at 16 i.  Slot c of row r
  // holds the row's chunk c ^ (r & 15), which keeps the fragment reads of 16 consecutive rows on distinct banks.
  const int k_row = DMA ? wave * (kWave / KVEC_ROW) + lane / KVEC_ROW : tid / KVEC_ROW;
  const int k_c = DMA ? (lane % KVEC_ROW) ^ (k_row & (KVEC_ROW - 1)) : tid % KVEC_ROW;
  uint32_t k_off = (k_c * EPV < a.D) ? k_row * k_row_bytes + k_c * EPV * E::kSize : kOutOfRange;
  uint4 kreg[KLOADS];
  auto fetch_k = [&]() {
#pragma unroll
    for (int i = 0; i < KLOADS; ++i) kreg[i] = buffer_load16(k_rsrc, k_off + i * (kBlock / KVEC_ROW) * k_row_bytes);
    k_off += BK * k_row_bytes;
  };
  const desc_t k_desc = make_desc(kbase, (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * E::kSize));
  auto dma_k = [&](T *kdst) {
    const uint32_t lds0 = lds_address(kdst) + wave * kWave * 16;
#pragma unroll
    for (int i = 0; i < KLOADS; ++i)
      buffer_load16_to_lds(k_desc, lds0 + i * kBlock * 16, k_off + i * (kBlock / KVEC_ROW) * k_row_bytes);
    k_off += BK * k_row_bytes;
  };
  auto stage_k = [&](T *kdst) {
#pragma unroll
    for (int i = 0; i < KLOADS; ++i)
      *reinterpret_cast<uint4 *>(&kdst[(k_row + i * (kBlock / KVEC_ROW)) * KPITCH + k_c * EPV]) = kreg[i];
  };

  // where this lane's vectors of the strip go: row sr + 8i of the wave's 32 rows, 8 keys at column sc
  T *strip = lds_c[wave];
  const int sr = lane / CVEC_ROW, sc = (lane % CVEC_ROW) * EPV;
  int k_end[CSTORES];          // only vectors holding a key the row may see are written
  uint32_t s_off[CSTORES];
#pragma unroll
  for (int i = 0; i < CSTORES; ++i) {
    const int row = qw + sr + i * (kWave / CVEC_ROW);
    k_end[i] = min(a.causal ? min(kl, row + (kl - ql) + 1) : kl, a.Sk);
    s_off[i] = (uint32_t)((score_row_offset<EPV>(a, row) + sc) * E::kSize);
  }

  if constexpr (DMA) {
    dma_k(lds_k[0]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // the wave's own Q rows have landed; the barrier below keeps the tiles and strips of the loop off them until
    // every wave has read its own
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs)
      qf[vs] = *reinterpret_cast<const uint4 *>(&q_stage[r * DP + (((2 * vs + g) ^ (r & (KVEC_ROW - 1))) * EPV)]);
  } else {
    fetch_k();
    stage_k(lds_k[0]);
  }
  // The Q fragments are used here, before the loop, so that the wait for their loads is placed here too.  Left
  // to the loop, that wait ("at most the four newest memory operations outstanding") would on every later
  // iteration also wait for the previous tile's score stores to be acknowledged.
#pragma unroll
  for (int vs = 0; vs < NVS; ++vs) asm volatile("" ::"v"(qf[vs].x), "v"(qf[vs].y), "v"(qf[vs].z), "v"(qf[vs].w));
  lds_barrier();
  for (int kt = 0; kt < nkt; ++kt) {
    const int k0 = kt * BK;
    const T *ksrc = lds_k[kt & 1];
    T *knext = lds_k[(kt + 1) & 1];
    if constexpr (DMA) dma_k(knext); else fetch_k();   // next tile (past the end: out of range, zeros)

    floatx16 s[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int x = 0; x < 16; ++x) s[kb][x] = 0.f;
    {
      constexpr int NST = NVS / 2;               // K fragments are read two steps ahead of the MFMAs
      uint4 kf[2][2][KB];
      auto load_stage = [&](int st, uint4 (&dst)[2][KB]) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
            dst[u][kb] = *reinterpret_cast<const uint4 *>(
                DMA ? &ksrc[(kb * 32 + r) * KP + (((M::k_of(2 * st + u, g, NVS) / EPV) ^ (r & (KVEC_ROW - 1))) * EPV)]
                    : &ksrc[(kb * 32 + r) * KP + M::k_of(2 * st + u, g, NVS)]);
      };
      load_stage(0, kf[0]);
#pragma unroll
      for (int st = 0; st < NST; ++st) {
        if (st + 1 < NST) load_stage(st + 1, kf[(st + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) M::step(kf[st & 1][u][kb], qf[2 * st + u], s[kb]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // register 4j+i of block kb holds key 32kb + 8j + 4g + i of query r: into the wave's strip, row-major
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        Pack<T, 4> pk;
#pragma unroll
        for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(s[kb][4 * j + i] * a.alpha);
        store_pack<T, 4>(&strip[r * CPITCH + kb * 32 + 8 * j + 4 * g], pk);
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the strip is this wave's own: no barrier needed
#pragma unroll
    for (int i = 0; i < CSTORES; ++i) {
      const uint4 v = *reinterpret_cast<const uint4 *>(&strip[(sr + i * (kWave / CVEC_ROW)) * CPITCH + sc]);
      const uint32_t off = s_off[i] + (uint32_t)(k0 * E::kSize);
      buffer_store16<STREAM ? 2 : 0>(s_rsrc, (k0 + sc < k_end[i]) ? off : kOutOfRange, v);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // strip read out before the next tile overwrites it

    // direct loads are not in the compiler's count of outstanding memory operations: the wait is written here.
    // They were issued before this tile's CSTORES score stores, so the tile has landed once only those are left.
    if constexpr (DMA) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(CSTORES) : "memory");
    else stage_k(knext);                         // waits for the loads of this iteration only
    lds_barrier();
  }
}

// ===========================================================================
// ctx = P V
// ===========================================================================
template <int DT, int DP, bool VEC, bool STREAM>
__global__ __launch_bounds__(kBlock) void attn_pv_kernel(AttnArgs a) {
  typedef Elem<DT> E;
  typedef typename E::T T;
  typedef Mma<DT> M;
  constexpr int EPV = M::EPV;
  constexpr int BK = (DT == EN_F32) ? 32 : 64;   // keys per tile
  constexpr int MT = DP / 64;                    // 32-channel MFMA tiles per wave
  constexpr int NT = 2;                          // 32-query MFMA tiles per wave
  constexpr int NVS = BK / M::KPV;               // vector steps over a key tile
  constexpr int PITCH = BK + EPV;                // LDS pitch of P rows and V^T rows, elements
  constexpr int PVEC_ROW = BK / EPV;
  constexpr int PLOADS = kQTile * PVEC_ROW / kBlock;
  constexpr int NQUAD = BK / 4;                  // groups of four keys in a tile
  constexpr int NCHUNK = DP / EPV;               // 128-bit channel chunks in a V row
  constexpr int VUNITS = NQUAD * NCHUNK;         // (key quad, channel chunk) units per tile
  constexpr int VLOADS = (VUNITS + kBlock - 1) / kBlock;
  static_assert(kQTile * PVEC_ROW % kBlock == 0, "P tile must divide over the block");
  __shared__ __attribute__((aligned(16))) T lds_p[kQTile * PITCH];
  __shared__ __attribute__((aligned(16))) T lds_v[DP * PITCH];

  int unit, qi;
  if (!map_block(a, unit, qi)) return;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
  const int q0 = qi * kQTile;
  const int tid = threadIdx.x;
  T *cbase = reinterpret_cast<T *>(a.out) + q_unit_offset(a, b, h);

  if (q0 >= ql) {
    if (a.zero_padding) {  // whole tile is padding
      const int rows = min(kQTile, a.Sq - q0);
      for (int i = tid; i < rows * a.D; i += kBlock) {
        const int row = i / a.D, d = i - row * a.D;
        cbase[(int64_t)(q0 + row) * a.q_ss + d] = E::from_float(0.f);
      }
    }
    return;
  }
  const int nk = tile_key_extent(a, min(q0 + kQTile, ql) - 1, kl, ql);
  const int nkt = (nk + BK - 1) / BK;

  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int wq = wave & 1, wd = wave >> 1;

  const T *pbase = reinterpret_cast<const T *>(a.a_ptr) + ((int64_t)unit * a.Sq) * a.Sk;
  const T *vbase = reinterpret_cast<const T *>(a.b_ptr) + k_unit_offset(a, b, h);

  floatx16 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int x = 0; x < 16; ++x) acc[mt][nt][x] = 0.f;

  // rows of padded queries, columns past the visible extent and V rows >= kl read as zero
  // through the bounds check; the loop body has no branches on the fast path.
  const rsrc_t p_rsrc = make_rsrc(pbase, (uint32_t)((int64_t)ql * a.Sk * E::kSize));
  const rsrc_t v_rsrc = make_rsrc(vbase, (uint32_t)(((int64_t)(max(kl, 1) - 1) * a.k_ss + a.D) * E::kSize));
  uint4 preg[PLOADS];
  uint4 vreg[VLOADS][4];
  // a probability row is read only as far as its own query sees: what lies past that need not have been written
  int p_vis[PLOADS];
#pragma unroll
  for (int i = 0; i < PLOADS; ++i) {
    const int q = q0 + (tid + i * kBlock) / PVEC_ROW;
    p_vis[i] = q < ql ? tile_key_extent(a, q, kl, ql) : 0;
  }
  auto fetch = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < PLOADS; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / PVEC_ROW, c = v % PVEC_ROW;
      const int q = q0 + row, k = k0 + c * EPV;
      if constexpr (VEC) {
        const uint32_t off = (uint32_t)(((int64_t)q * a.Sk + k) * E::kSize);
        preg[i] = buffer_load16<STREAM ? 2 : 0>(p_rsrc, (kt < nkt && k < p_vis[i]) ? off : kOutOfRange);
      } else if (kt < nkt && k < p_vis[i]) {
        const T *gp = pbase + (int64_t)q * a.Sk + k;
        {
          Pack<T, EPV> pk;
#pragma unroll
          for (int e = 0; e < EPV; ++e) pk.v[e] = (k + e < p_vis[i]) ? gp[e] : E::from_float(0.f);
          preg[i] = __builtin_bit_cast(uint4, pk);
        }
      } else {
        preg[i] = zero4();
      }
    }
#pragma unroll
    for (int i = 0; i < VLOADS; ++i) {
      const int u = tid + i * kBlock;
      const int c = (u % 4) + 4 * ((u / (4 * NQUAD)) % (NCHUNK / 4 > 0 ? NCHUNK / 4 : 1));
      const int kq = (u / 4) % NQUAD;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int key = k0 + kq * 4 + x;
        const uint32_t off = (uint32_t)(((int64_t)key * a.k_ss + c * EPV) * E::kSize);
        vreg[i][x] = buffer_load16(v_rsrc, (kt < nkt && u < VUNITS && key < kl && c * EPV < a.D) ? off : kOutOfRange);
      }
    }
  };
  if (nkt > 0) fetch(0);

  for (int kt = 0; kt < nkt; ++kt) {
    // P tile: straight copy.  V tile: four keys x EPV channels per unit, written transposed
    // so that a lane later reads consecutive keys of one channel with one 128-bit load.
#pragma unroll
    for (int i = 0; i < PLOADS; ++i) {
      const int v = tid + i * kBlock;
      const int row = v / PVEC_ROW, c = v % PVEC_ROW;
      *reinterpret_cast<uint4 *>(&lds_p[row * PITCH + c * EPV]) = preg[i];
    }
#pragma unroll
    for (int i = 0; i < VLOADS; ++i) {
      const int u = tid + i * kBlock;
      if (VUNITS % kBlock == 0 || u < VUNITS) {
        const int c = (u % 4) + 4 * ((u / (4 * NQUAD)) % (NCHUNK / 4 > 0 ? NCHUNK / 4 : 1));
        const int kq = (u / 4) % NQUAD;
        Pack<T, EPV> rows[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) rows[x] = __builtin_bit_cast(Pack<T, EPV>, vreg[i][x]);
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
          Pack<T, 4> col;
#pragma unroll
          for (int x = 0; x < 4; ++x) col.v[x] = rows[x].v[e];
          store_pack<T, 4>(&lds_v[(c * EPV + e) * PITCH + kq * 4], col);
        }
      }
    }
    lds_barrier();
    fetch(kt + 1);

#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      const int kk = M::k_of(vs, g, NVS);
      uint4 vf[MT], pf[NT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        vf[mt] = *reinterpret_cast<const uint4 *>(&lds_v[(wd * (DP / 2) + mt * 32 + r) * PITCH + kk]);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        pf[nt] = *reinterpret_cast<const uint4 *>(&lds_p[(wq * 64 + nt * 32 + r) * PITCH + kk]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) M::step(vf[mt], pf[nt], acc[mt][nt]);
    }
    lds_barrier();  // tiles are consumed before the next ones are written
  }

  // each lane owns four consecutive channels of one query row
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int q = q0 + wq * 64 + nt * 32 + r;
    if (q >= a.Sq) continue;
    const bool valid = q < ql;
    if (!valid && !a.zero_padding) continue;
    T *crow = cbase + (int64_t)q * a.q_ss;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = wd * (DP / 2) + mt * 32 + 8 * j + 4 * g;
        if (d < a.D) {
          Pack<T, 4> pk;
#pragma unroll
          for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(valid ? acc[mt][nt][4 * j + i] : 0.f);
          store_pack<T, 4>(crow + d, pk);
        }
      }
  }
}

// ===========================================================================
// ctx = P V, 16-bit operands with 16-byte aligned probability rows.
//
// Same strip form as QK^T above: wave w owns queries 32w..32w+31 and every channel,
// O^T += V^T P^T per 64-key tile.  V tiles are shared through LDS (transposed, double-
// buffered, fetched one tile ahead: one barrier per tile).  Each wave reads its own 32
// probability rows with row-contiguous 128-bit loads, one tile ahead, and passes them
// through a strip of LDS of its own to get the MFMA operand order; no barrier is involved.
// ===========================================================================
template <int DT, int DP, bool STREAM>
__global__ __launch_bounds__(kBlock, 3) void attn_pv_strip_kernel(AttnArgs a) {
  static_assert(DT != EN_F32, "16-bit storage only");
  static_assert(DP == 64 || DP == 128, "swizzles are written for 8 or 16 slots per V row");
  typedef Elem<DT> E;
  typedef typename E::T T;
  typedef Mma<DT> M;
  constexpr int EPV = 8;
  constexpr int BK = 64;                         // keys per tile
  constexpr int NVS = BK / 16;                   // MFMA steps over a key tile
  constexpr int DMT = DP / 32;                   // 32-channel MFMA tiles of the output
  constexpr int VVEC_ROW = DP / EPV;             // 16-byte slots per V row
  constexpr int VLOADS = BK * VVEC_ROW / kBlock; // direct loads per wave and V tile
  constexpr int RPL = kWave / VVEC_ROW;          // V rows one direct load of a wave covers
  constexpr int PVEC_ROW = BK / EPV;             // 16-byte slots per probability row of a tile: 8
  constexpr int PLOADS = 32 * PVEC_ROW / kWave;  // direct loads per wave and probability strip: 4, eight rows each
  constexpr uint32_t VROW_BYTES = DP * sizeof(T), PROW_BYTES = BK * sizeof(T);
  static_assert(BK * VVEC_ROW % kBlock == 0, "V tile must divide over the block");
  // Both operands travel from memory straight into LDS, unpadded, with their 16-byte chunks in XOR-swizzled slots:
  //   V tile [key][channel], two buffers: slot c of key k holds chunk c ^ vswz(k), vswz = 4 (k & 3) (16 slots) or
  //     4 ((k >> 1) & 1) (8 slots).  The transposing read of a 16-lane group takes 32 bytes from each of four
  //     consecutive keys; a half wave's 64 bytes per key then fall into four distinct quarters of the banks.
  //   probability strip [query][key] of each wave, 32 x 64: slot c of row q holds chunk c ^ ((q >> 1) & 7), which
  //     puts the 128-bit reads of 16 consecutive rows at one chunk on all 64 banks once.
  __shared__ __attribute__((aligned(16))) T lds_v[2][BK * DP];
  __shared__ __attribute__((aligned(16))) T lds_p[kBlock / kWave][32 * BK];

  int unit, qi;
  if (!map_block(a, unit, qi)) return;
  const int b = unit / a.H, h = unit % a.H;
  int kl, ql;
  seq_extents(a, b, kl, ql);
  const int q0 = qi * kQTile;
  const int tid = threadIdx.x;
  T *cbase = reinterpret_cast<T *>(a.out) + q_unit_offset(a, b, h);

  if (q0 >= ql) {
    if (a.zero_padding) {  // whole tile is padding
      const int rows = min(kQTile, a.Sq - q0);
      for (int i = tid; i < rows * a.D; i += kBlock) {
        const int row = i / a.D, d = i - row * a.D;
        cbase[(int64_t)(q0 + row) * a.q_ss + d] = E::from_float(0.f);
      }
    }
    return;
  }
  const int nk = tile_key_extent(a, min(q0 + kQTile, ql) - 1, kl, ql);
  const int nkt = (nk + BK - 1) / BK;

  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int qw = q0 + wave * 32;                 // first query of this wave
  const int q = qw + r;                          // query whose context this lane accumulates

  const T *pbase = reinterpret_cast<const T *>(a.a_ptr) + score_unit_offset<EPV>(a, unit);
  const T *vbase = reinterpret_cast<const T *>(a.b_ptr) + k_unit_offset(a, b, h);
  // rows of padded queries lie past the end of the descriptor and arrive as zeros; so do V rows >= kl
  const desc_t p_desc = make_desc(pbase, (uint32_t)(score_row_offset<EPV>(a, ql) * E::kSize));
  const desc_t v_desc = make_desc(vbase, kl > 0 ? (uint32_t)(((int64_t)(kl - 1) * a.k_ss + a.D) * E::kSize) : 0u);

  // ---- V: lane i of the wave's n-th load fills slot i % VVEC_ROW of tile row RPL (4n + wave) + i / VVEC_ROW
  const uint32_t v_row_bytes = (uint32_t)(a.k_ss * E::kSize);
  const int ld_row = wave * RPL + lane / VVEC_ROW, ld_slot = lane % VVEC_ROW;
  const int v_c = ld_slot ^ (DP == 128 ? 4 * (ld_row & 3) : 4 * ((ld_row >> 1) & 1));
  uint32_t v_off = (v_c * EPV < a.D) ? ld_row * v_row_bytes + v_c * EPV * E::kSize : kOutOfRange;
  auto fetch_v = [&](T *vdst) {
    const uint32_t v_lds = lds_address(vdst) + wave * kWave * 16;
#pragma unroll
    for (int i = 0; i < VLOADS; ++i) buffer_load16_to_lds(v_desc, v_lds + i * kBlock * 16, v_off + i * (kBlock / VVEC_ROW) * v_row_bytes);
    v_off += BK * v_row_bytes;
  };
  // transposing read: lane j of a 16-lane group points at key j / 4 of the group's four keys and at channels
  // 4 (j % 4) .. + 3 of the group's sixteen; the read hands lane i of the group channel i of those sixteen at the
  // four keys.  Byte offset inside a V buffer for channel tile mt and keys 8g + 0..3 of step 0:
  const int tj = lane & 15, tg = (lane >> 4) & 1;
  const int vsw = DP == 128 ? (tj >> 2) : ((tj >> 3) & 1);
  uint32_t v_frag[DMT];
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
    v_frag[mt] = (uint32_t)((8 * g + (tj >> 2)) * VROW_BYTES + (4 * (mt ^ vsw) + 2 * tg + ((tj >> 1) & 1)) * 16 + (tj & 1) * 8);

  // ---- probabilities: the wave's n-th load brings rows 8n .. 8n + 7 of its strip, lane i slot i % 8 of row
  //      8n + i / 8; the chunk it holds is (i % 8) ^ ((row >> 1) & 7) = (i % 8) ^ (i >> 4) ^ 4 (n & 1)
  T *strip = lds_p[wave];
  const uint32_t strip_lds = lds_address(strip);
  const int p_c0 = (lane & 7) ^ (lane >> 4);
  uint32_t p_off[PLOADS];
  int p_left[PLOADS];          // keys of the row still visible from this lane's chunk on, in tile 0: a row is read
                               // only as far as its own query sees, the rest need not have been written
#pragma unroll
  for (int i = 0; i < PLOADS; ++i) {
    const int row = qw + 8 * i + (lane >> 3);
    const int c = p_c0 ^ (4 * (i & 1));
    p_off[i] = (uint32_t)((score_row_offset<EPV>(a, row) + c * EPV) * E::kSize);
    p_left[i] = (row < ql ? tile_key_extent(a, row, kl, ql) : 0) - c * EPV;
  }
  auto fetch_p = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < PLOADS; ++i)
      buffer_load16_to_lds<STREAM ? 2 : 0>(p_desc, strip_lds + i * kWave * 16,
                                           (k0 < p_left[i]) ? p_off[i] + (uint32_t)(k0 * E::kSize) : kOutOfRange);
  };
  const uint32_t p_frag = (uint32_t)(r * PROW_BYTES);
  const int psw = (r >> 1) & 7;

  floatx16 o[DMT];
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
    for (int x = 0; x < 16; ++x) o[mt][x] = 0.f;

  fetch_v(lds_v[0]);
  fetch_p(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  lds_barrier();
  for (int kt = 0; kt < nkt; ++kt) {
    const char *vsrc = reinterpret_cast<const char *>(lds_v[kt & 1]);
    fetch_v(lds_v[(kt + 1) & 1]);                // next tile (past the end: out of range, zeros, no traffic)

    // B operands: keys 16vs + 8g .. +7 of this lane's query, out of the wave's own strip
    uint4 pf[NVS];
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs)
      pf[vs] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(strip) + p_frag + (((2 * vs + g) ^ psw) * 16));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave has read its strip: the next one may arrive
    fetch_p(kt + 1);

    // A operands: V^T at the same keys, read one step ahead of the MFMAs
    uint4 va[2][DMT];
    auto load_step = [&](int vs, uint4 (&dst)[DMT]) {
#pragma unroll
      for (int mt = 0; mt < DMT; ++mt) {
        const char *vt = vsrc + vs * 16 * VROW_BYTES + v_frag[mt];
        const uint2 lo = lds_read_tr16(vt);                       // keys 16vs + 8g + 0..3
        const uint2 hi = lds_read_tr16(vt + 4 * VROW_BYTES);      // keys 16vs + 8g + 4..7
        dst[mt] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    };
    load_step(0, va[0]);
#pragma unroll
    for (int vs = 0; vs < NVS; ++vs) {
      if (vs + 1 < NVS) load_step(vs + 1, va[(vs + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < DMT; ++mt) M::step(va[vs & 1][mt], pf[vs], o[mt]);
      __builtin_amdgcn_sched_barrier(0);
    }

    // direct loads are not in the compiler's count of outstanding memory operations: the wait is written here
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
  }

  // register 4j+i of tile mt holds channel 32mt + 8j + 4g + i of this lane's query
  if (a.ctx_vec16) {
    // A lane holds 8-byte pieces of its own row, 32 rows per store instruction; through LDS (the V buffers are free
    // behind the loop's last barrier, each wave takes the 32 rows' worth that is its own, so no barrier is needed)
    // the wave's tile leaves as whole rows: 16 bytes per lane, 64 / VVEC_ROW rows per instruction.  Chunk c of row r
    // sits in slot c ^ (r % VVEC_ROW): writes and reads both spread over all banks.
    char *stage = reinterpret_cast<char *>(&lds_v[0][0]) + wave * 32 * VROW_BYTES;
    const bool valid = q < ql;
#pragma unroll
    for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        Pack<T, 4> pk;
#pragma unroll
        for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(valid ? o[mt][4 * j + i] : 0.f);
        const int c = 4 * mt + j;
        *reinterpret_cast<Pack<T, 4> *>(stage + r * VROW_BYTES + ((c ^ (r & (VVEC_ROW - 1))) * 16) + g * 8) = pk;
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes, before its lanes read each other's
#pragma unroll
    for (int i = 0; i < 32 / RPL; ++i) {
      const int row = i * RPL + lane / VVEC_ROW, c = lane % VVEC_ROW;
      const uint4 v = *reinterpret_cast<const uint4 *>(stage + row * VROW_BYTES + ((c ^ (row & (VVEC_ROW - 1))) * 16));
      const int qrow = q0 + wave * 32 + row;
      if (qrow < (a.zero_padding ? a.Sq : ql) && c * EPV < a.D) *reinterpret_cast<uint4 *>(cbase + (int64_t)qrow * a.q_ss + c * EPV) = v;
    }
    return;
  }
  if (q >= a.Sq) return;
  const bool valid = q < ql;
  if (!valid && !a.zero_padding) return;
  T *crow = cbase + (int64_t)q * a.q_ss;
#pragma unroll
  for (int mt = 0; mt < DMT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = mt * 32 + 8 * j + 4 * g;
      if (d < a.D) {
        Pack<T, 4> pk;
#pragma unroll
        for (int i = 0; i < 4; ++i) pk.v[i] = E::from_float(valid ? o[mt][4 * j + i] : 0.f);
        store_pack<T, 4>(crow + d, pk);
      }
    }
}

// ===========================================================================
// workgroup order for a batch: real query tiles only, longest sequence first
// ===========================================================================
// table[w] for workgroup w of a launch of ceil(B H / 8) * 8 * ntq workgroups.  Workgroups go to the XCDs round-robin,
// so entries w = 8 j + x are XCD x's sequence: the (batch, head) units are dealt to the XCDs in the order of
// decreasing sequence length (units of one sequence on consecutive XCDs), and tiles past a sequence's end get no
// entry; what is left of the table is -1.  Within an XCD either
//   unit by unit, each unit's query tiles from the last (longest under a causal mask) to the first
//     (tiles_first == 0): the tiles of a unit run together and share its K and V in the XCD's L2; or
//   tile index by tile index from the last to the first, every unit that has the tile (tiles_first == 1): the
//     long workgroups of all units start first -- the better schedule when a unit's K and V are small enough
//     to be re-read cheaply (512-key, 64-channel units: 21.3 -> 19.6 us; 1024 x 128: 213 -> 225 us).
// One workgroup; the sort is a rank count (batch <= 1024), larger batches keep their order.  The fill is spread over
// the whole workgroup when the batch is sorted (a serial walk by eight threads took 43 us for 896 units of up to
// eight tiles).
__global__ __launch_bounds__(1024) void attn_tile_table_kernel(const int32_t *__restrict__ lens, int batch, int heads,
                                                               int seq_len, int ntq, int32_t *__restrict__ table,
                                                               int capacity, int tiles_first, int q_tile) {
  __shared__ int32_t s_len[1024];
  __shared__ int32_t s_order[1024];
  const int tid = threadIdx.x;
  for (int i = tid; i < capacity; i += 1024) table[i] = -1;
  const bool sorted = batch <= 1024;
  if (sorted) {
    if (tid < batch) s_len[tid] = min(max(lens[tid], 0), seq_len);
    __syncthreads();
    if (tid < batch) {
      const int n = s_len[tid];
      int rank = 0;
      for (int j = 0; j < batch; ++j) rank += (s_len[j] > n || (s_len[j] == n && j < tid)) ? 1 : 0;
      s_order[rank] = tid;
    }
  }
  __syncthreads();   // also orders the -1 fill before the entries written below
  const int units = batch * heads;
  auto tiles_of = [&](int u, int &unit) {          // u-th unit in sorted order -> its index and tile count
    const int p = u / heads, h = u - p * heads;
    const int b = sorted ? s_order[p] : p;
    const int n = sorted ? s_len[b] : min(max(lens[b], 0), seq_len);
    unit = b * heads + h;
    return (n + q_tile - 1) / q_tile;
  };
  constexpr int kChunks = 1024 / kXcds;             // threads per XCD list
  constexpr int kMaxTiles = 256;
  if (sorted && ntq <= kMaxTiles) {
    // Every thread takes a contiguous chunk of one XCD's unit list (units x, x + 8, x + 16, ... of the sorted order).
    // Sorted by length, the tile counts along a list never increase, so the units that have tile qi are a prefix of
    // the list: a unit's place among them is its place in the list.
    __shared__ int32_t s_sum[kXcds][kChunks + 1];   // unit-major: tiles in the chunks before this one
    __shared__ int32_t s_cnt[kXcds][kMaxTiles + 1]; // tiles-first: units of the list that have tile qi
    const int x = tid % kXcds, c = tid / kXcds;
    const int list_len = (units - x + kXcds - 1) / kXcds;            // units x + 8 i, i < list_len
    const int per = (list_len + kChunks - 1) / kChunks;
    const int i0 = min(c * per, list_len), i1 = min(i0 + per, list_len);
    for (int i = tid; i < kXcds * (kMaxTiles + 1); i += 1024) (&s_cnt[0][0])[i] = 0;
    __syncthreads();
    int mine = 0, unit;
    for (int i = i0; i < i1; ++i) {
      const int nt = tiles_of(x + kXcds * i, unit);
      mine += nt;
      if (tiles_first && nt > 0) atomicAdd(&s_cnt[x][nt - 1], 1);     // units whose LAST tile is nt - 1
    }
    s_sum[x][c] = mine;
    __syncthreads();
    if (tid < kXcds) {
      if (tiles_first) {      // units that have tile qi = units whose last tile is >= qi; then where tile qi's run starts
        int run = 0;
        for (int qi = ntq - 1; qi >= 0; --qi) { run += s_cnt[tid][qi]; s_cnt[tid][qi] = run; }
        int start = 0;
        for (int qi = ntq - 1; qi >= 0; --qi) { const int n = s_cnt[tid][qi]; s_cnt[tid][qi] = start; start += n; }
      } else {
        int run = 0;
        for (int k = 0; k < kChunks; ++k) { const int n = s_sum[tid][k]; s_sum[tid][k] = run; run += n; }
      }
    }
    __syncthreads();
    if (tiles_first) {
      for (int i = i0; i < i1; ++i) {
        const int nt = tiles_of(x + kXcds * i, unit);
        for (int qi = nt - 1; qi >= 0; --qi) table[(s_cnt[x][qi] + i) * kXcds + x] = unit * ntq + qi;
      }
    } else {
      int j = s_sum[x][c];
      for (int i = i0; i < i1; ++i) {
        const int nt = tiles_of(x + kXcds * i, unit);
        for (int qi = nt - 1; qi >= 0; --qi) table[j++ * kXcds + x] = unit * ntq + qi;
      }
    }
    return;
  }
  if (tid < kXcds) {      // batches too large to sort, rows of more than 256 tiles: one thread per XCD walks its list
    int j = 0, unit;
    if (tiles_first) {
      for (int qi = ntq - 1; qi >= 0; --qi)
        for (int u = tid; u < units; u += kXcds)
          if (qi < tiles_of(u, unit)) table[j++ * kXcds + tid] = unit * ntq + qi;
    } else {
      for (int u = tid; u < units; u += kXcds) {
        const int nt = tiles_of(u, unit);
        for (int qi = nt - 1; qi >= 0; --qi) table[j++ * kXcds + tid] = unit * ntq + qi;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static bool strides_vec_ok(int64_t sb, int64_t sh, int64_t ss, int epv) {
  return (sb % epv) == 0 && (sh % epv) == 0 && (ss % epv) == 0;
}

// bytes of the score tensor the kernels go through: all of [B,H,Sq,Sk], or the packed causal prefixes
template <int DT>
static int64_t score_tensor_bytes(const AttnArgs &a) {
  constexpr int EPV = 16 / Elem<DT>::kSize;
  return (int64_t)a.units * (a.packed_scores ? packed_row_start<EPV * kPackedRowVectors>(a.Sq) : (int64_t)a.Sq * a.Sk) * Elem<DT>::kSize;
}

template <int DT>
static int launch_qk(AttnArgs &a, hipStream_t s) {
  const unsigned grid = (unsigned)(ceil_div(a.units, kXcds) * kXcds * a.ntq);
  // a score tensor too large to stay in the memory-side cache is written with the non-temporal policy
  const bool stream = score_tensor_bytes<DT>(a) >= kStreamScoreBytes;
  if (a.packed_scores && (DT == EN_F32 || !a.vec_out)) return EN_ERR_UNSUPPORTED;
  if constexpr (DT != EN_F32) {
    if (a.vec_out) {   // 16-bit, aligned rows
      if (a.D <= 64) {
        if (stream) attn_qk_strip_kernel<DT, 64, true><<<grid, kBlock, 0, s>>>(a);
        else attn_qk_strip_kernel<DT, 64, false><<<grid, kBlock, 0, s>>>(a);
      } else {
        if (stream) attn_qk_strip_kernel<DT, 128, true><<<grid, kBlock, 0, s>>>(a);
        else attn_qk_strip_kernel<DT, 128, false><<<grid, kBlock, 0, s>>>(a);
      }
      EN_RETURN_IF_LAUNCH_FAILED();
      return EN_OK;
    }
  }
  if (a.vec_out) {
    if (a.D <= 64) {
      if (stream) attn_qk_kernel<DT, 64, true, true><<<grid, kBlock, 0, s>>>(a);
      else attn_qk_kernel<DT, 64, true, false><<<grid, kBlock, 0, s>>>(a);
    } else {
      if (stream) attn_qk_kernel<DT, 128, true, true><<<grid, kBlock, 0, s>>>(a);
      else attn_qk_kernel<DT, 128, true, false><<<grid, kBlock, 0, s>>>(a);
    }
  } else {
    if (a.D <= 64) attn_qk_kernel<DT, 64, false, false><<<grid, kBlock, 0, s>>>(a);
    else attn_qk_kernel<DT, 128, false, false><<<grid, kBlock, 0, s>>>(a);
  }
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

template <int DT>
static int launch_pv(AttnArgs &a, hipStream_t s) {
  const unsigned grid = (unsigned)(ceil_div(a.units, kXcds) * kXcds * a.ntq);
  // probabilities of a tensor too large to stay cached are read with the non-temporal policy
  const bool stream = score_tensor_bytes<DT>(a) >= kStreamScoreBytes;
  if (a.packed_scores && (DT == EN_F32 || !a.vec_out)) return EN_ERR_UNSUPPORTED;
  if constexpr (DT != EN_F32) {
    if (a.vec_out) {   // 16-bit, aligned rows
      if (a.D <= 64) {
        if (stream) attn_pv_strip_kernel<DT, 64, true><<<grid, kBlock, 0, s>>>(a);
        else attn_pv_strip_kernel<DT, 64, false><<<grid, kBlock, 0, s>>>(a);
      } else {
        if (stream) attn_pv_strip_kernel<DT, 128, true><<<grid, kBlock, 0, s>>>(a);
        else attn_pv_strip_kernel<DT, 128, false><<<grid, kBlock, 0, s>>>(a);
      }
      EN_RETURN_IF_LAUNCH_FAILED();
      return EN_OK;
    }
  }
  if (a.vec_out) {
    if (a.D <= 64) {
      if (stream) attn_pv_kernel<DT, 64, true, true><<<grid, kBlock, 0, s>>>(a);
      else attn_pv_kernel<DT, 64, true, false><<<grid, kBlock, 0, s>>>(a);
    } else {
      if (stream) attn_pv_kernel<DT, 128, true, true><<<grid, kBlock, 0, s>>>(a);
      else attn_pv_kernel<DT, 128, true, false><<<grid, kBlock, 0, s>>>(a);
    }
  } else {
    if (a.D <= 64) attn_pv_kernel<DT, 64, false, false><<<grid, kBlock, 0, s>>>(a);
    else attn_pv_kernel<DT, 128, false, false><<<grid, kBlock, 0, s>>>(a);
  }
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

static int check_common(const void *x, const void *y, const void *z, const int32_t *k_lens, int batch, int head_num,
                        int q_seq_len, int k_seq_len, int size_per_head, int dtype) {
  if (!x || !y || !z || !k_lens) return EN_ERR_NULL;
  if (batch < 1 || head_num < 1 || q_seq_len < 1 || k_seq_len < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  const int es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  const int epv = 16 / es;
  if (size_per_head > 128 || (size_per_head % epv) != 0) return EN_ERR_UNSUPPORTED;
  if ((int64_t)batch * head_num > INT32_MAX / 64) return EN_ERR_SHAPE;
  // per-(batch, head) byte offsets are 32-bit buffer offsets
  if ((int64_t)q_seq_len * k_seq_len * es >= (1ll << 31)) return EN_ERR_UNSUPPORTED;
  return EN_OK;
}

}  // namespace en

extern "C" {

int64_t en_attn_tile_table_elems(int batch, int head_num, int q_seq_len, int query_tile) {
  using namespace en;
  if (query_tile == 0) query_tile = kQTile;
  if (batch < 1 || head_num < 1 || q_seq_len < 1 || (query_tile != kQTile && query_tile != 2 * kQTile)) return 0;
  return ceil_div((int64_t)batch * head_num, (int64_t)kXcds) * kXcds * ceil_div(q_seq_len, query_tile);
}

int en_attn_tile_table(const int32_t *seq_lens, int batch, int head_num, int q_seq_len, int tiles_first,
                       int query_tile, int32_t *table, en_stream_t stream) {
  using namespace en;
  if (!seq_lens || !table) return EN_ERR_NULL;
  if (query_tile == 0) query_tile = kQTile;
  if (batch < 1 || head_num < 1 || q_seq_len < 1) return EN_ERR_SHAPE;
  if (query_tile != kQTile && query_tile != 2 * kQTile) return EN_ERR_UNSUPPORTED;
  const int64_t cap = en_attn_tile_table_elems(batch, head_num, q_seq_len, query_tile);
  if (cap > INT32_MAX || (int64_t)batch * head_num > INT32_MAX / 64) return EN_ERR_SHAPE;
  attn_tile_table_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(seq_lens, batch, head_num, q_seq_len,
                                                               (int)ceil_div(q_seq_len, query_tile), table, (int)cap,
                                                               tiles_first ? 1 : 0, query_tile);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_attn_qk(const void *q, const void *k, void *scores, const int32_t *k_lens, const int32_t *q_lens, int batch,
               int head_num, int q_seq_len, int k_seq_len, int size_per_head, int64_t q_stride_b,
               int64_t q_stride_h, int64_t q_stride_s, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
               float alpha, int causal, int dtype, const int32_t *q_row_offsets, const int32_t *k_row_offsets,
               int packed_scores, const int32_t *tile_table, en_stream_t stream) {
  using namespace en;
  int rc = check_common(q, k, scores, k_lens, batch, head_num, q_seq_len, k_seq_len, size_per_head, dtype);
  if (rc) return rc;
  // the packed score layout is that of causal self-attention: row q holds q + 1 scores
  if (packed_scores && (!causal || q_lens || q_seq_len != k_seq_len)) return EN_ERR_UNSUPPORTED;
  if (tile_table && q_lens) return EN_ERR_UNSUPPORTED;      // the table lists the query tiles of min(k_lens, q_seq_len) rows
  const int es = dtype_size(dtype), epv = 16 / es;
  if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(scores, es)) return EN_ERR_ALIGN;
  if (!strides_vec_ok(q_stride_b, q_stride_h, q_stride_s, epv) ||
      !strides_vec_ok(k_stride_b, k_stride_h, k_stride_s, epv))
    return EN_ERR_ALIGN;
  // 32-bit byte offsets into K, advanced a tile at a time up to two tiles past the end
  if (k_stride_s < 0 || ((int64_t)k_seq_len + 256) * k_stride_s * es >= (1ll << 31)) return EN_ERR_UNSUPPORTED;
  AttnArgs a{};
  a.a_ptr = q; a.b_ptr = k; a.out = scores; a.k_lens = k_lens; a.q_lens = q_lens;
  a.B = batch; a.H = head_num; a.Sq = q_seq_len; a.Sk = k_seq_len; a.D = size_per_head;
  a.q_sb = q_stride_b; a.q_sh = q_stride_h; a.q_ss = q_stride_s;
  a.k_sb = k_stride_b; a.k_sh = k_stride_h; a.k_ss = k_stride_s;
  a.alpha = alpha; a.causal = causal ? 1 : 0; a.zero_padding = 0;
  a.q_row0 = q_row_offsets; a.k_row0 = k_row_offsets; a.packed_scores = packed_scores ? 1 : 0;
  a.tile_table = tile_table;
  a.vec_out = ((packed_scores || (k_seq_len % epv) == 0) && aligned_to(scores, 16)) ? 1 : 0;
  a.ntq = (int)ceil_div(q_seq_len, kQTile);
  a.units = batch * head_num;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return launch_qk<EN_F32>(a, s);
    case EN_F16: return launch_qk<EN_F16>(a, s);
    default: return launch_qk<EN_BF16>(a, s);
  }
}

int en_attn_pv(const void *p, const void *v, void *ctx, const int32_t *k_lens, const int32_t *q_lens, int batch,
               int head_num, int q_seq_len, int k_seq_len, int size_per_head, int64_t v_stride_b,
               int64_t v_stride_h, int64_t v_stride_s, int64_t c_stride_b, int64_t c_stride_h, int64_t c_stride_s,
               int causal, int zero_padding, int dtype, const int32_t *c_row_offsets, const int32_t *v_row_offsets,
               int packed_scores, const int32_t *tile_table, en_stream_t stream) {
  using namespace en;
  int rc = check_common(p, v, ctx, k_lens, batch, head_num, q_seq_len, k_seq_len, size_per_head, dtype);
  if (rc) return rc;
  if (packed_scores && (!causal || q_lens || q_seq_len != k_seq_len)) return EN_ERR_UNSUPPORTED;
  if (tile_table && q_lens) return EN_ERR_UNSUPPORTED;      // the table lists the query tiles of min(k_lens, q_seq_len) rows
  // a packed context has no padding rows: what follows a sequence's last row is the next sequence
  if (c_row_offsets && zero_padding) return EN_ERR_UNSUPPORTED;
  const int es = dtype_size(dtype), epv = 16 / es;
  if (!aligned_to(p, es) || !aligned_to(v, 16) || !aligned_to(ctx, 4 * es)) return EN_ERR_ALIGN;
  if (!strides_vec_ok(v_stride_b, v_stride_h, v_stride_s, epv) ||
      !strides_vec_ok(c_stride_b, c_stride_h, c_stride_s, 4))
    return EN_ERR_ALIGN;
  // 32-bit byte offsets into V, advanced a tile at a time up to two tiles past the end
  if (v_stride_s < 0 || ((int64_t)k_seq_len + 256) * v_stride_s * es >= (1ll << 31)) return EN_ERR_UNSUPPORTED;
  AttnArgs a{};
  a.a_ptr = p; a.b_ptr = v; a.out = ctx; a.k_lens = k_lens; a.q_lens = q_lens;
  a.B = batch; a.H = head_num; a.Sq = q_seq_len; a.Sk = k_seq_len; a.D = size_per_head;
  a.q_sb = c_stride_b; a.q_sh = c_stride_h; a.q_ss = c_stride_s;
  a.k_sb = v_stride_b; a.k_sh = v_stride_h; a.k_ss = v_stride_s;
  a.alpha = 1.f; a.causal = causal ? 1 : 0; a.zero_padding = zero_padding ? 1 : 0;
  a.q_row0 = c_row_offsets; a.k_row0 = v_row_offsets; a.packed_scores = packed_scores ? 1 : 0;
  a.tile_table = zero_padding ? nullptr : tile_table;      // the tiles a table leaves out are the ones to fill with zeros
  a.vec_out = ((packed_scores || (k_seq_len % epv) == 0) && aligned_to(p, 16)) ? 1 : 0;
  a.ctx_vec16 = (aligned_to(ctx, 16) && strides_vec_ok(c_stride_b, c_stride_h, c_stride_s, epv)) ? 1 : 0;
  a.ntq = (int)ceil_div(q_seq_len, kQTile);
  a.units = batch * head_num;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case EN_F32: return launch_pv<EN_F32>(a, s);
    case EN_F16: return launch_pv<EN_F16>(a, s);
    default: return launch_pv<EN_BF16>(a, s);
  }
}

}  // extern "C"
