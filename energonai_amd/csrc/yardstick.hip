// Bandwidth yardsticks: kernels that do nothing but move bytes in the access patterns of the library's
// memory-bound kernels, so that "what this part reaches on this pattern" is a measured figure beside every
// kernel's own rate instead of a guess.
//
//   stream_kernel   one contiguous range: copy, read only, write only; plain or non-temporal accesses
//                   (the pattern of depad, the transposes, the LayerNorm, the decode kernels' cache reads).
//   prefix_kernel   the causal prefixes of a score tensor: row q of a (batch, head) unit holds q + 1 elements,
//                   only rows q < seq_lens[b] exist; in the padded [B,H,S,S] layout or in the packed one.
//                   Read and written back in place (scale_mask_softmax), written only (QK^T), read only (PV),
//                   or read from one tensor and written to another.
//   prefix_tile_walk_kernel  the same prefixes read a 128-row tile at a time along the keys, as PV reads them.
//
// Neither is called by any op of the library; bench.py times them (--copy-yardstick and the yardstick_GBps
// column of its kernel tables).
#include "common.hip.h"

namespace en {

// mode: 0 copy (with dst == src: a pass in place), 1 read only, 2 write only.  NT: non-temporal loads and stores.  `key` is 0 at run time; it keeps
// the compiler from proving anything about the values moved.
template <int MODE, bool NT>
__global__ __launch_bounds__(kBlock) void stream_kernel(const uint4 *src, uint4 *dst, int64_t nvec, uint32_t key,
                                                        uint32_t *sink) {
  constexpr int U = 4;
  const int64_t stride = (int64_t)gridDim.x * kBlock * U;
  uint32_t acc = 0;
  for (int64_t base = ((int64_t)blockIdx.x * U) * kBlock + threadIdx.x; base < nvec; base += stride) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + (int64_t)u * kBlock;
      v[u] = make_uint4(key, key, key, key);
      if (MODE != 2 && i < nvec) v[u] = load16<NT>(src + i);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + (int64_t)u * kBlock;
      if (MODE == 1) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
      else if (i < nvec) {
        v[u].x ^= key;                             // 0 at run time: a store in place the compiler cannot drop
        store16<NT>(dst + i, v[u]);
      }
    }
  }
  if (MODE == 1 && acc == 0x9e3779b9u && key == 1u) sink[0] = acc;    // never true: the reads must still happen
}

struct PrefixArgs {
  unsigned char *a;        // the tensor read (and written, in place)
  unsigned char *b;        // out of place: the tensor written
  const int32_t *lens;
  int H, S;
  int es;                  // element size
  int packed;              // packed causal layout (common.hip.h) instead of [B,H,S,S]
  uint32_t key;
  uint32_t *sink;
};

// mode: 0 read and write back in place, 1 write only, 2 read only, 3 read a, write b.
// [B,H,S,S]: one lane group per row, 64 rows per workgroup; the group is 16, 32 or 64 lanes wide, whichever covers
// the workgroup's longest row in one trip of four 16-byte vectors per lane, so every lane has work and all of a
// row's bytes are in flight at once.  Packed layout: the rows of a unit lie back to back (each rounded up to 128
// bytes), so a unit's valid rows are ONE contiguous range and are moved as such, four vectors per lane and trip --
// the upper bound for any kernel on that layout (it also moves the few bytes between a row's last vector and the
// end of its 128-byte group).
template <int MODE, bool NT>
__global__ __launch_bounds__(kBlock) void prefix_kernel(PrefixArgs p) {
  constexpr int U = 4, ROWS = 64;
  const int unit = blockIdx.y, b = unit / p.H;
  const int ql = min(p.lens[b], p.S);
  uint32_t acc = 0;
  auto move = [&](const uint4 *src, uint4 *dst, int first, int step, int64_t nvec) {
    for (int64_t v0 = first; v0 < nvec; v0 += (int64_t)step * U) {
      uint4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = v0 + (int64_t)u * step;
        v[u] = make_uint4(p.key, p.key, p.key, p.key);
        if (MODE != 1 && i < nvec) v[u] = load16<NT>(src + i);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = v0 + (int64_t)u * step;
        if (MODE == 2) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
        else if (i < nvec) {
          v[u].x ^= p.key;                         // 0 at run time: an in-place store the compiler cannot drop
          store16<NT>(dst + i, v[u]);
        }
      }
    }
  };
  if (p.packed) {
    const int64_t unit_elems = p.es == 4 ? packed_row_start<4 * kPackedRowVectors>(p.S) : packed_row_start<8 * kPackedRowVectors>(p.S);
    const int64_t valid_elems = p.es == 4 ? packed_row_start<4 * kPackedRowVectors>(ql) : packed_row_start<8 * kPackedRowVectors>(ql);
    const int64_t nvec = valid_elems * p.es / 16;
    const int64_t first = (int64_t)blockIdx.x * kBlock * U;        // this workgroup's share: kBlock * U vectors
    if (first >= nvec) return;
    const int64_t off = (int64_t)unit * unit_elems * p.es + first * 16;
    move(reinterpret_cast<const uint4 *>(p.a + off), reinterpret_cast<uint4 *>((MODE == 3 ? p.b : p.a) + off), threadIdx.x,
         kBlock, min(nvec - first, (int64_t)kBlock * U));
  } else {
    const int q0 = blockIdx.x * ROWS;
    if (q0 >= ql) return;
    const int q_last = min(q0 + ROWS, ql) - 1;
    const int nv_max = ((q_last + 1) * p.es + 15) / 16;
    const int lpr = nv_max <= 16 * U ? 16 : (nv_max <= 32 * U ? 32 : 64);
    const int lane = threadIdx.x % lpr, grp = threadIdx.x / lpr;
    for (int q = q0 + grp; q <= q_last; q += kBlock / lpr) {
      const int64_t off = ((int64_t)unit * p.S + q) * p.S * p.es;
      move(reinterpret_cast<const uint4 *>(p.a + off), reinterpret_cast<uint4 *>((MODE == 3 ? p.b : p.a) + off), lane, lpr,
           ((q + 1) * p.es + 15) / 16);
    }
  }
  if (MODE == 2 && acc == 0x9e3779b9u && p.key == 1u) p.sink[0] = acc;
}

// The causal prefixes read the way the attention kernels walk them: a workgroup takes a tile of 128 rows and moves
// along the keys in steps of 128 bytes per row (64 fp16 keys), every row as far as its own prefix goes, so that one
// step touches 128 pieces of 128 bytes, a row pitch apart (PV reads its probabilities so; QK^T writes its scores
// so).  Eight lanes per row piece, four rows per lane and step, the next step's loads in flight while this one's
// are consumed.  `lds_bytes` of dynamic LDS that nothing uses limit the workgroups per CU to what a kernel holding
// that much would have (48 KB: three per CU).  es = 2 only.
template <bool NT, int PIECE = 128>
__global__ __launch_bounds__(kBlock) void prefix_tile_walk_kernel(PrefixArgs p) {
  extern __shared__ unsigned char unused_lds[];
  constexpr int ROWS = 128;                     // rows per tile; PIECE: bytes per row and step
  constexpr int LPP = PIECE / 16, GROUPS = kBlock / LPP, RPL = ROWS / GROUPS;
  const int unit = blockIdx.y, b = unit / p.H;
  const int ql = min(p.lens[b], p.S);
  const int q0 = (int)blockIdx.x * ROWS;
  if (q0 >= ql) return;
  const int lane8 = threadIdx.x % LPP, rsub = threadIdx.x / LPP;
  const int64_t unit_elems = p.packed ? packed_row_start<8 * kPackedRowVectors>(p.S) : (int64_t)p.S * p.S;
  const unsigned char *base = p.a + unit * unit_elems * 2;
  int64_t off[RPL];
  int row_bytes[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int q = q0 + rsub + GROUPS * i;
    off[i] = (p.packed ? packed_row_start<8 * kPackedRowVectors>(q) : (int64_t)q * p.S) * 2 + lane8 * 16;
    row_bytes[i] = q < ql ? (q + 1) * 2 - lane8 * 16 : 0;           // bytes of the prefix from this lane's chunk on
  }
  const int steps = (min(q0 + ROWS, ql) * 2 + PIECE - 1) / PIECE;
  uint32_t acc = 0;
  uint4 cur[RPL], nxt[RPL];
  auto fetch = [&](uint4 (&v)[RPL], int st) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      v[i] = make_uint4(0u, 0u, 0u, 0u);
      if (st * PIECE < row_bytes[i]) v[i] = load16<NT>(base + off[i] + (int64_t)st * PIECE);
    }
  };
  fetch(cur, 0);
  for (int st = 0; st < steps; ++st) {
    fetch(nxt, st + 1);
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
      acc ^= cur[i].x ^ cur[i].y ^ cur[i].z ^ cur[i].w;
      cur[i] = nxt[i];
    }
  }
  if (acc == 0x9e3779b9u && p.key == 1u) p.sink[0] = acc;
}

template <int MODE>
static void launch_stream(const void *src, void *dst, int64_t nvec, int nt, uint32_t *sink, hipStream_t s) {
  const int64_t want = ceil_div(nvec, (int64_t)kBlock * 4);
  const int grid = (int)(want < 256 * 16 ? want : 256 * 16);
  if (nt) stream_kernel<MODE, true><<<grid, kBlock, 0, s>>>((const uint4 *)src, (uint4 *)dst, nvec, 0u, sink);
  else stream_kernel<MODE, false><<<grid, kBlock, 0, s>>>((const uint4 *)src, (uint4 *)dst, nvec, 0u, sink);
}

template <int MODE>
static void launch_prefix(const PrefixArgs &p, int batch, int nt, hipStream_t s) {
  const int64_t unit_vecs = (p.es == 4 ? packed_row_start<4 * kPackedRowVectors>(p.S) : packed_row_start<8 * kPackedRowVectors>(p.S)) * p.es / 16;
  const dim3 grid((unsigned)(p.packed ? ceil_div(unit_vecs, (int64_t)kBlock * 4) : ceil_div(p.S, 64)), (unsigned)(batch * p.H), 1);
  if (nt) prefix_kernel<MODE, true><<<grid, kBlock, 0, s>>>(p);
  else prefix_kernel<MODE, false><<<grid, kBlock, 0, s>>>(p);
}

}  // namespace en

extern "C" {

int en_stream_yardstick(const void *src, void *dst, int64_t nbytes, int mode, int nontemporal, en_stream_t stream) {
  using namespace en;
  if (!dst || (mode != 2 && !src)) return EN_ERR_NULL;
  if (nbytes < 16 || (nbytes % 16) != 0) return EN_ERR_SHAPE;
  if (mode < 0 || mode > 2) return EN_ERR_UNSUPPORTED;
  if ((mode != 2 && !aligned_to(src, 16)) || !aligned_to(dst, 16)) return EN_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  const int64_t nvec = nbytes / 16;
  // read only: dst is never written (the sink condition cannot hold) but must be a valid address
  if (mode == 0) launch_stream<0>(src, dst, nvec, nontemporal, nullptr, s);
  else if (mode == 1) launch_stream<1>(src, dst, nvec, nontemporal, (uint32_t *)dst, s);
  else launch_stream<2>(src, dst, nvec, nontemporal, nullptr, s);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_prefix_yardstick(void *scores, void *scores_out, const int32_t *seq_lens, int batch, int head_num, int seq_len,
                        int packed, int mode, int nontemporal, int elem_size, en_stream_t stream) {
  using namespace en;
  if (!scores || !seq_lens || (mode == 3 && !scores_out)) return EN_ERR_NULL;
  if (batch < 1 || head_num < 1 || seq_len < 1 || (int64_t)batch * head_num > 65535) return EN_ERR_SHAPE;
  if (elem_size != 2 && elem_size != 4) return EN_ERR_DTYPE;
  if (mode < 0 || mode > 7) return EN_ERR_UNSUPPORTED;
  if (mode >= 4 && elem_size != 2) return EN_ERR_DTYPE;
  if (!packed && ((int64_t)seq_len * elem_size) % 16 != 0) return EN_ERR_ALIGN;     // rows start on 16-byte boundaries
  if (!aligned_to(scores, 16) || (scores_out && !aligned_to(scores_out, 16))) return EN_ERR_ALIGN;
  PrefixArgs p{(unsigned char *)scores, (unsigned char *)scores_out, seq_lens, head_num, seq_len, elem_size, packed ? 1 : 0,
               0u, (uint32_t *)scores};
  hipStream_t s = (hipStream_t)stream;
  if (mode >= 4) {      // 4: the tile walk with as many workgroups per CU as fit; 5: with three per CU
    const dim3 grid((unsigned)ceil_div(seq_len, 128), (unsigned)(batch * head_num), 1);
    const size_t lds = (mode == 5 || mode == 7) ? 48 * 1024 : 0;
    if (mode >= 6) {
      if (nontemporal) prefix_tile_walk_kernel<true, 256><<<grid, kBlock, lds, s>>>(p);
      else prefix_tile_walk_kernel<false, 256><<<grid, kBlock, lds, s>>>(p);
    } else if (nontemporal) prefix_tile_walk_kernel<true><<<grid, kBlock, lds, s>>>(p);
    else prefix_tile_walk_kernel<false><<<grid, kBlock, lds, s>>>(p);
    EN_RETURN_IF_LAUNCH_FAILED();
    return EN_OK;
  }
  switch (mode) {
    case 0: launch_prefix<0>(p, batch, nontemporal, s); break;
    case 1: launch_prefix<1>(p, batch, nontemporal, s); break;
    case 2: launch_prefix<2>(p, batch, nontemporal, s); break;
    default: launch_prefix<3>(p, batch, nontemporal, s); break;
  }
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // extern "C"
