// MFMA building blocks shared by the attention kernels: per-dtype 32x32 MFMA
// step on 128-bit operand vectors, the argument block, and the mapping from
// workgroup id to (batch*head unit, query tile) that keeps a unit on one XCD.
#pragma once

#include "common.hip.h"

namespace en {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kQTile = 128;  // query rows per workgroup
constexpr int64_t kStreamScoreBytes = 512ll << 20;  // score tensors at least this large bypass the caches

// ---------------------------------------------------------------------------
// per-dtype MFMA step on one 128-bit vector per lane of each operand.
//   EPV  elements in a 128-bit vector
//   KPV  contraction indices consumed per vector step by the two lane groups
//   k_of contraction index held by element 0 of lane group g's vector at step vs
// A and B use the same mapping, so any bijection gives the same sum.
// ---------------------------------------------------------------------------
template <int DT> struct Mma;

template <> struct Mma<EN_F16> {
  static constexpr int EPV = 8, KPV = 16;
  __device__ static __forceinline__ int k_of(int vs, int g, int) { return vs * 16 + g * 8; }
  __device__ static __forceinline__ void step(const uint4 &a, const uint4 &b, floatx16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<EN_BF16> {
  static constexpr int EPV = 8, KPV = 16;
  __device__ static __forceinline__ int k_of(int vs, int g, int) { return vs * 16 + g * 8; }
  __device__ static __forceinline__ void step(const uint4 &a, const uint4 &b, floatx16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<EN_F32> {
  static constexpr int EPV = 4, KPV = 8;
  // lane group g owns the contiguous half [g*nvs*4, (g+1)*nvs*4) of the contraction range
  __device__ static __forceinline__ int k_of(int vs, int g, int nvs) { return g * nvs * 4 + vs * 4; }
  __device__ static __forceinline__ void step(const uint4 &a, const uint4 &b, floatx16 &c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
};

__device__ __forceinline__ uint4 zero4() { return make_uint4(0u, 0u, 0u, 0u); }

struct AttnArgs {
  const void *a_ptr;   // q (QK) or p (PV)
  const void *b_ptr;   // k (QK) or v (PV)
  void *out;           // scores (QK) or ctx (PV)
  const int32_t *k_lens;
  const int32_t *q_lens;
  int B, H, Sq, Sk, D;
  int64_t q_sb, q_sh, q_ss;  // strides of q (QK) / ctx (PV), elements
  int64_t k_sb, k_sh, k_ss;  // strides of k (QK) / v (PV), elements
  float alpha;
  int causal;
  int zero_padding;
  int vec_out;   // output rows may be written with 128-bit stores
  int ctx_vec16; // PV: ctx rows may be written with 128-bit stores (16-byte aligned base and strides)
  int ntq;       // query tiles per unit
  int units;     // B * H
  // Packed operands: batch b's rows start at row q_row0[b] (q in QK, ctx in PV) / k_row0[b] (k in QK, v in PV)
  // of a tensor that holds the valid rows of all sequences back to back; null = rows start at b * batch stride.
  const int32_t *q_row0;
  const int32_t *k_row0;
  int packed_scores;   // scores / probabilities are the packed causal prefixes (common.hip.h), not [B,H,Sq,Sk]
  const int32_t *tile_table;   // workgroup id -> unit * ntq + query tile, -1 = nothing (en_attn_tile_table); null: computed
};

// first element of (batch b, head h) in q / ctx and in k / v
__device__ __forceinline__ int64_t q_unit_offset(const AttnArgs &a, int b, int h) {
  return (int64_t)b * a.q_sb + (a.q_row0 ? (int64_t)a.q_row0[b] * a.q_ss : 0) + (int64_t)h * a.q_sh;
}
__device__ __forceinline__ int64_t k_unit_offset(const AttnArgs &a, int b, int h) {
  return (int64_t)b * a.k_sb + (a.k_row0 ? (int64_t)a.k_row0[b] * a.k_ss : 0) + (int64_t)h * a.k_sh;
}
// scores of a unit: first element, elements up to the start of row q, elements of the rows below ql
template <int EPV>
__device__ __forceinline__ int64_t score_unit_offset(const AttnArgs &a, int unit) {
  return (int64_t)unit * (a.packed_scores ? packed_row_start<EPV * kPackedRowVectors>(a.Sq) : (int64_t)a.Sq * a.Sk);
}
template <int EPV>
__device__ __forceinline__ int64_t score_row_offset(const AttnArgs &a, int q) {
  return a.packed_scores ? packed_row_start<EPV * kPackedRowVectors>(q) : (int64_t)q * a.Sk;
}

// workgroup id -> (unit, query tile): see the header comment.  With a tile table (built once per batch by
// en_attn_tile_table) the workgroups of the sequences' real query tiles come first, longest sequence first, and the
// rest of the grid finds -1 and leaves; without one every (unit, tile) pair of the padded shape has a workgroup and
// those past a sequence's end leave after reading its length.
__device__ __forceinline__ bool map_block(const AttnArgs &a, int &unit, int &qi) {
  const int bid = blockIdx.x;
  if (a.tile_table) {
    const int code = a.tile_table[bid];
    if (code < 0) return false;
    unit = code / a.ntq;
    qi = code - unit * a.ntq;
    return true;
  }
  const int xcd = bid % kXcds;
  const int slot = bid / kXcds;
  unit = (slot / a.ntq) * kXcds + xcd;
  qi = a.ntq - 1 - (slot % a.ntq);
  return unit < a.units;
}

__device__ __forceinline__ void seq_extents(const AttnArgs &a, int b, int &kl, int &ql) {
  kl = min(a.k_lens[b], a.Sk);
  ql = a.q_lens ? a.q_lens[b] : min(kl, a.Sq);
  ql = min(ql, a.Sq);
}

// keys the last valid query row of a tile may see
__device__ __forceinline__ int tile_key_extent(const AttnArgs &a, int q_last, int kl, int ql) {
  int n = a.causal ? min(kl, q_last + (kl - ql) + 1) : kl;
  return max(n, 0);
}

}  // namespace en
