// Shared host/device helpers for the gfx950 kernels: status bookkeeping,
// element traits for fp32/fp16/bf16 storage, 128-bit vector access and
// wave64 reductions built on DPP row operations.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "energon_hip.h"

namespace en {

constexpr int kWave = 64;       // gfx950 wavefront width
constexpr int kBlock = 256;     // default workgroup: 4 waves, one per SIMD
constexpr int kXcds = 8;        // MI355X: 8 XCDs, workgroups are dealt to them round-robin

// ---- host side ------------------------------------------------------------

int record_hip_error(hipError_t e);  // stores e for en_last_hip_error(), returns EN_ERR_HIP

#define EN_RETURN_IF_LAUNCH_FAILED()                      \
  do {                                                    \
    hipError_t en_e_ = hipGetLastError();                 \
    if (en_e_ != hipSuccess) return ::en::record_hip_error(en_e_); \
  } while (0)

inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int dtype_size(int dt) { return dt == EN_F32 ? 4 : ((dt == EN_F16 || dt == EN_BF16) ? 2 : 0); }

// ---- element traits ---------------------------------------------------------

typedef _Float16 half_t;

__device__ __forceinline__ float bf16_bits_to_float(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
// Round to nearest even in hardware (v_cvt_pk_bf16_f32 on gfx950; NaN stays NaN).
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

template <int DT> struct Elem;
template <> struct Elem<EN_F32> {
  typedef float T;
  static constexpr int kSize = 4;
  __device__ static __forceinline__ float to_float(T v) { return v; }
  __device__ static __forceinline__ T from_float(float f) { return f; }
  static constexpr uint32_t kNegInfWord = 0xff800000u;   // -inf in every element of a 32-bit word
};
template <> struct Elem<EN_F16> {
  typedef half_t T;
  static constexpr int kSize = 2;
  __device__ static __forceinline__ float to_float(T v) { return (float)v; }
  __device__ static __forceinline__ T from_float(float f) { return (T)f; }
  static constexpr uint32_t kNegInfWord = 0xfc00fc00u;
};
template <> struct Elem<EN_BF16> {
  typedef uint16_t T;
  static constexpr int kSize = 2;
  __device__ static __forceinline__ float to_float(T v) { return bf16_bits_to_float(v); }
  __device__ static __forceinline__ T from_float(float f) { return float_to_bf16_bits(f); }
  static constexpr uint32_t kNegInfWord = 0xff80ff80u;
};

// N elements of T moved as one access (N * sizeof(T) is 4, 8 or 16 bytes).
template <typename T, int N> struct alignas(sizeof(T) * N) Pack { T v[N]; };

template <typename T, int N>
__device__ __forceinline__ Pack<T, N> load_pack(const T *p) { return *reinterpret_cast<const Pack<T, N> *>(p); }
template <typename T, int N>
__device__ __forceinline__ void store_pack(T *p, const Pack<T, N> &x) { *reinterpret_cast<Pack<T, N> *>(p) = x; }

// Outputs at least this large cannot stay in the 256 MB memory-side cache for the
// consumer kernel anyway, so they are written with non-temporal stores (measured:
// +10..25 % on such tensors, -5 % when applied to small, cache-resident ones).
constexpr int64_t kStreamStoreBytes = 96ll << 20;
// Inputs are read with non-temporal loads only when the tensor moved is larger than the memory-side cache: a
// smaller one has often just been written by the kernel before and is served from that cache, and the policy then
// costs time (133 MB rows: depad 39 -> 47 us, LayerNorm 60 -> 72 us; 495 MB: 181 -> 175 us, 274 -> 268 us).
constexpr int64_t kStreamLoadBytes = 384ll << 20;

// 128-bit global accesses, optionally non-temporal (streamed once: do not keep in cache).
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ uint4 load16(const void *p) {
  if (NT) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
  }
  return *reinterpret_cast<const uint4 *>(p);
}
template <bool NT>
__device__ __forceinline__ void store16(void *p, const uint4 &v) {
  if (NT) {
    u32x4 x = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(x, reinterpret_cast<u32x4 *>(p));
  } else {
    *reinterpret_cast<uint4 *>(p) = v;
  }
}

// Buffer accesses with hardware bounds checking: a load whose offset lies outside
// [0, bytes) returns zero and a store there is dropped, so ragged edges need no
// branches and the compiler can count outstanding operations statically.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr uint32_t kOutOfRange = 0x80000000u;  // any offset >= 2^31 is outside every resource built here

__device__ __forceinline__ rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
// AUX is the cache-policy immediate of the instruction; 2 = non-temporal (streamed once).
template <int AUX = 0>
__device__ __forceinline__ uint4 buffer_load16(rsrc_t r, uint32_t byte_offset) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_offset, 0, AUX);
  return make_uint4(v.x, v.y, v.z, v.w);
}
template <int AUX = 0>
__device__ __forceinline__ void buffer_store16(rsrc_t r, uint32_t byte_offset, const uint4 &v) {
  const u32x4 x = {v.x, v.y, v.z, v.w};
  __builtin_amdgcn_raw_buffer_store_b128(x, r, (int)byte_offset, 0, AUX);
}

// Loads that go from memory straight into LDS, without passing through registers.  One instruction of a wave
// writes 64 x 16 bytes to consecutive LDS addresses starting at the (wave-uniform) byte address `lds_addr`:
// lane i's 16 bytes land at lds_addr + 16 i, whatever offset the lane reads from.  An offset outside the
// descriptor's range writes zeros.  The compiler does not see the LDS write: the caller waits with
// `s_waitcnt vmcnt(n)` (these loads count like any other) before a barrier that publishes the data.  A wait the
// compiler computes for its own loads and stores stays correct: operations it does not know of only make the
// counter larger, so its waits become stricter, never weaker.
typedef u32x4 desc_t;
__device__ __forceinline__ desc_t make_desc(const void *base, uint32_t bytes) {
  const uint64_t p = (uint64_t)(uintptr_t)base;
  return desc_t{(uint32_t)p, (uint32_t)(p >> 32), bytes, 0x00020000u};
}
__device__ __forceinline__ uint32_t lds_address(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}
// AUX 2 = non-temporal, as for the loads above.
template <int AUX = 0>
__device__ __forceinline__ void buffer_load16_to_lds(desc_t d, uint32_t lds_addr, uint32_t byte_offset) {
  // M0 carries the LDS address; one wait state separates its write from the load that reads it
  if constexpr (AUX == 2)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds"
                 :: "s"(lds_addr), "v"(byte_offset), "s"(d) : "memory");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(lds_addr), "v"(byte_offset), "s"(d) : "memory");
}

// Transposing LDS read of 16-bit elements.  Within each group of 16 lanes, lane j supplies the address of four
// consecutive elements; taking those sixteen pieces in lane order as one run of 64 elements, lane i receives
// elements i, i + 16, i + 32, i + 48 of the run: element i % 4 of the pieces of lanes i / 4, i / 4 + 4,
// i / 4 + 8 and i / 4 + 12.  Lanes that point at rows of a row-major tile (lane j at row j / 4, columns
// 4 (j % 4) .. + 3) thus receive a column each: lane i gets column i of rows 0..3.
typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 lds_read_tr16(const void *p) {
  const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4 *)(__attribute__((address_space(3))) void *)const_cast<void *>(p));
  return __builtin_bit_cast(uint2, v);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits
// for every outstanding global load and store of the wave, which would cancel
// any prefetch that is meant to stay in flight across the barrier.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- wave64 reductions --------------------------------------------------------
//
// Steps inside a 16-lane DPP row use quad_perm / row_half_mirror / row_mirror
// (no LDS traffic, full rate); the two steps that cross rows go through the
// LDS crossbar (ds_bpermute via __shfl_xor).  Every lane ends with the result.
// All lanes of the wave must be active at the call.

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

struct OpSum { __device__ static __forceinline__ float apply(float a, float b) { return a + b; } };
struct OpMax { __device__ static __forceinline__ float apply(float a, float b) { return fmaxf(a, b); } };

// Reduce over aligned groups of WIDTH lanes (WIDTH = 2..64, power of two).
template <typename Op, int WIDTH>
__device__ __forceinline__ float group_allreduce(float v) {
  static_assert(WIDTH >= 1 && WIDTH <= 64 && (WIDTH & (WIDTH - 1)) == 0, "WIDTH must be a power of two <= 64");
  if (WIDTH >= 2) v = Op::apply(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
  if (WIDTH >= 4) v = Op::apply(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
  if (WIDTH >= 8) v = Op::apply(v, dpp_move<0x141>(v));  // row_half_mirror
  if (WIDTH >= 16) v = Op::apply(v, dpp_move<0x140>(v)); // row_mirror
  if (WIDTH >= 32) v = Op::apply(v, __shfl_xor(v, 16, kWave));
  if (WIDTH >= 64) v = Op::apply(v, __shfl_xor(v, 32, kWave));
  return v;
}

template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v) { return group_allreduce<Op, 64>(v); }

// Reduce over a workgroup of NWAVES waves; `slots` is NWAVES floats of LDS
// owned by this reduction (a second reduction needs its own slots or a barrier).
template <typename Op, int NWAVES>
__device__ __forceinline__ float block_allreduce(float v, float *slots) {
  v = wave_allreduce<Op>(v);
  if (NWAVES == 1) return v;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  if (lane == 0) slots[wave] = v;
  __syncthreads();
  float r = slots[0];
#pragma unroll
  for (int w = 1; w < NWAVES; ++w) r = Op::apply(r, slots[w]);
  return r;
}

// ---- packed causal scores -------------------------------------------------------------------------------
// Under a causal mask of a self-attention batch row q of a (batch, head) unit holds q + 1 visible scores.  In the
// padded [B,H,S,S] layout those prefixes start a whole row pitch apart: a kernel that streams them touches short,
// ragged pieces of memory (measured: 4.7 TB/s for an in-place pass over them against 6.5 TB/s over one
// contiguous range).  The packed layout keeps only the prefixes, each rounded up to a whole group of V elements,
// back to back: row q starts at packed_row_start(q) elements into its unit and holds V * (q / V + 1) elements;
// every unit owns a slot of packed_row_start(S) elements, S the bucket length, whatever its length.  V is 128
// bytes' worth of elements (kPackedRowVectors 16-byte vectors): rows then start on cache-line boundaries, and a
// wave's 128-byte stores of a score tile each fill one line (with 16-byte groups the same stores straddled two
// lines and QK^T ran at 0.55 of its speed on the padded layout).
constexpr int kPackedRowVectors = 8;
template <int V>
__host__ __device__ __forceinline__ int64_t packed_row_start(int64_t q) {
  const int64_t t = q / V;
  return V * (V * t * (t + 1) / 2 + (q - V * t) * (t + 1));
}

// pad.hip: depad and transpose_pad (of all head_num rows per token; valid rows only when zero_padding == 0) in
// one launch when both move 16-byte multiples, as two launches otherwise.  Same results as en_depad followed
// by en_transpose_pad_heads.
int depad_and_transpose_pad(const void *hidden_padded, void *x_packed, const void *qkv_packed, void *qkv_padded,
                            const int32_t *cu_seqlens, int batch, int max_seq_len, int64_t hidden, int head_num,
                            int size_per_head, int elem_size, int left_padded, int zero_padding, hipStream_t stream);

}  // namespace en
