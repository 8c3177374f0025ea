// What the two fused attention kernels share: the argument block and two lane-level helpers.
#pragma once

#include "attn_common.hip.h"

namespace en {

// The lane's number in its wave, counted afresh (two VALU instructions) where a value derived from it is needed only
// now and then, instead of keeping that value in a register through the key loop: the kernel has none to spare.
__device__ __forceinline__ int lane_now() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
}

struct FusedArgs {
  AttnArgs base;             // a_ptr = q, b_ptr = k, out = ctx; q_s* = q strides, k_s* = k strides
  const void *v;
  int64_t v_sb, v_sh, v_ss;
  int64_t c_sb, c_sh, c_ss;
  const int32_t *q_row0;     // packed layout: first row of batch b in q / ctx (else null)
  const int32_t *k_row0;     // packed layout: first row of batch b in k / v (else null)
  float scale;
  int c_vec16;               // ctx rows may be written with 128-bit stores (16-byte aligned base and strides)
};

// Both halves of the wave get (x of lanes 0..31, x of lanes 32..63): one VALU swap, no LDS round trip.
__device__ __forceinline__ void halves_of(float x, float &lo, float &hi) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  lo = __uint_as_float(r[0]);
  hi = __uint_as_float(r[1]);
}

// fused_wide.hip: the kernel whose waves own 64 queries each (256-query workgroups), for heads of 65..128 channels.
constexpr int kWideQTile = 256;
int launch_fused_wide(int dtype, FusedArgs &fa, hipStream_t s);
// fused_f32.hip: fp32 storage, heads of up to 64 channels, 64-row query tiles.
int launch_fused_f32(FusedArgs &fa, hipStream_t s);

}  // namespace en
