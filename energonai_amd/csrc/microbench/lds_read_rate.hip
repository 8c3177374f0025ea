// LDS read throughput per CU for the fragment reads of the attention kernels (128-bit reads in the K tile's swizzled
// pattern, transposing 64-bit reads in the V tile's) against plain consecutive reads.  A measuring stick, not part of
// the library:
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/lds_read_rate energonai_amd/csrc/microbench/lds_read_rate.hip && /tmp/lds_read_rate
#include <hip/hip_runtime.h>
#include <cstdio>
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
template <int MODE>
__global__ __launch_bounds__(256) void k(int reps, float *sink) {
  __shared__ __attribute__((aligned(16))) char lds[49152];
  const int lane = threadIdx.x & 63;
  for (int i = threadIdx.x; i < 49152 / 4; i += 256) reinterpret_cast<int *>(lds)[i] = i;
  __syncthreads();
  u32x4 acc = {0, 0, 0, 0};
  // K-fragment pattern: lane (r, g): row r (256-byte rows), chunk (g ^ r & 15) ^ 2 vs
  const int r = lane & 31, g = lane >> 5;
  const unsigned kbase = r * 256 + ((g ^ (r & 15)) * 16);
  // V^T pattern of the transposing read
  const int tj = lane & 15, tg = (lane >> 4) & 1, vsw = tj >> 2;
  const unsigned vbase = ((4 * g + (tj >> 2)) * 256 + (2 * tg + ((tj >> 1) & 1)) * 16 + (tj & 1) * 8) ^ (64 * vsw);
  for (int it = 0; it < reps; ++it) {
    if (MODE == 0) {            // 16 x ds_read_b128 (one key tile of K fragments)
#pragma unroll
      for (int vs = 0; vs < 8; ++vs)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          const u32x4 v = *reinterpret_cast<const u32x4 *>(lds + ((kbase ^ (vs * 32)) + kb * 8192 + (it & 1) * 16384));
          acc ^= v;
        }
    } else if (MODE == 1) {     // 32 x ds_read_b64_tr_b16 (one key tile of V^T fragments)
#pragma unroll
      for (int gi = 0; gi < 4; ++gi)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh) {
            const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4 *)(__attribute__((address_space(3))) void *)(lds + ((vbase ^ (mt * 64)) + gi * 4096 + hh * 2048 + (it & 1) * 16384)));
            acc.x ^= (unsigned)v.x; acc.y ^= (unsigned)v.y; acc.z ^= (unsigned)v.z; acc.w ^= (unsigned)v.w;
          }
    } else if (MODE == 2) {     // 32 x plain ds_read_b64, each lane its own consecutive 8 bytes
#pragma unroll
      for (int j = 0; j < 32; ++j) {
        const uint2 v = *reinterpret_cast<const uint2 *>(lds + lane * 8 + j * 512 + (it & 1) * 16384);
        acc.x ^= v.x; acc.y ^= v.y;
      }
    } else {                    // 16 x ds_read_b128, each lane its own consecutive 16 bytes
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const u32x4 v = *reinterpret_cast<const u32x4 *>(lds + lane * 16 + j * 1024 + (it & 1) * 16384);
        acc ^= v;
      }
    }
  }
  if (acc.x == 0x12345678u) sink[0] = 1.f;
}
template <int MODE>
static void run(const char *name, int wgs, float *sink) {
  const int reps = 2000;
  hipEvent_t a, b; (void)hipEventCreate(&a); (void)hipEventCreate(&b);
  k<MODE><<<wgs, 256>>>(reps, sink);
  (void)hipDeviceSynchronize();
  (void)hipEventRecord(a);
  k<MODE><<<wgs, 256>>>(reps, sink);
  (void)hipEventRecord(b); (void)hipEventSynchronize(b);
  float ms; (void)hipEventElapsedTime(&ms, a, b);
  const double bytes = (double)wgs * 4 * reps * 16384.0;    // 16 KB per wave and repetition in every mode
  printf("%-52s %4d wgs: %8.1f us  %6.1f B/ns/CU\n", name, wgs, ms * 1e3, bytes / (ms * 1e6) / 256);
}
int main() {
  float *sink; (void)hipMalloc(&sink, 4);
  for (int wgs : {256, 512, 768}) {
    run<0>("K fragments: ds_read_b128, swizzled rows", wgs, sink);
    run<1>("V^T fragments: ds_read_b64_tr_b16", wgs, sink);
    run<2>("ds_read_b64, consecutive", wgs, sink);
    run<3>("ds_read_b128, consecutive", wgs, sink);
  }
  return 0;
}
