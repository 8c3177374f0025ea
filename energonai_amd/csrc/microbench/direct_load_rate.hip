// Throughput per CU of loads that go from memory straight into LDS against loads into registers (with and without a
// ds_write behind them), for data that sits in L1 / L2 (8 KB and 32 KB per workgroup) and beyond (1 MB per workgroup).
// A measuring stick for the attention kernels, not part of the library:
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/direct_load_rate energonai_amd/csrc/microbench/direct_load_rate.hip && /tmp/direct_load_rate
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 make_desc(const void *base, unsigned bytes) {
  const unsigned long long p = (unsigned long long)base;
  return u32x4{(unsigned)p, (unsigned)(p >> 32), bytes, 0x00020000u};
}
template <int MODE>
__global__ __launch_bounds__(256) void k(const char *src, size_t region, int reps, float *sink) {
  __shared__ __attribute__((aligned(16))) char lds[32768];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const char *base = src + (size_t)blockIdx.x * region;
  const u32x4 d = make_desc(base, (unsigned)region);
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char *)lds + wave * 1024;
  u32x4 acc = {0, 0, 0, 0};
  unsigned off = wave * 1024 + lane * 16;
  for (int r = 0; r < reps; ++r) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const unsigned o = (off + i * 4096) % (unsigned)region;
      if (MODE == 0) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds0 + i * 4096), "v"(o), "s"(d) : "memory");
      } else if (MODE == 3) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(lds0 + i * 4096 + j * 256), "v"((o & ~1023u) + j * 256 + lane * 4), "s"(d) : "memory");
      } else {
        u32x4 v;
        asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(v) : "v"(o), "s"(d) : "memory");
        if (MODE == 2) {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          *reinterpret_cast<u32x4 *>(lds + wave * 1024 + i * 4096 + lane * 16) = v;
        } else {
          asm volatile("s_waitcnt vmcnt(7)" ::: "memory");   // keeps eight in flight without reading the data early
          acc ^= v;
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    off += 32768;
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  if (acc.x == 0x12345678u && lds[threadIdx.x] == 77) sink[0] = 1.f;
}
template <int MODE>
static void run(const char *name, const char *src, size_t region, int wgs, int reps, float *sink) {
  hipEvent_t a, b; (void)hipEventCreate(&a); (void)hipEventCreate(&b);
  k<MODE><<<wgs, 256>>>(src, region, reps, sink);
  (void)hipDeviceSynchronize();
  (void)hipEventRecord(a);
  k<MODE><<<wgs, 256>>>(src, region, reps, sink);
  (void)hipEventRecord(b); (void)hipEventSynchronize(b);
  float ms; (void)hipEventElapsedTime(&ms, a, b);
  const double bytes = (double)wgs * reps * 32768.0;
  printf("%-34s region %7zu B x %4d wgs: %8.1f us  %7.2f TB/s  %6.1f B/clk/CU at 2.4 GHz\n", name, region, wgs, ms * 1e3, bytes / ms / 1e9,
         bytes / (ms * 1e-3) / 256 / 2.4e9);
}
int main() {
  const size_t total = 1ull << 30;
  char *src; (void)hipMalloc(&src, total); (void)hipMemset(src, 1, total);
  float *sink; (void)hipMalloc(&sink, 4);
  for (size_t region : {(size_t)8192, (size_t)32768, (size_t)1 << 20}) {
    for (int wgs : {256, 768}) {
      const int reps = 400;
      run<0>("to LDS, 16 bytes per lane", src, region, wgs, reps, sink);
      run<3>("to LDS, 4 bytes per lane", src, region, wgs, reps, sink);
      run<1>("to registers, 16 bytes per lane", src, region, wgs, reps, sink);
      run<2>("to registers, then ds_write", src, region, wgs, reps, sink);
    }
  }
  return 0;
}
