// Do the matrix pipe and the vector pipe of a SIMD work at the same time for two waves?  One workgroup of eight waves
// per CU (two waves per SIMD): waves 0..3 issue nothing but MFMAs (four independent accumulators), waves 4..7 nothing
// but vector arithmetic (fused multiply-adds and exp2, four independent chains).  Timed alone and together: if the
// pipes overlap, "together" takes as long as the slower of the two alone; if they take turns, as long as their sum.
// A second case puts both kinds of instruction into ONE wave's stream (after every MFMA a few vector instructions that
// do not depend on it), with one or two such waves per SIMD: does a wave's own vector work run in the shadow of its
// own MFMAs?  A third does the same with single named instructions (register operands only) behind the 32x32x16 and
// the 16x16x32 MFMA, to see whether the kind of instruction or the shape of the MFMA matters.
// A measuring stick for the fused attention kernel, not part of the library:
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/mfma_valu_coexec energonai_amd/csrc/microbench/mfma_valu_coexec.hip && /tmp/mfma_valu_coexec
#include <hip/hip_runtime.h>
#include <cstdio>
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));

template <bool EXP>
__global__ __launch_bounds__(512, 1) void k(int mode, int reps, int valu_per_rep, float *sink) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool mfma_wave = wave < 4;
  if ((mode == 0 && !mfma_wave) || (mode == 1 && mfma_wave)) return;
  if (mfma_wave) {
    floatx16 acc[4];
    for (int i = 0; i < 4; ++i)
      for (int x = 0; x < 16; ++x) acc[i][x] = 0.f;
    halfx8 a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(threadIdx.x * 0.001f + i); b[i] = (_Float16)(0.5f + i); }
    for (int r = 0; r < reps; ++r) {
#pragma unroll
      for (int j = 0; j < 8; ++j)               // 32 MFMAs per repetition: one key step of a wave of the fused kernel
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < 4; ++i)
      for (int x = 0; x < 16; ++x) s += acc[i][x];
    if (s == 12345.678f) sink[0] = s;
  } else {
    float v[4] = {threadIdx.x * 1e-3f, 0.1f, 0.2f, 0.3f};
    for (int r = 0; r < reps; ++r) {
      for (int j = 0; j < valu_per_rep / 4; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (EXP) v[i] = __builtin_amdgcn_exp2f(v[i]) * 0.5f - 0.25f;      // one exp2, one fused multiply-add
          else v[i] = __builtin_fmaf(v[i], 0.999f, 0.001f);
        }
      }
    }
    if (v[0] + v[1] + v[2] + v[3] == 12345.678f) sink[1] = v[0];
  }
}

// One or two waves per SIMD, every wave the same stream: after each of the 32 MFMAs of a repetition, PER vector
// instructions that do not depend on it (every second one an exp2 when EXP).  MODE 0: the MFMAs alone, 1: the vector
// instructions alone, 2: both.  MODE is a template argument so that no branch sits between the instructions.
template <int PER, bool EXP, int MODE>
__global__ __launch_bounds__(256, 2) void k_same_wave(int reps, float *sink) {
  floatx16 acc[4];
  for (int i = 0; i < 4; ++i)
    for (int x = 0; x < 16; ++x) acc[i][x] = 0.f;
  halfx8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(threadIdx.x * 0.001f + i); b[i] = (_Float16)(0.5f + i); }
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = threadIdx.x * 1e-3f + i;
  for (int r = 0; r < reps; ++r) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (MODE != 1) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
        if (MODE != 0) {
#pragma unroll
          for (int u = 0; u < PER; ++u) {
            if (EXP && (u & 1)) v[u & 7] = __builtin_amdgcn_exp2f(v[u & 7]);
            else v[u & 7] = __builtin_fmaf(v[u & 7], 0.999f, 0.001f);
          }
        }
        __builtin_amdgcn_sched_barrier(0);      // keep the order written here
      }
  }
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int x = 0; x < 16; ++x) s += acc[i][x];
  for (int i = 0; i < 8; ++i) s += v[i];
  if (s == 12345.678f) sink[0] = s;
}

template <int PER, bool EXP, int MODE>
static float run_same(int wgs, int reps, float *sink) {
  hipEvent_t a, b;
  (void)hipEventCreate(&a);
  (void)hipEventCreate(&b);
  k_same_wave<PER, EXP, MODE><<<wgs, 256>>>(reps, sink);
  (void)hipDeviceSynchronize();
  (void)hipEventRecord(a);
  k_same_wave<PER, EXP, MODE><<<wgs, 256>>>(reps, sink);
  (void)hipEventRecord(b);
  (void)hipEventSynchronize(b);
  float ms;
  (void)hipEventElapsedTime(&ms, a, b);
  return ms * 1e3f;
}

template <bool EXP>
static float run(int mode, int reps, int valu_per_rep, float *sink) {
  hipEvent_t a, b;
  (void)hipEventCreate(&a);
  (void)hipEventCreate(&b);
  k<EXP><<<256, 512>>>(mode, reps, valu_per_rep, sink);
  (void)hipDeviceSynchronize();
  (void)hipEventRecord(a);
  k<EXP><<<256, 512>>>(mode, reps, valu_per_rep, sink);
  (void)hipEventRecord(b);
  (void)hipEventSynchronize(b);
  float ms;
  (void)hipEventElapsedTime(&ms, a, b);
  return ms * 1e3f;
}

template <int PER, bool EXP>
static void same_wave_case(const char *what, int reps, float *sink) {
  for (int wgs : {256, 512}) {
    const float m = run_same<PER, EXP, 0>(wgs, reps, sink), v = run_same<PER, EXP, 1>(wgs, reps, sink), both = run_same<PER, EXP, 2>(wgs, reps, sink);
    printf("%d wave%s per SIMD, %s after each MFMA: MFMA alone %8.1f us, vector alone %8.1f us, interleaved %8.1f us (max %8.1f, sum %8.1f)\n",
           wgs / 256, wgs > 256 ? "s" : "", what, m, v, both, m > v ? m : v, m + v);
  }
}

typedef float floatx4 __attribute__((ext_vector_type(4)));
// OP: 0 fma with register operands, 1 add of two registers, 2 multiply by inline constant, 3 cvt_pk_f16_f32, 4 exp2, 5 max3, 6 v_mov/xor int
template <int OP>
__device__ __forceinline__ void vop(float (&v)[8], int u) {
  float &x = v[u & 7];
  const float y = v[(u + 1) & 7];
  if (OP == 0) asm volatile("v_fma_f32 %0, %0, %1, %0" : "+v"(x) : "v"(y));
  if (OP == 1) asm volatile("v_add_f32 %0, %0, %1" : "+v"(x) : "v"(y));
  if (OP == 2) asm volatile("v_mul_f32 %0, 0.5, %0" : "+v"(x));
  if (OP == 3) asm volatile("v_cvt_pk_f16_f32 %0, %0, %1" : "+v"(x) : "v"(y));
  if (OP == 4) asm volatile("v_exp_f32 %0, %0" : "+v"(x));
  if (OP == 5) asm volatile("v_max3_f32 %0, %0, %1, %1" : "+v"(x) : "v"(y));
  if (OP == 6) asm volatile("v_xor_b32 %0, 1, %0" : "+v"(x));
}

template <int SHAPE, int OP, int PER, int MODE>
__global__ __launch_bounds__(256, 2) void kk(int reps, float *sink) {
  floatx16 acc[4];
  floatx4 acc4[8];
  for (int i = 0; i < 4; ++i)
    for (int x = 0; x < 16; ++x) acc[i][x] = 0.f;
  for (int i = 0; i < 8; ++i)
    for (int x = 0; x < 4; ++x) acc4[i][x] = 0.f;
  halfx8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(threadIdx.x * 0.001f + i); b[i] = (_Float16)(0.5f + i); }
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = threadIdx.x * 1e-3f + i;
  for (int r = 0; r < reps; ++r) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (MODE != 1) {
          if (SHAPE == 32) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
          else {
            acc4[2 * i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc4[2 * i], 0, 0, 0);
          }
        }
        if (MODE != 0) {
#pragma unroll
          for (int u = 0; u < PER; ++u) vop<OP>(v, u);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (SHAPE == 16) {
          if (MODE != 1) acc4[2 * i + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc4[2 * i + 1], 0, 0, 0);
          if (MODE != 0) {
#pragma unroll
            for (int u = 0; u < PER; ++u) vop<OP>(v, u + PER);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
  }
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int x = 0; x < 16; ++x) s += acc[i][x];
  for (int i = 0; i < 8; ++i)
    for (int x = 0; x < 4; ++x) s += acc4[i][x];
  for (int i = 0; i < 8; ++i) s += v[i];
  if (s == 12345.678f) sink[0] = s;
}

template <int SHAPE, int OP, int PER, int MODE>
static float run1(int wgs, int reps, float *sink) {
  hipEvent_t a, b;
  (void)hipEventCreate(&a);
  (void)hipEventCreate(&b);
  kk<SHAPE, OP, PER, MODE><<<wgs, 256>>>(reps, sink);
  (void)hipDeviceSynchronize();
  (void)hipEventRecord(a);
  kk<SHAPE, OP, PER, MODE><<<wgs, 256>>>(reps, sink);
  (void)hipEventRecord(b);
  (void)hipEventSynchronize(b);
  float ms;
  (void)hipEventElapsedTime(&ms, a, b);
  return ms * 1e3f;
}
template <int SHAPE, int OP, int PER>
static void one(const char *what, float *sink) {
  const int reps = 10000;
  for (int wgs : {256, 512}) {
    const float m = run1<SHAPE, OP, PER, 0>(wgs, reps, sink), v = run1<SHAPE, OP, PER, 1>(wgs, reps, sink), both = run1<SHAPE, OP, PER, 2>(wgs, reps, sink);
    printf("mfma %2d, %d/SIMD, %d x %-10s per slot: MFMA %7.1f  vec %7.1f  both %7.1f  (max %7.1f sum %7.1f) hidden %4.0f%%\n", SHAPE, wgs / 256,
           SHAPE == 16 ? 2 * PER : PER, what, m, v, both, m > v ? m : v, m + v, 100.f * (m + v - both) / (m < v ? m : v));
    fflush(stdout);
  }
}
int main() {
  float *sink;
  (void)hipMalloc(&sink, 8);
  const int reps = 20000;
  // 32 MFMAs (1024 cycles of the matrix pipe) against 128..512 vector instructions per repetition
  for (int valu : {128, 256, 512}) {
    const float m = run<false>(0, reps, valu, sink), v = run<false>(1, reps, valu, sink), both = run<false>(2, reps, valu, sink);
    printf("32 MFMA | %3d fma          : MFMA alone %8.1f us, vector alone %8.1f us, together %8.1f us (max %8.1f, sum %8.1f)\n", valu, m, v,
           both, m > v ? m : v, m + v);
  }
  for (int valu : {64, 128, 256}) {
    const float m = run<true>(0, reps, valu, sink), v = run<true>(1, reps, valu, sink), both = run<true>(2, reps, valu, sink);
    printf("32 MFMA | %3d exp2 + %3d fma: MFMA alone %8.1f us, vector alone %8.1f us, together %8.1f us (max %8.1f, sum %8.1f)\n", valu,
           valu, m, v, both, m > v ? m : v, m + v);
  }
  same_wave_case<4, false>("4 fma", reps, sink);
  same_wave_case<8, false>("8 fma", reps, sink);
  same_wave_case<12, false>("12 fma", reps, sink);
  same_wave_case<4, true>("2 fma + 2 exp2", reps, sink);
  same_wave_case<8, true>("4 fma + 4 exp2", reps, sink);
  one<32, 0, 4>("fma", sink);
  one<32, 1, 4>("add", sink);
  one<32, 2, 4>("mul const", sink);
  one<32, 3, 4>("cvt_pk", sink);
  one<32, 4, 2>("exp", sink);
  one<32, 4, 4>("exp", sink);
  one<32, 5, 4>("max3", sink);
  one<32, 6, 4>("xor", sink);
  one<16, 0, 2>("fma", sink);
  one<16, 1, 2>("add", sink);
  one<16, 4, 1>("exp", sink);
  one<16, 4, 2>("exp", sink);
  return 0;
}
