// LayerNorm forward with an optional fused residual add.
//
// Single pass over HBM: each row is read once into VGPRs with 128-bit loads
// (TPR lanes share a row, VPL vectors per lane), the mean and then the
// centred sum of squares are reduced from the registers (two-pass statistics
// without a second trip to memory: wave64 DPP reductions, LDS only to combine
// waves), and the normalised row is written once.  All arithmetic is fp32 with
// a single rounding at the store.  Rows that do not fit the register tiling,
// or are not 16-byte aligned, take the three-pass workgroup-per-row kernel.
#include "common.hip.h"

#include <math.h>

namespace en {

struct LnArgs {
  void *out;
  float *mean;
  float *invvar;
  void *sum_out;
  const void *in;
  const void *residual;
  const int32_t *res_off;   // residual row of output row t is t + res_off[t] (null: t)
  const void *gamma;
  const void *beta;
  int64_t n1;
  int n2;
  float eps;
};

template <int DTI, int DTO, int VPL, int TPR, bool STREAM, bool STREAM_LD = false>
__global__ __launch_bounds__(TPR < kBlock ? kBlock : TPR) void layernorm_rows_kernel(LnArgs a) {
  typedef Elem<DTI> EI;
  typedef Elem<DTO> EO;
  typedef typename EI::T TI;
  typedef typename EO::T TO;
  constexpr int BLOCK = TPR < kBlock ? kBlock : TPR;
  constexpr int EPV = 16 / EI::kSize;  // elements per 128-bit input vector
  constexpr int NW = TPR / kWave;      // waves sharing a row
  constexpr int ROWS_PER_BLOCK = BLOCK / TPR;
  __shared__ float s_a[NW > 1 ? NW : 1];
  __shared__ float s_b[NW > 1 ? NW : 1];

  const int t = threadIdx.x % TPR;
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / TPR;
  const bool active = row < a.n1;  // uniform per wave (TPR is a multiple of 64)
  if (!active) return;             // ROWS_PER_BLOCK > 1 only when a row is one wave: no barrier follows

  const int nvec = a.n2 / EPV;
  const TI *in = reinterpret_cast<const TI *>(a.in) + row * a.n2;
  TI *sum_out = a.sum_out ? reinterpret_cast<TI *>(a.sum_out) + row * a.n2 : nullptr;

  // The row's own loads go out first: where the residual row is found through res_off, its address hangs on a
  // load of its own, and loads issue in order -- placed first it would hold the others back for its whole latency.
  uint4 raw[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int v = t + TPR * j;
    raw[j] = (v < nvec) ? load16<STREAM_LD>(in + v * EPV) : make_uint4(0u, 0u, 0u, 0u);
  }
  const TI *res = a.residual ? reinterpret_cast<const TI *>(a.residual) + (row + (a.res_off ? a.res_off[row] : 0)) * a.n2 : nullptr;

  float x[VPL][EPV];
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int v = t + TPR * j;
    if (v < nvec) {
      const Pack<TI, EPV> pk = __builtin_bit_cast(Pack<TI, EPV>, raw[j]);
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[j][e] = EI::to_float(pk.v[e]);
      if (res) {
        const Pack<TI, EPV> rk = __builtin_bit_cast(Pack<TI, EPV>, load16<STREAM_LD>(res + v * EPV));
#pragma unroll
        for (int e = 0; e < EPV; ++e) x[j][e] += EI::to_float(rk.v[e]);
      }
      if (sum_out) {
        Pack<TI, EPV> sk;
#pragma unroll
        for (int e = 0; e < EPV; ++e) sk.v[e] = EI::from_float(x[j][e]);
        store_pack<TI, EPV>(sum_out + v * EPV, sk);
      }
#pragma unroll
      for (int e = 0; e < EPV; ++e) s += x[j][e];
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) x[j][e] = 0.f;
    }
  }
  s = block_allreduce<OpSum, NW>(s, s_a);
  const float mu = s / (float)a.n2;
  float d2 = 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int v = t + TPR * j;
    if (v < nvec) {
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        const float d = x[j][e] - mu;
        d2 += d * d;
      }
    }
  }
  d2 = block_allreduce<OpSum, NW>(d2, s_b);
  const float var = d2 / (float)a.n2;
  const float inv = 1.0f / sqrtf(var + a.eps);

  const TO *gamma = reinterpret_cast<const TO *>(a.gamma);
  const TO *beta = reinterpret_cast<const TO *>(a.beta);
  TO *out = reinterpret_cast<TO *>(a.out) + row * a.n2;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int v = t + TPR * j;
    if (v < nvec) {
      const Pack<TO, EPV> g = load_pack<TO, EPV>(gamma + v * EPV);
      const Pack<TO, EPV> bt = load_pack<TO, EPV>(beta + v * EPV);
      Pack<TO, EPV> o;
#pragma unroll
      for (int e = 0; e < EPV; ++e)
        o.v[e] = EO::from_float((x[j][e] - mu) * inv * EO::to_float(g.v[e]) + EO::to_float(bt.v[e]));
      if constexpr (sizeof(TO) * EPV == 16) store16<STREAM>(out + v * EPV, __builtin_bit_cast(uint4, o));
      else store_pack<TO, EPV>(out + v * EPV, o);
    }
  }
  if (t == 0) {
    if (a.mean) a.mean[row] = mu;
    if (a.invvar) a.invvar[row] = inv;
  }
}

// Any n2, any alignment: one workgroup per row, three strided passes.
template <int DTI, int DTO>
__global__ __launch_bounds__(kBlock) void layernorm_generic_kernel(LnArgs a) {
  typedef Elem<DTI> EI;
  typedef Elem<DTO> EO;
  typedef typename EI::T TI;
  typedef typename EO::T TO;
  __shared__ float s_a[kBlock / kWave];
  __shared__ float s_b[kBlock / kWave];
  const int64_t row = blockIdx.x;
  const TI *in = reinterpret_cast<const TI *>(a.in) + row * a.n2;
  const TI *res = a.residual ? reinterpret_cast<const TI *>(a.residual) + (row + (a.res_off ? a.res_off[row] : 0)) * a.n2 : nullptr;
  TI *sum_out = a.sum_out ? reinterpret_cast<TI *>(a.sum_out) + row * a.n2 : nullptr;
  float s = 0.f;
  for (int i = threadIdx.x; i < a.n2; i += kBlock) {
    float v = EI::to_float(in[i]);
    if (res) v += EI::to_float(res[i]);
    s += v;
  }
  s = block_allreduce<OpSum, kBlock / kWave>(s, s_a);
  const float mu = s / (float)a.n2;
  float d2 = 0.f;
  for (int i = threadIdx.x; i < a.n2; i += kBlock) {
    float v = EI::to_float(in[i]);
    if (res) v += EI::to_float(res[i]);
    d2 += (v - mu) * (v - mu);
  }
  d2 = block_allreduce<OpSum, kBlock / kWave>(d2, s_b);
  const float inv = 1.0f / sqrtf(d2 / (float)a.n2 + a.eps);
  const TO *gamma = reinterpret_cast<const TO *>(a.gamma);
  const TO *beta = reinterpret_cast<const TO *>(a.beta);
  TO *out = reinterpret_cast<TO *>(a.out) + row * a.n2;
  for (int i = threadIdx.x; i < a.n2; i += kBlock) {
    float v = EI::to_float(in[i]);
    if (res) v += EI::to_float(res[i]);
    if (sum_out) sum_out[i] = EI::from_float(v);
    out[i] = EO::from_float((v - mu) * inv * EO::to_float(gamma[i]) + EO::to_float(beta[i]));
  }
  if (threadIdx.x == 0) {
    if (a.mean) a.mean[row] = mu;
    if (a.invvar) a.invvar[row] = inv;
  }
}

template <int DTI, int DTO, int VPL, int TPR>
static void launch_rows(const LnArgs &a, hipStream_t s) {
  constexpr int BLOCK = TPR < kBlock ? kBlock : TPR;
  constexpr int ROWS_PER_BLOCK = BLOCK / TPR;
  const unsigned grid = (unsigned)ceil_div(a.n1, ROWS_PER_BLOCK);
  // outputs too large to stay in the memory-side cache are written with non-temporal stores
  // and inputs too large to have stayed there are read with non-temporal loads
  const int64_t bytes = a.n1 * a.n2 * Elem<DTO>::kSize;
  if (bytes >= kStreamLoadBytes) layernorm_rows_kernel<DTI, DTO, VPL, TPR, true, true><<<grid, BLOCK, 0, s>>>(a);
  else if (bytes >= kStreamStoreBytes) layernorm_rows_kernel<DTI, DTO, VPL, TPR, true><<<grid, BLOCK, 0, s>>>(a);
  else layernorm_rows_kernel<DTI, DTO, VPL, TPR, false><<<grid, BLOCK, 0, s>>>(a);
}

template <int DTI, int DTO, int TPR>
static bool launch_vpl(const LnArgs &a, int vpl, hipStream_t s) {
  if (vpl <= 1) launch_rows<DTI, DTO, 1, TPR>(a, s);
  else if (vpl <= 2) launch_rows<DTI, DTO, 2, TPR>(a, s);
  else if (vpl <= 3) launch_rows<DTI, DTO, 3, TPR>(a, s);
  else if (vpl <= 4) launch_rows<DTI, DTO, 4, TPR>(a, s);
  else if (vpl <= 6) launch_rows<DTI, DTO, 6, TPR>(a, s);
  else if (vpl <= 8) launch_rows<DTI, DTO, 8, TPR>(a, s);
  else return false;
  return true;
}

template <int DTI, int DTO>
static int dispatch(const LnArgs &a, hipStream_t s) {
  constexpr int EPV = 16 / Elem<DTI>::kSize;
  constexpr int OUT_VEC_BYTES = EPV * Elem<DTO>::kSize;
  if (a.n1 > (int64_t)INT32_MAX) return EN_ERR_SHAPE;
  const bool vec_ok = (a.n2 % EPV) == 0 && aligned_to(a.in, 16) && aligned_to(a.out, OUT_VEC_BYTES) &&
                      aligned_to(a.gamma, OUT_VEC_BYTES) && aligned_to(a.beta, OUT_VEC_BYTES) &&
                      (!a.residual || aligned_to(a.residual, 16)) && (!a.sum_out || aligned_to(a.sum_out, 16));
  const int nvec = vec_ok ? a.n2 / EPV : 0;
  bool done = false;
  if (vec_ok) {
    if (nvec <= 2 * 64) done = launch_vpl<DTI, DTO, 64>(a, (nvec + 63) / 64, s);
    // at most four vectors per lane while the row fits 512 lanes: rows of 1025..2048 vectors measured 288 us
    // with 256 lanes x 6 vectors against 267 us with 512 lanes x 3 (20142 rows of 12288 fp16, residual added)
    // rows that would put four vectors on each of 256 lanes go to 512 lanes x 2 when there are many of them:
    // 7168-wide fp16 rows (896 vectors) x 9244: 60.6 -> 58.8 us, 8192-wide x 32768: 264 -> 256 us; with fewer
    // vectors (5120-wide: 48 -> 52 us) or few rows (2048 rows: 15.4 -> 16.3 us) 256 lanes stay ahead
    else if (nvec > 3 * 256 && nvec <= 4 * 256 && a.n1 >= 4096) done = launch_vpl<DTI, DTO, 512>(a, 2, s);
    else if (nvec <= 4 * 256) done = launch_vpl<DTI, DTO, 256>(a, (nvec + 255) / 256, s);
    else if (nvec <= 4 * 512) done = launch_vpl<DTI, DTO, 512>(a, (nvec + 511) / 512, s);
    else if (nvec <= 8 * 1024) done = launch_vpl<DTI, DTO, 1024>(a, (nvec + 1023) / 1024, s);
  }
  if (!done) layernorm_generic_kernel<DTI, DTO><<<(unsigned)a.n1, kBlock, 0, s>>>(a);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // namespace en

extern "C" int en_layernorm_fwd(void *out, float *mean, float *invvar, void *sum_out, const void *in,
                                const void *residual, const int32_t *residual_row_offsets, const void *gamma,
                                const void *beta, int64_t n1, int64_t n2, float eps, int in_dtype, int out_dtype,
                                en_stream_t stream) {
  using namespace en;
  if (!out || !in || !gamma || !beta) return EN_ERR_NULL;
  if (n1 < 0 || n2 < 1 || n2 > (int64_t)INT32_MAX) return EN_ERR_SHAPE;
  if (n1 == 0) return EN_OK;
  const int esi = dtype_size(in_dtype), eso = dtype_size(out_dtype);
  if (!esi || !eso) return EN_ERR_DTYPE;
  if (!aligned_to(in, esi) || !aligned_to(out, eso) || !aligned_to(gamma, eso) || !aligned_to(beta, eso) ||
      (residual && !aligned_to(residual, esi)) || (sum_out && !aligned_to(sum_out, esi)))
    return EN_ERR_ALIGN;
  if (residual_row_offsets && !residual) return EN_ERR_NULL;
  LnArgs a{out, mean, invvar, sum_out, in, residual, residual_row_offsets, gamma, beta, n1, (int)n2, eps};
  hipStream_t s = (hipStream_t)stream;
  if (in_dtype == EN_F32 && out_dtype == EN_F32) return dispatch<EN_F32, EN_F32>(a, s);
  if (in_dtype == EN_F32 && out_dtype == EN_F16) return dispatch<EN_F32, EN_F16>(a, s);
  if (in_dtype == EN_F32 && out_dtype == EN_BF16) return dispatch<EN_F32, EN_BF16>(a, s);
  if (in_dtype == EN_F16 && out_dtype == EN_F16) return dispatch<EN_F16, EN_F16>(a, s);
  if (in_dtype == EN_BF16 && out_dtype == EN_BF16) return dispatch<EN_BF16, EN_BF16>(a, s);
  return EN_ERR_DTYPE;
}
