// The whole padding-removal step behind one call: the seven ops
//   depad -> transpose_pad -> QK^T -> scale_mask_softmax -> PV -> transpose_depad -> residual + LayerNorm
// issued back to back on the caller's stream.  Nothing new is computed here -- every op runs the kernel
// its entry point runs -- but a Python caller pays for one foreign call instead of seven, which is what
// bounds small batches (seven calls cost about 60 us of host time, more than the GPU needs for a BERT-base
// batch of a few hundred tokens), and depad, which depends on nothing before the LayerNorm, shares the
// launch of transpose_pad: six launches.
#include "common.hip.h"

#include <initializer_list>
#include <mutex>

namespace en {

// Scratch of en_padding_removal_layer_noalloc: every intermediate that en_padding_removal_layer takes from its
// caller lives here instead.  One copy per GPU the library runs on, held until the process ends.
constexpr int64_t kLayerScratchBytes = EN_LAYER_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kLayerScratchBytes];

// In host code `scratch` is only a handle for hipGetSymbolAddress; the array's device address differs per GPU
// and is looked up once per device, with that device current.
constexpr int kMaxDevices = 64;
static unsigned char *g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

static int scratch_for_current_device(unsigned char **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return record_hip_error(e);
  if (dev < 0 || dev >= kMaxDevices) return EN_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return record_hip_error(e);
    if (!p) return EN_ERR_UNSUPPORTED;
    g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
  }
  *out = g_scratch_ptr[dev];
  return EN_OK;
}

// Lays out 256-byte aligned pieces of the scratch array: take() returns a piece's offset, or -1 for a piece the
// call does not need.  `used` may run past the end (checked by the caller before anything is launched) but never
// wraps: a piece that does not fit what is left pins it at one past the array's size, whatever follows.
struct Layout {
  int64_t used = 0;
  int64_t take(bool wanted, int64_t bytes) {
    if (!wanted) return -1;
    const int64_t at = used;
    if (bytes < 0 || used > kLayerScratchBytes || bytes > kLayerScratchBytes - used) used = kLayerScratchBytes + 1;
    else used += (bytes + 255) / 256 * 256;
    return at;
  }
};

// Product of extents that stops growing at one past the array's size, so that absurd shapes cannot wrap the
// signed arithmetic of a piece's size into something small.
static int64_t piece_bytes(std::initializer_list<int64_t> factors) {
  int64_t p = 1;
  for (int64_t f : factors) {
    if (f < 0) return -1;
    if (f == 0) return 0;
    if (p > (kLayerScratchBytes + 1) / f) return kLayerScratchBytes + 1;
    p *= f;
  }
  return p;
}

}  // namespace en

extern "C" int en_padding_removal_layer(const void *hidden_padded, const void *qkv_packed, const void *dense_out,
                                        const void *gamma, const void *beta, void *x_packed, void *qkv_padded,
                                        void *scores, void *ctx, void *ctx_packed, void *y,
                                        const int32_t *cu_seqlens, const int32_t *seq_lens, int batch,
                                        int max_seq_len, int head_num, int size_per_head, int64_t hidden,
                                        int64_t total_tokens, float scale, float eps, int causal, int left_padded,
                                        int attention_form, const int32_t *fold_depad_offsets, int dtype,
                                        const int32_t *tile_table, en_stream_t stream) {
  using namespace en;
  if (!hidden_padded || !qkv_packed || !gamma || !beta || !ctx_packed || !y || !cu_seqlens || !seq_lens)
    return EN_ERR_NULL;
  if (!x_packed && !fold_depad_offsets) return EN_ERR_NULL;
  if (attention_form < 0 || attention_form > 4) return EN_ERR_UNSUPPORTED;
  if (attention_form < 2 && (!qkv_padded || !ctx)) return EN_ERR_NULL;
  if ((attention_form == 0 || attention_form >= 3) && !scores) return EN_ERR_NULL;
  const int es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  if (total_tokens < 0 || hidden < 1) return EN_ERR_SHAPE;
  if (!dense_out && hidden != (int64_t)head_num * size_per_head) return EN_ERR_SHAPE;
  if (total_tokens == 0) return EN_OK;
  const int B = batch, S = max_seq_len, H = head_num, D = size_per_head;
  int rc = EN_OK;
  // depad depends on nothing the attention chain produces: with transpose_pad to run it shares that launch
  const bool depad_alone = !fold_depad_offsets && attention_form >= 2;
  if (depad_alone) {
    rc = en_depad(hidden_padded, x_packed, cu_seqlens, B, S, hidden, es, left_padded, stream);
    if (rc) return rc;
  }
  const unsigned char *qkv_bytes = static_cast<const unsigned char *>(qkv_padded);
  if (attention_form == 2) {
    // fused attention on the packed projections: no padded tensor at all
    const unsigned char *pk = static_cast<const unsigned char *>(qkv_packed);
    const int64_t in_strides[3] = {0, 3 * D, (int64_t)3 * H * D};
    const int64_t out_strides[3] = {0, D, (int64_t)H * D};
    rc = en_attn_fused(pk, pk + (int64_t)D * es, pk + (int64_t)2 * D * es, ctx_packed, seq_lens, nullptr, B, H, S, S, D,
                       in_strides, in_strides, in_strides, out_strides, cu_seqlens, cu_seqlens, scale, causal, dtype,
                       dtype == EN_F32 ? nullptr : tile_table, 0, stream);      // the fp32 kernel's tiles are not the table's
    if (rc) return rc;
  } else if (attention_form >= 3) {
    // The three kernels on the packed projections: q, k, v are read where the projection left them (batch b at
    // row cu_seqlens[b], token pitch 3*H*D) and the context is written as packed [T,H,D] rows, so neither
    // transpose_pad nor transpose_depad runs and no padded tensor exists.  Form 4 also keeps the scores packed.
    const unsigned char *pk = static_cast<const unsigned char *>(qkv_packed);
    const void *q = pk, *k = pk + (int64_t)D * es, *v = pk + (int64_t)2 * D * es;
    const int64_t th = 3 * D, ts = (int64_t)3 * H * D;
    const int packed_scores = attention_form == 4;
    rc = en_attn_qk(q, k, scores, seq_lens, nullptr, B, H, S, S, D, 0, th, ts, 0, th, ts, 1.0f, causal, dtype, cu_seqlens,
                    cu_seqlens, packed_scores, tile_table, stream);
    if (rc) return rc;
    if (packed_scores) rc = en_scale_mask_softmax_packed(scores, seq_lens, B, H, S, scale, dtype, stream);
    else rc = en_scale_mask_softmax(scores, seq_lens, nullptr, B, H, S, S, scale, causal, 1, dtype, stream);
    if (rc) return rc;
    rc = en_attn_pv(scores, v, ctx_packed, seq_lens, nullptr, B, H, S, S, D, 0, th, ts, 0, D, (int64_t)H * D, causal, 0,
                    dtype, cu_seqlens, cu_seqlens, packed_scores, tile_table, stream);
    if (rc) return rc;
  } else {
    // the attention entry points never read a row at or past a sequence's length: no zero fill of the padding
    if (fold_depad_offsets)
      rc = en_transpose_pad_heads(qkv_packed, qkv_padded, cu_seqlens, B, S, H, 3 * D, H, 0, 0, es, stream);
    else
      rc = depad_and_transpose_pad(hidden_padded, x_packed, qkv_packed, qkv_padded, cu_seqlens, B, S, hidden, H, 3 * D,
                                   es, left_padded, 0, (hipStream_t)stream);
    if (rc) return rc;
    // q, k, v are the thirds of the last dimension of the padded [B,H,S,3D] buffer
    const int64_t sb = (int64_t)H * S * 3 * D, sh = (int64_t)S * 3 * D, ss = 3 * D;
    const void *q = qkv_bytes, *k = qkv_bytes + (int64_t)D * es, *v = qkv_bytes + (int64_t)2 * D * es;
    const int64_t cb = (int64_t)H * S * D, ch = (int64_t)S * D, cs = D;
    if (attention_form == 1) {
      const int64_t in_strides[3] = {sb, sh, ss};
      const int64_t out_strides[3] = {cb, ch, cs};
      rc = en_attn_fused(q, k, v, ctx, seq_lens, nullptr, B, H, S, S, D, in_strides, in_strides, in_strides,
                         out_strides, nullptr, nullptr, scale, causal, dtype, dtype == EN_F32 ? nullptr : tile_table, 0,
                         stream);
      if (rc) return rc;
    } else {
      rc = en_attn_qk(q, k, scores, seq_lens, nullptr, B, H, S, S, D, sb, sh, ss, sb, sh, ss, 1.0f, causal, dtype,
                      nullptr, nullptr, 0, tile_table, stream);
      if (rc) return rc;
      // the PV kernel reads a probability row only as far as its own query sees: no tail is written
      rc = en_scale_mask_softmax(scores, seq_lens, nullptr, B, H, S, S, scale, causal, 1, dtype, stream);
      if (rc) return rc;
      rc = en_attn_pv(scores, v, ctx, seq_lens, nullptr, B, H, S, S, D, sb, sh, ss, cb, ch, cs, causal, 0, dtype, nullptr,
                      nullptr, 0, tile_table, stream);
      if (rc) return rc;
    }
    rc = en_transpose_depad(ctx, ctx_packed, cu_seqlens, B, S, H, D, es, stream);
    if (rc) return rc;
  }
  // with the offsets the residual rows come straight out of the padded activations: no depad copy at all
  return en_layernorm_fwd(y, nullptr, nullptr, nullptr, dense_out ? dense_out : ctx_packed,
                          fold_depad_offsets ? hidden_padded : x_packed, fold_depad_offsets, gamma, beta, total_tokens,
                          hidden, eps, dtype, dtype, stream);
}

extern "C" int en_padding_removal_layer_noalloc(const void *hidden_padded, const void *qkv_packed, const void *dense_out,
                                                const void *gamma, const void *beta, void *y, const void *seq_lens,
                                                int lens_are_i64, int batch, int max_seq_len, int head_num,
                                                int size_per_head, int64_t hidden, int64_t total_tokens, float scale,
                                                float eps, int causal, int left_padded, int attention_form,
                                                int fold_depad, int dtype, en_stream_t stream) {
  using namespace en;
  if (!hidden_padded || !qkv_packed || !gamma || !beta || !y || !seq_lens) return EN_ERR_NULL;
  if (attention_form < 0 || attention_form > 4) return EN_ERR_UNSUPPORTED;
  const int64_t es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  if (batch < 1 || batch > 65536 || max_seq_len < 1 || head_num < 1 || size_per_head < 1 || hidden < 1 ||
      total_tokens < 0 || total_tokens > (int64_t)batch * max_seq_len)
    return EN_ERR_SHAPE;
  if (total_tokens == 0) return EN_OK;
  const int64_t B = batch, S = max_seq_len, H = head_num, D = size_per_head, T = total_tokens;
  // the same pieces, in the same roles, as the caller-owned buffers of en_padding_removal_layer
  Layout l;
  const bool padded = attention_form < 2;
  const int64_t o_cu = l.take(true, (B + 1) * 4), o_lens = l.take(true, B * 4);
  const int64_t o_offs = l.take(fold_depad != 0, piece_bytes({T, 4})), o_x = l.take(fold_depad == 0, piece_bytes({T, hidden, es}));
  // packed scores: a unit's slot is below S * (S + 128 bytes' worth) elements, so the product below bounds it
  const bool scores_fit = piece_bytes({B, H, S, S, es}) <= kLayerScratchBytes;
  const int64_t score_bytes = attention_form == 4
      ? (scores_fit ? en_packed_scores_elems(batch, head_num, max_seq_len, dtype) * es : kLayerScratchBytes + 1)
      : piece_bytes({B, H, S, S, es});
  const int64_t o_qkv = l.take(padded, piece_bytes({B, H, S, 3 * D, es}));
  const int64_t o_scores = l.take(attention_form == 0 || attention_form >= 3, score_bytes);
  const int64_t o_ctx = l.take(padded, piece_bytes({B, H, S, D, es})), o_ctxp = l.take(true, piece_bytes({T, H, D, es}));
  if (l.used > kLayerScratchBytes) return EN_ERR_SCRATCH;
  unsigned char *base = nullptr;   // the array's address on the current device; never the array's name
  int rc = scratch_for_current_device(&base);
  if (rc) return rc;
  auto at = [&](int64_t off) -> void * { return off < 0 ? nullptr : base + off; };
  int32_t *cu = static_cast<int32_t *>(at(o_cu)), *lens32 = static_cast<int32_t *>(at(o_lens));
  int32_t *offs = static_cast<int32_t *>(at(o_offs));
  rc = en_prefix_sum(seq_lens, lens_are_i64, batch, cu, lens32, stream);
  if (rc) return rc;
  if (fold_depad) {
    rc = en_padding_offsets(lens32, batch, max_seq_len, left_padded, offs, stream);
    if (rc) return rc;
  }
  // Nothing here has to start at zero: every kernel of the step writes what the next one reads, and reads are
  // bounded by the sequence lengths, so what an earlier (larger) call left in the array is never looked at.
  return en_padding_removal_layer(hidden_padded, qkv_packed, dense_out, gamma, beta, at(o_x), at(o_qkv), at(o_scores),
                                  at(o_ctx), at(o_ctxp), y, cu, lens32, batch, max_seq_len, head_num,
                                  size_per_head, hidden, total_tokens, scale, eps, causal, left_padded, attention_form,
                                  offs, dtype, nullptr, stream);
}
