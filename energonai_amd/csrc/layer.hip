// The whole padding-removal step behind one call: the seven ops
//   depad -> transpose_pad -> QK^T -> scale_mask_softmax -> PV -> transpose_depad -> residual + LayerNorm
// issued back to back on the caller's stream.  Nothing new is computed here -- every op runs the kernel
// its entry point runs -- but a Python caller pays for one foreign call instead of seven, which is what
// bounds small batches (seven calls cost about 60 us of host time, more than the GPU needs for a BERT-base
// batch of a few hundred tokens), and depad, which depends on nothing before the LayerNorm, shares the
// launch of transpose_pad: six launches.
#include "common.hip.h"

extern "C" int en_padding_removal_layer(const void *hidden_padded, const void *qkv_packed, const void *dense_out,
                                        const void *gamma, const void *beta, void *x_packed, void *qkv_padded,
                                        void *scores, void *ctx, void *ctx_packed, void *y,
                                        const int32_t *cu_seqlens, const int32_t *seq_lens, int batch,
                                        int max_seq_len, int head_num, int size_per_head, int64_t hidden,
                                        int64_t total_tokens, float scale, float eps, int causal, int left_padded,
                                        int attention_form, const int32_t *fold_depad_offsets, int dtype,
                                        en_stream_t stream) {
  using namespace en;
  if (!hidden_padded || !qkv_packed || !gamma || !beta || !ctx_packed || !y || !cu_seqlens || !seq_lens)
    return EN_ERR_NULL;
  if (!x_packed && !fold_depad_offsets) return EN_ERR_NULL;
  if (attention_form < 0 || attention_form > 2) return EN_ERR_UNSUPPORTED;
  if (attention_form != 2 && (!qkv_padded || !ctx)) return EN_ERR_NULL;
  if (attention_form == 0 && !scores) return EN_ERR_NULL;
  const int es = dtype_size(dtype);
  if (!es) return EN_ERR_DTYPE;
  if (total_tokens < 0 || hidden < 1) return EN_ERR_SHAPE;
  if (!dense_out && hidden != (int64_t)head_num * size_per_head) return EN_ERR_SHAPE;
  if (total_tokens == 0) return EN_OK;
  const int B = batch, S = max_seq_len, H = head_num, D = size_per_head;
  int rc = EN_OK;
  // depad depends on nothing the attention chain produces: with transpose_pad to run it shares that launch
  const bool depad_alone = !fold_depad_offsets && attention_form == 2;
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
                       stream);
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
                         out_strides, nullptr, nullptr, scale, causal, dtype, stream);
      if (rc) return rc;
    } else {
      rc = en_attn_qk(q, k, scores, seq_lens, nullptr, B, H, S, S, D, sb, sh, ss, sb, sh, ss, 1.0f, causal, dtype,
                      stream);
      if (rc) return rc;
      // the PV kernel reads a probability row only as far as its own query sees: no tail is written
      rc = en_scale_mask_softmax(scores, seq_lens, nullptr, B, H, S, S, scale, causal, 1, dtype, stream);
      if (rc) return rc;
      rc = en_attn_pv(scores, v, ctx, seq_lens, nullptr, B, H, S, S, D, sb, sh, ss, cb, ch, cs, causal, 0, dtype, stream);
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
