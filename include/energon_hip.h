/* energon_hip.h — C ABI of libenergon_hip.so (gfx950 / MI355X).
 *
 * One shared library replaces the reference's four pybind11 torch extensions
 * for the padding-removal path (energonai_transpose_pad, energonai_scale_mask,
 * energonai_layer_norm; reference setup.py:132-147).  Every entry point takes
 * raw device pointers, plain integer extents, a dtype tag and the HIP stream
 * to launch on; it never allocates, frees or retains device memory, never
 * synchronises the host, and returns 0 on success or a negative en_status.
 *
 * Paths cited below are relative to the reference checkout,
 * energonai/kernel/cuda_native/.
 */
#ifndef ENERGON_HIP_H
#define ENERGON_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *en_stream_t; /* a hipStream_t; NULL = the legacy default stream */

enum en_dtype { EN_F32 = 0, EN_F16 = 1, EN_BF16 = 2 };

enum en_status {
  EN_OK = 0,
  EN_ERR_NULL = -1,        /* a required pointer is NULL */
  EN_ERR_SHAPE = -2,       /* an extent is negative, zero where it may not be, or exceeds a kernel limit */
  EN_ERR_DTYPE = -3,       /* dtype tag or element size not supported by this entry point */
  EN_ERR_ALIGN = -4,       /* pointer or stride not aligned to the element size */
  EN_ERR_UNSUPPORTED = -5, /* valid request this build has no kernel for (message names it) */
  EN_ERR_HIP = -6,         /* the HIP runtime reported an error; see en_last_hip_error() */
  EN_ERR_SCRATCH = -7      /* the call needs more than EN_LAYER_SCRATCH_BYTES of the library's static scratch */
};

/* Library version (major*10000 + minor*100 + patch). */
int en_version(void);
/* Digest of the source files this library was compiled from (set by the build; "unknown" otherwise).  The
 * Python binding compares it with the sources beside it and refuses a library that is older than they are.
 * No counterpart in the reference, whose extensions are rebuilt by setup.py. */
const char *en_source_hash(void);
/* Static description of an en_status value. */
const char *en_status_string(int status);
/* hipError_t (as int) recorded by the last EN_ERR_HIP on this thread, and its text. */
int en_last_hip_error(void);
const char *en_last_hip_error_string(void);

/* ---- offsets ---------------------------------------------------------- */

/* cu_seqlens[b] = sum_{b'<b} seq_lens[b'], cu_seqlens[batch] = total.
 * Replaces the serial prefix loop every reference block runs
 * (csrc/transpose_pad_fusion_kernel.cu:24-27,70-73).  seq_lens is int32, or
 * int64 when lens_are_i64 != 0 (the reference test passes int64,
 * tests/test_kernel/test_transpose_pad_fusion_kernel.py:6); lens32_out, if not
 * NULL, receives the lengths as int32.  batch <= 65536. */
int en_prefix_sum(const void *seq_lens, int lens_are_i64, int batch, int32_t *cu_seqlens, int32_t *lens32_out,
                  en_stream_t stream);

/* ---- packing / unpacking (bit-exact, any 2- or 4-byte element) ---------- */

/* depad: [B,S,hid] -> [T,hid], valid rows only (transpose_pad.py:30-37).
 * left_padded != 0 takes rows S-len..S of each sequence instead of 0..len. */
int en_depad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len, int64_t hidden,
             int elem_size, int left_padded, en_stream_t stream);

/* repad: [T,hid] -> [B,S,hid], the inverse of en_depad with zeros in the padding
 * rows; the exit of the packed path (the reference callers use
 * ft_rebuild_padding for right-padded batches, examples/gpt/gpt.py:321-323, and
 * left-pad their generation batches, examples/opt/batch.py:12-24).  Every row
 * of dst is written. */
int en_repad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len, int64_t hidden,
             int elem_size, int left_padded, en_stream_t stream);

/* transpose_pad_wrapper (csrc/transpose_pad_fusion_wrapper.cpp:33-57, kernel
 * csrc/transpose_pad_fusion_kernel.cu:58-96): [T,H,Dk] -> [B,H,S,Dk]; every
 * byte of dst is written, padding rows as zero. */
int en_transpose_pad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len, int head_num,
                     int size_per_head, int elem_size, en_stream_t stream);

/* en_transpose_pad whose packed source holds src_head_rows rows of size_per_head
 * elements per token, of which rows src_head_first .. src_head_first+head_num-1
 * are moved: fills a [B,H,S,D] K or V cache from the k / v third of a fused
 * projection output without first copying that third out (the reference makes
 * the thirds contiguous with .contiguous(), energonai/model/attention.py:74).
 * zero_padding = 0 leaves rows s >= len[b] of dst untouched: for a destination
 * whose readers are bounded by the sequence lengths (the attention and decode
 * entry points here are), which saves the writes of the padding. */
int en_transpose_pad_heads(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len,
                           int head_num, int size_per_head, int src_head_rows, int src_head_first,
                           int zero_padding, int elem_size, en_stream_t stream);

/* transpose_depad_wrapper (wrapper.cpp:59-83, kernel.cu:8-46):
 * [B,H,S,D] -> [T,H,D]; every byte of dst is written when T = cu_seqlens[B]. */
int en_transpose_depad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len,
                       int head_num, int size_per_head, int elem_size, en_stream_t stream);

/* ft_build_padding_offsets_wrapper (wrapper.cpp:96-107, kernel.cu:112-139):
 * tmp_mask_offset[t] = sum_{b'<b(t)} (max_seq_len - len[b']) for each valid
 * token t; valid_word_num[0] = T.  seq_lens int32. */
int en_ft_build_offsets(const int32_t *seq_lens, int batch, int max_seq_len, int32_t *valid_word_num,
                        int32_t *tmp_mask_offset, en_stream_t stream);

/* row_offsets[t] = (row of token t in the padded [B*S] numbering) - t, for right- or
 * left-padded batches: the left-pad-aware form of the offsets above (the reference
 * assumes right padding, kernel.cu:118-130, while its generation batches are padded on
 * the left, examples/opt/batch.py:12-24).  row_offsets has sum(seq_lens) entries. */
int en_padding_offsets(const int32_t *seq_lens, int batch, int max_seq_len, int left_padded, int32_t *row_offsets,
                       en_stream_t stream);

/* ft_remove_padding_wrapper (wrapper.cpp:113-139, kernel.cu:142-166):
 * tgt[t,:] = src[t + tmp_mask_offset[t],:]; also copies the offsets into
 * mask_offset. */
int en_ft_remove_padding(const void *src, void *tgt, const int32_t *tmp_mask_offset, int32_t *mask_offset,
                         int valid_word_num, int64_t hidden, int elem_size, en_stream_t stream);

/* ft_rebuild_padding_wrapper (wrapper.cpp:146-172, kernel.cu:178-199):
 * tgt[B*S,hid]: row t + mask_offset[t] = src[t,:], all other rows zero; every
 * byte of tgt is written (no separate memset). */
int en_ft_rebuild_padding(const void *src, void *tgt, const int32_t *mask_offset, int valid_word_num,
                          int64_t hidden, int batch, int max_seq_len, int elem_size, en_stream_t stream);

/* ft_transpose_rebuild_padding_wrapper (wrapper.cpp:181-209, kernel.cu:213-255):
 * Q,K,V [T,H,D] -> caller-owned q_buf,k_buf,v_buf [B,H,S,D]; padding rows of the
 * buffers are not touched.  K/V (and their buffers) may be NULL to move one
 * tensor only.  No limit on H*D. */
int en_ft_transpose_rebuild(const void *Q, const void *K, const void *V, void *q_buf, void *k_buf, void *v_buf,
                            int batch, int seq_len, int head_num, int size_per_head, int valid_word_num,
                            const int32_t *mask_offset, int elem_size, en_stream_t stream);

/* ft_transpose_remove_padding_wrapper (wrapper.cpp:218-244, kernel.cu:268-305):
 * [B,H,S,D] -> [T,H*D]. */
int en_ft_transpose_remove(const void *src, void *dst, int valid_word_num, int batch, int seq_len, int head_num,
                           int size_per_head, const int32_t *mask_offset, int elem_size, en_stream_t stream);

/* ---- scale + mask + softmax ------------------------------------------- */

/* scale_mask_softmax_wrapper (csrc/scale_mask_softmax_wrapper.cpp:25-44, kernel
 * csrc/scale_mask_softmax_kernel.cu:11-57), in place on src [B,H,Sq,Sk].
 * For each b and each query row q < q_lens[b]: the first n visible entries
 * become softmax(scale * src[..., :n]) and the remaining Sk-n entries zero;
 * n = k_lens[b] when causal == 0, else min(k_lens[b], q + k_lens[b] - q_lens[b] + 1).
 * Rows q >= q_lens[b] are not touched (as in the reference, kernel.cu:14-17).
 * q_lens == NULL means q_lens[b] = min(k_lens[b], Sq).  tail_rows == 0 zeroes the
 * whole tail of every row as the reference does; tail_rows == t > 0 (a power of
 * two) zeroes a row only as far as the last row of its t-row query tile can see
 * and leaves the rest of the row untouched.  t = 1 writes the visible prefix
 * alone (to the end of its last 16-byte vector), which is all en_attn_pv reads.
 * The reference call is Sq == Sk, scale 1, causal 1, q_lens NULL, tail_rows 0.
 * No limit on Sk; fp32 math. */
int en_scale_mask_softmax(void *src, const int32_t *k_lens, const int32_t *q_lens, int batch, int head_num,
                          int q_seq_len, int k_seq_len, float scale, int causal, int tail_rows, int dtype,
                          en_stream_t stream);

/* Packed causal scores.  Under a causal mask of a self-attention batch row q of a (batch, head) unit holds
 * q + 1 visible scores; in [B,H,S,S] those prefixes start a whole row pitch apart and every kernel of the
 * chain QK^T -> softmax -> PV streams short ragged pieces of memory.  The packed layout keeps the prefixes only,
 * each rounded up to a whole group of 128 bytes, back to back.  With V = 128 / element size entries per group
 * (64 for fp16 / bf16, 32 for fp32) and t = q / V (integer division), row q of a unit starts
 *   row_start(q) = V * (V * t * (t + 1) / 2 + (q - V * t) * (t + 1))
 * elements into the unit and holds V * (t + 1) elements; every unit owns a slot as large as a full-length one,
 * row_start(seq_len) elements (seq_len = 1024, fp16: 557 056), unit (b, h) the slot b * head_num + h.
 * en_packed_scores_elems returns the elements of the whole tensor, batch * head_num * row_start(seq_len)
 * (0 on bad arguments).  Of a row's group the kernels write the visible prefix only: QK^T up to the end of the
 * 16-byte vector that holds the last visible score, the softmax zeros up to that same point; the rest of the
 * group is never written and never read.
 * An internal format of the step: the reference's [B,H,S,S] tensor (scale_mask_softmax_wrapper.cpp:25-44) stays
 * the format of en_scale_mask_softmax. */
int64_t en_packed_scores_elems(int batch, int head_num, int seq_len, int dtype);
/* en_scale_mask_softmax on packed causal scores, in place: row q < seq_lens[b] becomes softmax(scale * row[:q+1])
 * with zeros up to the end of its last vector; rows of padded queries do not exist.  seq_len <= 2048 (16-bit)
 * / 1024 (fp32); scale > 0. */
int en_scale_mask_softmax_packed(void *scores, const int32_t *seq_lens, int batch, int head_num, int seq_len,
                                 float scale, int dtype, en_stream_t stream);

/* ---- LayerNorm forward -------------------------------------------------- */

/* forward_affine (csrc/layer_norm_cuda.cpp:82-103, kernel
 * csrc/layer_norm_cuda_kernel.cu:243-279,571-601): rows [n1,n2];
 * x = in (+ residual, added in fp32, when residual != NULL);
 * out = gamma * (x - mean) * rsqrt(var + eps) + beta, biased variance, fp32
 * statistics, one rounding to out_dtype.  gamma/beta have out_dtype.
 * mean/invvar (fp32 [n1]) and sum_out (x rounded to in_dtype, [n1,n2]) are
 * optional (NULL to skip).  Supported (in,out): (f32,f32) (f32,f16) (f32,bf16)
 * (f16,f16) (bf16,bf16), the pairs of csrc/type_shim.h:26-73.
 * residual_row_offsets (device, n1 entries, or NULL): the residual of output row t is row
 * t + residual_row_offsets[t] of `residual`, which lets the kernel take it straight from the
 * padded [B,S,n2] activations (offsets from en_padding_offsets) instead of a depad copy. */
int en_layernorm_fwd(void *out, float *mean, float *invvar, void *sum_out, const void *in, const void *residual,
                     const int32_t *residual_row_offsets, const void *gamma, const void *beta, int64_t n1, int64_t n2,
                     float eps, int in_dtype, int out_dtype, en_stream_t stream);

/* ---- attention contractions (torch.matmul in the reference callers) ----- */

/* scores[b,h,i,j] = alpha * sum_d q[b,h,i,d] * k[b,h,j,d]
 * (examples/bert/bert.py:110, examples/gpt/gpt.py:109).  q/k are addressed as
 * base + b*stride_b + h*stride_h + s*stride_s + d (strides in elements), so
 * the chunk views of the fused [B,H,S,3D] buffer are passed without a copy.
 * scores is contiguous [B,H,Sq,Sk].  Only entries softmax will read are
 * written: rows i < q_lens[b], columns j < visible(i) rounded up to 16 bytes;
 * everything else in scores is left untouched.  q_lens NULL as above.
 * fp32 accumulation on MFMA; D a multiple of 8 (16-bit) / 4 (fp32), D <= 128.
 * q_row_offsets / k_row_offsets (device, batch entries, or NULL): q / k hold the valid rows of all sequences
 * back to back (the [1,T,H,3D] projection output of examples/bert/bert.py:100) and batch b starts at that row
 * (give stride_b = 0, stride_s = the token pitch): the contraction then needs no transpose_pad before it.
 * packed_scores != 0 (causal self-attention only: q_lens NULL, q_seq_len == k_seq_len; 16-bit dtypes): scores
 * are written in the packed layout of en_packed_scores_elems instead of [B,H,Sq,Sk].
 * tile_table (device, from en_attn_tile_table for the same k_lens, batch, head_num and q_seq_len, or NULL; q_lens
 * must be NULL with it): the order of the workgroups of the launch; same results, a shorter end of the launch. */
int en_attn_qk(const void *q, const void *k, void *scores, const int32_t *k_lens, const int32_t *q_lens, int batch,
               int head_num, int q_seq_len, int k_seq_len, int size_per_head, int64_t q_stride_b,
               int64_t q_stride_h, int64_t q_stride_s, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
               float alpha, int causal, int dtype, const int32_t *q_row_offsets, const int32_t *k_row_offsets,
               int packed_scores, const int32_t *tile_table, en_stream_t stream);

/* ctx[b,h,i,:] = sum_j p[b,h,i,j] * v[b,h,j,:]  (examples/bert/bert.py:119,
 * examples/gpt/gpt.py:125) over j < visible(i) only; p contiguous [B,H,Sq,Sk]
 * as left by en_scale_mask_softmax (any tail_rows: of row i only the 16-byte
 * vectors that hold a visible entry are read), v strided like k above, ctx
 * addressed with its own strides.  Rows i >= q_lens[b] of ctx are written as zero when
 * zero_padding != 0 and left untouched otherwise.
 * c_row_offsets / v_row_offsets as q_row_offsets / k_row_offsets of en_attn_qk: with c_row_offsets the context is
 * written as packed [T,H,D] rows (strides 0, D, H*D), which is what transpose_depad would produce
 * (zero_padding must then be 0: a packed tensor has no padding rows).  packed_scores and tile_table as in
 * en_attn_qk (the table is not used when zero_padding != 0). */
int en_attn_pv(const void *p, const void *v, void *ctx, const int32_t *k_lens, const int32_t *q_lens, int batch,
               int head_num, int q_seq_len, int k_seq_len, int size_per_head, int64_t v_stride_b,
               int64_t v_stride_h, int64_t v_stride_s, int64_t c_stride_b, int64_t c_stride_h, int64_t c_stride_s,
               int causal, int zero_padding, int dtype, const int32_t *c_row_offsets, const int32_t *v_row_offsets,
               int packed_scores, const int32_t *tile_table, en_stream_t stream);

/* Single-query forms of the two contractions for cached decode (one new token
 * per sequence against a ragged cache; the reference recomputes the whole
 * square each step, energonai/model/attention.py:61-71,106-118).
 * q [B,H,D] contiguous, k_cache/v_cache [B,H,Smax,D] with strides as above,
 * scores/p [B,H,Smax] contiguous, ctx [B,H,D] contiguous.  Streaming kernels:
 * bound by the K/V bytes read.  D a multiple of 8 (16-bit) / 4 (fp32), up to
 * 512 / 256; head sizes such as 80 and 96 are supported. */
int en_decode_qk(const void *q, const void *k_cache, void *scores, const int32_t *kv_lens, int batch, int head_num,
                 int k_seq_len, int size_per_head, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                 float alpha, int dtype, en_stream_t stream);
int en_decode_pv(const void *p, const void *v_cache, void *ctx, const int32_t *kv_lens, int batch, int head_num,
                 int k_seq_len, int size_per_head, int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                 int dtype, en_stream_t stream);

/* Both contractions and the softmax between them in one pass over the cache:
 * ctx[b,h,:] = sum_j softmax_j(scale * <q[b,h,:], k_cache[b,h,j,:]>) v_cache[b,h,j,:] over j < kv_lens[b].
 * The reference recomputes the whole square from a concatenated history on every step and keeps its last row
 * (energonai/model/attention.py:61-71,106-118); en_decode_qk -> en_scale_mask_softmax -> en_decode_pv compute the
 * same row in three launches with the scores passing through memory; here K and V are each read once and nothing
 * else touches memory.  q and ctx [B,H,D] contiguous; k_strides / v_strides point to three int64 in host memory
 * (batch, head, position strides in elements) of the [B,H,Smax,D] caches.  scale must be positive.  A sequence
 * with kv_lens[b] == 0 gets a zero row.  fp32 statistics and accumulation; dtypes and head sizes as
 * en_decode_qk.
 * workspace (device, 4-byte aligned, or NULL): a batch too small to fill the chip with one workgroup per
 * (batch, head) -- fewer than 512 such units -- has the keys of each unit shared between several workgroups, whose
 * partial results (fp32) pass through this buffer and are combined by a second small kernel;
 * en_decode_attn_workspace_bytes gives the size that asks for (0: no sharing for this shape).  With NULL, or fewer
 * bytes than that, every unit keeps one workgroup.  Nothing in the buffer has to be initialised or kept. */
int64_t en_decode_attn_workspace_bytes(int batch, int head_num, int k_seq_len, int size_per_head);
int en_decode_attn(const void *q, const void *k_cache, const void *v_cache, void *ctx, const int32_t *kv_lens, int batch,
                   int head_num, int k_seq_len, int size_per_head, const int64_t *k_strides, const int64_t *v_strides,
                   float scale, int dtype, void *workspace, int64_t workspace_bytes, en_stream_t stream);

/* Appends the new token's K and V rows to [B,H,Smax,D] caches at position
 * kv_lens[b] (the caller then adds one to kv_lens); replaces the reference's
 * torch.cat of the whole projection history on every step
 * (energonai/model/attention.py:66-71,89-98).  k_new / v_new are addressed as
 * base + b*new_stride_b + h*new_stride_h + d, the caches as
 * base + b*stride_b + h*stride_h + s*stride_s + d (elements of elem_size bytes).
 * A sequence with kv_lens[b] >= k_seq_len (or < 0) has no room: its rows are not written.  So that this cannot
 * go unnoticed, overflow (device, one int32, or NULL) counts such sequences: the kernel adds one to it for each
 * (the caller zeroes it when it likes and reads it when it likes; the call itself never synchronises). */
int en_kv_append(const void *k_new, const void *v_new, void *k_cache, void *v_cache, const int32_t *kv_lens,
                 int batch, int head_num, int k_seq_len, int size_per_head, int64_t new_stride_b,
                 int64_t new_stride_h, int64_t cache_stride_b, int64_t cache_stride_h, int64_t cache_stride_s,
                 int elem_size, int32_t *overflow, en_stream_t stream);

/* The K/V cache in pages (a further form of the cache that replaces the reference's concatenated history,
 * energonai/model/attention.py:61-71,89-98; the reference has no counterpart): K and V live in pools of
 * num_pages pages of page_size positions (a power of two, at least 16), page p, head h, row r, channel d at
 * p*strides[0] + h*strides[1] + r*strides[2] + d elements, e.g. a contiguous [num_pages, H, page_size, D] tensor.
 * page_table (device, int32 [batch, max_pages_per_seq]) names the pages of each sequence in order: position s of
 * sequence b is row s % page_size of page page_table[b][s / page_size].  Entries past a sequence's last page are
 * never followed; an id outside 0 .. num_pages-1 that a kernel does meet reads as zeros (attention) or leaves the
 * row unwritten and is counted in overflow (append, fill), so a wrong table cannot fault.  Sequences share the
 * pools, so memory is held for the positions in use, rounded up to pages, instead of batch * Smax.
 *   en_kv_fill_paged    prefill: rows cu_seqlens[b] .. of a packed [T, src_head_rows, D] source (heads
 *                       src_head_first .. +head_num-1, as en_transpose_pad_heads) to positions 0 .. len-1
 *   en_kv_append_paged  one new row per (batch, head) at position kv_lens[b], as en_kv_append
 *   en_decode_attn_paged  en_decode_attn over the pages (same kernel, the page a wave-uniform choice of buffer);
 *                       workspace as there, sized by en_decode_attn_workspace_bytes(batch, head_num,
 *                       max_pages_per_seq * page_size, size_per_head) */
int en_kv_fill_paged(const void *src, void *pool, const int32_t *cu_seqlens, const int32_t *page_table, int batch,
                     int max_seq_len, int head_num, int size_per_head, int src_head_rows, int src_head_first,
                     int max_pages_per_seq, int page_size, int num_pages, const int64_t *pool_strides, int elem_size,
                     int32_t *overflow, en_stream_t stream);
int en_kv_append_paged(const void *k_new, const void *v_new, void *k_pool, void *v_pool, const int32_t *kv_lens,
                       const int32_t *page_table, int batch, int head_num, int max_pages_per_seq, int page_size,
                       int num_pages, int size_per_head, int64_t new_stride_b, int64_t new_stride_h,
                       const int64_t *pool_strides, int elem_size, int32_t *overflow, en_stream_t stream);
int en_decode_attn_paged(const void *q, const void *k_pool, const void *v_pool, void *ctx, const int32_t *kv_lens,
                         const int32_t *page_table, int batch, int head_num, int max_pages_per_seq, int page_size,
                         int num_pages, int size_per_head, const int64_t *k_strides, const int64_t *v_strides, float scale,
                         int dtype, void *workspace, int64_t workspace_bytes, en_stream_t stream);

/* Fused attention (an addition: the reference callers run matmul, softmax, matmul,
 * examples/bert/bert.py:108-119): ctx[b,h,i,:] = sum_j softmax_j(scale * <q_i, k_j>) v[b,h,j,:]
 * over the keys row i may see (same rule as en_scale_mask_softmax), without ever
 * writing the [B,H,Sq,Sk] scores to memory.  q, k, v, ctx are addressed as
 * base + b*strides[0] + h*strides[1] + s*strides[2] + d (elements; each *_strides
 * points to three int64 in host memory).  Packed operands (all valid rows back
 * to back, as in the [1,T,H,3D] projection output of examples/bert/bert.py:100)
 * are addressed by passing q_row_offsets (for q and ctx) and/or k_row_offsets
 * (for k and v): device arrays of batch entries, the exclusive prefix of the
 * lengths; batch b then starts at row offsets[b] (give stride[0] = 0), so neither
 * transpose_pad before nor transpose_depad after is needed; q_seq_len / k_seq_len
 * are then upper bounds of the lengths.  Null offsets select the padded layout.
 * scale must be positive.  Rows i >= q_lens[b] of ctx are left untouched.  fp16 / bf16, fp32 accumulation and statistics; D a multiple of 8, D <= 128.
 * query_tile: query rows per workgroup.  128 = four waves of 32 queries; 256 = four waves of 64 queries (heads of
 * 65..128 channels only): half the LDS reads, tile loads and barriers per FLOP at two waves per SIMD instead of
 * three; 0 = what en_attn_fused_query_tile names for these arguments.  tile_table as in en_attn_qk, built for the
 * same query_tile. */
int en_attn_fused_query_tile(int q_seq_len, int k_seq_len, int size_per_head, int causal, int dtype);
int en_attn_fused(const void *q, const void *k, const void *v, void *ctx, const int32_t *k_lens,
                  const int32_t *q_lens, int batch, int head_num, int q_seq_len, int k_seq_len, int size_per_head,
                  const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                  const int64_t *c_strides, const int32_t *q_row_offsets, const int32_t *k_row_offsets, float scale,
                  int causal, int dtype, const int32_t *tile_table, int query_tile, en_stream_t stream);

/* Workgroup order for en_attn_qk, en_attn_pv and en_attn_fused on one batch of sequences (no counterpart in the
 * reference, whose callers run torch.matmul): table gets en_attn_tile_table_elems(batch, head_num, q_seq_len,
 * query_tile) int32 entries that list the query tiles of query_tile rows (128, or 256 for en_attn_fused with that
 * query_tile; 0 = 128) the sequences really have (min(seq_lens[b], q_seq_len) rows each), the
 * longest sequence first, so that the launch wastes no workgroup slots on tiles past a sequence's end and its long
 * workgroups start first.  tiles_first == 0 keeps the query tiles of a (batch, head) unit together (they share its
 * K and V in L2); tiles_first != 0 runs the last tiles of all units first, then the second-to-last ... (the better
 * order when a unit's K and V are small: about 256 KB or less).  Built once per batch and reused by every layer;
 * one small kernel on `stream`. */
int64_t en_attn_tile_table_elems(int batch, int head_num, int q_seq_len, int query_tile);
int en_attn_tile_table(const int32_t *seq_lens, int batch, int head_num, int q_seq_len, int tiles_first,
                       int query_tile, int32_t *table, en_stream_t stream);

/* ---- measurement helper ------------------------------------------------- */

/* The whole step in one call: depad, transpose_pad, QK^T, scale_mask_softmax, PV,
 * transpose_depad, residual + LayerNorm launched back to back on `stream`, each through
 * its own entry point above (the sequence of examples/bert/bert.py:54-62,91-134 with the
 * projections left to the caller).  One foreign call instead of seven for callers whose
 * per-call overhead matters (Python: about 60 us for the seven).  The caller owns every
 * buffer: x_packed [T,hid] (residual stream), qkv_padded [B,H,S,3D], scores [B,H,S,S],
 * ctx [B,H,S,D], ctx_packed [T,H*D], y [T,hid].  dense_out [T,hid], if not NULL, is what
 * the LayerNorm adds to x_packed instead of ctx_packed (the output projection lies between
 * the two in a real layer).  attention_form: 0 = the three separate ops, 1 = en_attn_fused
 * on the padded buffer (scores unused), 2 = en_attn_fused on the packed projections
 * (qkv_padded, scores and ctx unused), 3 = the three separate ops on the packed projections
 * (row offsets into qkv_packed and ctx_packed: transpose_pad and transpose_depad do not run;
 * qkv_padded and ctx unused), 4 = form 3 with the scores in the packed causal layout
 * (causal, 16-bit dtypes; scores needs en_packed_scores_elems elements).  fold_depad_offsets (en_padding_offsets of this
 * batch, or NULL): if given, depad is not run and x_packed may be NULL; the LayerNorm takes
 * its residual rows straight from hidden_padded.  gamma/beta in the activation dtype.  tile_table
 * (en_attn_tile_table for seq_lens, batch, head_num, max_seq_len, or NULL) is handed to the attention kernels of
 * forms 1 to 4. */
int en_padding_removal_layer(const void *hidden_padded, const void *qkv_packed, const void *dense_out,
                             const void *gamma, const void *beta, void *x_packed, void *qkv_padded, void *scores,
                             void *ctx, void *ctx_packed, void *y, const int32_t *cu_seqlens,
                             const int32_t *seq_lens, int batch, int max_seq_len, int head_num, int size_per_head,
                             int64_t hidden, int64_t total_tokens, float scale, float eps, int causal,
                             int left_padded, int attention_form, const int32_t *fold_depad_offsets, int dtype,
                             const int32_t *tile_table, en_stream_t stream);

/* en_padding_removal_layer for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Every
 * buffer en_padding_removal_layer takes from its caller besides the inputs and y -- cu_seqlens and the int32
 * lengths (computed here from seq_lens: int32, or int64 when lens_are_i64 != 0), the fold_depad offsets,
 * x_packed, qkv_padded, scores, ctx, ctx_packed -- lives in one static device array of
 * EN_LAYER_SCRATCH_BYTES inside the library, one copy per GPU, held until the process ends.  The pieces a
 * call needs (each rounded up to 256 bytes; e = element size, T = total_tokens):
 *   always                 (B+1)*4 + B*4 + T*H*D*e
 *   fold_depad != 0        + T*4                     else  + T*hidden*e
 *   attention_form 0 or 1  + B*H*S*3D*e + B*H*S*D*e
 *   attention_form 0 or 3  + B*H*S*S*e
 *   attention_form 4       + en_packed_scores_elems(B, H, S, dtype)*e
 * A call that needs more returns EN_ERR_SCRATCH before anything is launched.  Arguments otherwise as
 * en_padding_removal_layer (fold_depad != 0 stands for passing fold_depad_offsets).  No hipMalloc, hipFree
 * or other allocating call is made; the first call on a device looks up the array's address
 * (hipGetSymbolAddress), so make that call outside a stream capture.  Every call on a GPU uses that GPU's one
 * array: calls that overlap on the same GPU (two streams, two threads) race; calls on one stream do not.
 * Nothing in the array has to be cleared between calls. */
#define EN_LAYER_SCRATCH_BYTES (64ll << 20)
int en_padding_removal_layer_noalloc(const void *hidden_padded, const void *qkv_packed, const void *dense_out,
                                     const void *gamma, const void *beta, void *y, const void *seq_lens,
                                     int lens_are_i64, int batch, int max_seq_len, int head_num, int size_per_head,
                                     int64_t hidden, int64_t total_tokens, float scale, float eps, int causal,
                                     int left_padded, int attention_form, int fold_depad, int dtype,
                                     en_stream_t stream);

/* Plain device-to-device copy of nbytes (multiple of 16, 16-byte aligned) with
 * the same 128-bit access pattern the packing kernels use.  Used as the
 * bandwidth yardstick and to calibrate hardware byte counters. */
int en_copy_bytes(const void *src, void *dst, int64_t nbytes, en_stream_t stream);

/* Bandwidth yardsticks (measurement helpers like en_copy_bytes; no counterpart in the reference; no op of the
 * library calls them).  en_stream_yardstick moves one contiguous range of nbytes (multiple of 16): mode 0 copies
 * src to dst (dst == src: a pass in place), 1 only reads src (dst: any valid 16-byte aligned address, not written), 2 only writes dst;
 * nontemporal != 0 uses non-temporal loads and stores.  en_prefix_yardstick walks the causal prefixes of a score
 * tensor -- row q of (batch, head) unit u holds q + 1 elements, rows q < seq_lens[b] only -- in the [B,H,S,S]
 * layout or (packed != 0) the packed layout of en_packed_scores_elems: mode 0 reads every prefix and writes it
 * back in place (the pattern of en_scale_mask_softmax with tail_rows 1), 1 only writes (en_attn_qk), 2 only
 * reads (en_attn_pv), 3 reads scores and writes scores_out.  Whole 16-byte vectors are moved.  Modes 0-3 take each
 * row (packed: each unit) as one contiguous range.  Modes 4-7 (2-byte elements) only read, the way the attention
 * kernels walk a score tensor: one workgroup per tile of 128 rows, moving along the keys in steps of 128 bytes per
 * row (4, 5) or 256 bytes (6, 7), the next step's loads in flight while this step's are consumed; 5 and 7 hold
 * 48 KB of LDS per workgroup, i.e. three workgroups per CU as the attention kernels have. */
int en_stream_yardstick(const void *src, void *dst, int64_t nbytes, int mode, int nontemporal, en_stream_t stream);
int en_prefix_yardstick(void *scores, void *scores_out, const int32_t *seq_lens, int batch, int head_num, int seq_len,
                        int packed, int mode, int nontemporal, int elem_size, en_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ENERGON_HIP_H */
