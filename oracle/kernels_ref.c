/* Plain-C replay of the reference's CUDA kernels for the padding-removal path.
 *
 * TEST INFRASTRUCTURE ONLY: built by oracle/Makefile into
 * oracle/_build/liboracle_c.so and loaded by the tests through ctypes to pin
 * oracle/eager.py at sizes the pure-Python replay cannot reach.  The product
 * never links or loads it.
 *
 * Each function walks the reference launch grid with ordinary loops
 * (blockIdx -> outer loop, threadIdx -> inner loop) and applies the same index
 * arithmetic.  Element payloads are moved as raw bytes (elem_size 2 or 4) so
 * fp16/bf16/fp32 tensors are all covered bit-exactly.  Paths cited are relative
 * to the reference checkout, energonai/kernel/cuda_native/csrc/.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* transpose_pad_fusion_kernel.cu:58-84 */
void orc_transpose_pad(const void *src, void *dst, const int32_t *seq_lens, int batch_size, int seq_len,
                       int head_num, int size_per_head, int elem_size) {
  const char *s = (const char *)src;
  char *d = (char *)dst;
  const size_t row = (size_t)size_per_head * elem_size;
  for (long block = 0; block < (long)batch_size * head_num * seq_len; ++block) {
    int batch_index = (int)(block / ((long)head_num * seq_len));
    int head_index = (int)((block % ((long)head_num * seq_len)) / seq_len);
    int seq_index = (int)(block % seq_len);
    long sum_len = 0;
    for (int i = 0; i < batch_index; ++i) sum_len += seq_lens[i];
    if (seq_index >= seq_lens[batch_index]) {
      memset(d + (size_t)block * row, 0, row);
    } else {
      memcpy(d + (size_t)block * row,
             s + ((size_t)(sum_len + seq_index) * head_num + head_index) * row, row);
    }
  }
}

/* transpose_pad_fusion_kernel.cu:8-35; dst must arrive zeroed (wrapper.cpp:70) */
void orc_transpose_depad(const void *src, void *dst, const int32_t *seq_lens, int batch_size, int seq_len,
                         int head_num, int size_per_head, int elem_size) {
  const char *s = (const char *)src;
  char *d = (char *)dst;
  const size_t row = (size_t)size_per_head * elem_size;
  for (long block = 0; block < (long)batch_size * head_num * seq_len; ++block) {
    int batch_index = (int)(block / ((long)head_num * seq_len));
    int head_index = (int)((block % ((long)head_num * seq_len)) / seq_len);
    int seq_index = (int)(block % seq_len);
    if (seq_index >= seq_lens[batch_index]) continue;
    long sum_len = 0;
    for (int i = 0; i < batch_index; ++i) sum_len += seq_lens[i];
    memcpy(d + ((size_t)(sum_len + seq_index) * head_num + head_index) * row, s + (size_t)block * row, row);
  }
}

/* transpose_pad_fusion_kernel.cu:112-131 */
void orc_build_offsets(const int32_t *sequence_length, int batch_size, int max_seq_len, int32_t *valid_word_num,
                       int32_t *tmp_mask_offset) {
  int total_seq_len = 0, cum_offset = 0, index = 0;
  for (int i = 0; i < batch_size; i++) {
    const int seq_len = sequence_length[i];
    for (int j = 0; j < seq_len; j++) tmp_mask_offset[index++] = cum_offset;
    cum_offset += max_seq_len - seq_len;
    total_seq_len += seq_len;
  }
  valid_word_num[0] = total_seq_len;
}

/* transpose_pad_fusion_kernel.cu:142-156 */
void orc_remove_padding(const void *src, void *tgt, const int32_t *tmp_mask_offset, int32_t *mask_offset, int m,
                        int n, int elem_size) {
  const size_t row = (size_t)n * elem_size;
  for (int bid = 0; bid < m; ++bid) {
    mask_offset[bid] = tmp_mask_offset[bid];
    memcpy((char *)tgt + (size_t)bid * row, (const char *)src + (size_t)(bid + mask_offset[bid]) * row, row);
  }
}

/* transpose_pad_fusion_kernel.cu:178-189; tgt must arrive zeroed (wrapper.cpp:158) */
void orc_rebuild_padding(const void *src, void *tgt, const int32_t *mask_offset, int m, int n, int elem_size) {
  const size_t row = (size_t)n * elem_size;
  for (int bid = 0; bid < m; ++bid)
    memcpy((char *)tgt + (size_t)(bid + mask_offset[bid]) * row, (const char *)src + (size_t)bid * row, row);
}

/* transpose_pad_fusion_kernel.cu:213-236, one tensor */
void orc_transpose_rebuild_padding(const void *Q, void *q_buf, int seq_len, int head_num, int size_per_head,
                                   const int32_t *mask_offset, int valid_word_num, int elem_size) {
  const size_t row = (size_t)size_per_head * elem_size;
  for (int bid = 0; bid < valid_word_num; ++bid) {
    const int b = (bid + mask_offset[bid]) / seq_len;
    const int s = (bid + mask_offset[bid]) % seq_len;
    for (int h = 0; h < head_num; ++h)
      memcpy((char *)q_buf + (((size_t)b * head_num + h) * seq_len + s) * row,
             (const char *)Q + ((size_t)bid * head_num + h) * row, row);
  }
}

/* transpose_pad_fusion_kernel.cu:268-289 */
void orc_transpose_remove_padding(const void *src, void *dst, int seq_len, int head_num, int size_per_head,
                                  const int32_t *mask_offset, int valid_word_num, int elem_size) {
  const size_t row = (size_t)size_per_head * elem_size;
  for (int bid = 0; bid < valid_word_num; ++bid) {
    const int b = (bid + mask_offset[bid]) / seq_len;
    const int s = (bid + mask_offset[bid]) % seq_len;
    for (int h = 0; h < head_num; ++h)
      memcpy((char *)dst + ((size_t)bid * head_num + h) * row,
             (const char *)src + (((size_t)b * head_num + h) * seq_len + s) * row, row);
  }
}

/* scale_mask_softmax_kernel.cu:11-42 on fp32 storage, in place; -inf is the
 * reference's -1e8 (common.h:15); expf and true division stand in for the
 * reference's fast-math forms. */
void orc_softmax_f32(float *correlation, const int32_t *real_seq_len, int batch_size, int head_num,
                     int batch_seq_len) {
  const float NEG = -100000000.f;
  const int S = batch_seq_len;
  const long grid_y = (long)head_num * S;
  for (int bx = 0; bx < batch_size; ++bx)
    for (long by = 0; by < grid_y; ++by) {
      const int qpos = (int)(by % S);
      if (qpos >= real_seq_len[bx]) continue;
      float *row = correlation + ((size_t)bx * grid_y + by) * S;
      float mx = NEG;
      for (int t = 0; t < S; ++t) {
        float v = (t > qpos) ? NEG : row[t];
        mx = v > mx ? v : mx;
      }
      float sum = 0.f;
      for (int t = 0; t < S; ++t) {
        float e = (t > qpos) ? 0.f : expf(row[t] - mx);
        row[t] = e;
        sum += e;
      }
      for (int t = 0; t < S; ++t) row[t] = row[t] / sum;
    }
}

/* layer_norm_cuda_kernel.cu:14-41 */
static void welford(float curr, float *mu, float *sigma2, float *count) {
  *count = *count + 1.f;
  float delta = curr - *mu;
  float lmean = *mu + delta / *count;
  *mu = lmean;
  float delta2 = curr - lmean;
  *sigma2 = *sigma2 + delta * delta2;
}
static void chan(float muB, float sigma2B, float countB, float *mu, float *sigma2, float *count) {
  float delta = muB - *mu;
  float nA = *count, nB = countB;
  *count = *count + countB;
  float nX = *count;
  if (nX > 0.f) {
    nA = nA / nX;
    nB = nB / nX;
    *mu = nA * *mu + nB * muB;
    *sigma2 = *sigma2 + sigma2B + delta * delta * nA * nB * nX;
  } else {
    *mu = 0.f;
    *sigma2 = 0.f;
  }
}

/* layer_norm_cuda_kernel.cu:43-116,243-279 with the launch shape of :571-583
 * (block 32x4): 128 per-thread Welford streams over 4-element strides, five
 * rotating intra-warp Chan merges, then the inter-warp tree.  fp32 in and out. */
void orc_layer_norm_f32(float *out, float *mean, float *invvar, const float *vals, int n1, int n2, float eps,
                        const float *gamma, const float *beta) {
  enum { BX = 32, BY = 4, NUMX = BX * BY };
  for (int i1 = 0; i1 < n1; ++i1) {
    const float *lvals = vals + (size_t)i1 * n2;
    float mu[NUMX], s2[NUMX], cnt[NUMX];
    for (int thrx = 0; thrx < NUMX; ++thrx) {
      mu[thrx] = s2[thrx] = cnt[thrx] = 0.f;
      int l = 4 * thrx;
      for (; l + 3 < n2; l += 4 * NUMX)
        for (int k = 0; k < 4; ++k) welford(lvals[l + k], &mu[thrx], &s2[thrx], &cnt[thrx]);
      for (; l < n2; ++l) welford(lvals[l], &mu[thrx], &s2[thrx], &cnt[thrx]);
    }
    for (int y = 0; y < BY; ++y)
      for (int l = 0; l <= 4; ++l) {
        float muB[BX], s2B[BX], cB[BX];
        for (int x = 0; x < BX; ++x) {
          int srcLane = (x + (1 << l)) & 31;
          muB[x] = mu[y * BX + srcLane];
          s2B[x] = s2[y * BX + srcLane];
          cB[x] = cnt[y * BX + srcLane];
        }
        for (int x = 0; x < BX; ++x) chan(muB[x], s2B[x], cB[x], &mu[y * BX + x], &s2[y * BX + x], &cnt[y * BX + x]);
      }
    for (int offset = BY / 2; offset > 0; offset /= 2)
      for (int y = 0; y < offset; ++y)
        chan(mu[(y + offset) * BX], s2[(y + offset) * BX], cnt[(y + offset) * BX], &mu[y * BX], &s2[y * BX],
             &cnt[y * BX]);
    const float m = mu[0];
    const float sigma2 = s2[0] / (float)n2;
    const float c_invvar = 1.0f / sqrtf(sigma2 + eps);
    for (int i = 0; i < n2; ++i) out[(size_t)i1 * n2 + i] = gamma[i] * (c_invvar * (lvals[i] - m)) + beta[i];
    mean[i1] = m;
    invvar[i1] = c_invvar;
  }
}
