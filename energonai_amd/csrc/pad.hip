// Packing / unpacking kernels: depad, transpose_pad, transpose_depad and the
// ft_* offset family.  All of them are row gathers: an output row of `vpr`
// vectors is either a copy of one input row or zero.  One kernel body does the
// moving; a small "map" object per operation says, for each row of a block's
// tile, where it comes from and where it goes.  The map is evaluated once per
// row by the first lanes of the block and parked in LDS, so the per-sequence
// offsets are looked up once per tile instead of once per element, and the
// streaming loop is pure 128-bit loads and stores.
//
// Payloads are moved as raw bytes (vector type picked from row size and
// pointer alignment), so every 2- and 4-byte dtype is bit-exact by
// construction.
#include "common.hip.h"

namespace en {

constexpr int kMaxTileRows = 64;     // rows a block may own
// target vectors per block: 8 KiB at 16 B.  Many short-lived workgroups keep more independent rows in
// flight than few large ones (c3 transpose_pad: 227 us at 128 KiB, 203 us at 32 KiB, 190 us at 8 KiB)
constexpr int kTileVecs = 512;
constexpr int64_t kZeroRow = -1;     // source: write zeros
constexpr int64_t kSkipRow = -1;     // destination: leave untouched

struct Ptrs3 {
  const void *src[3];
  void *dst[3];
};

// ---------------------------------------------------------------------------
// maps: operator()(tile_x, tile_y, r, &src_row, &dst_row) in units of rows of
// the respective tensor; active(tile_x, tile_y) is a block-uniform early out.
// ---------------------------------------------------------------------------

// transpose_pad: grid.x = head + H * s_tile (heads fastest so that blocks in
// flight together read neighbouring pieces of the same packed token rows).
// The packed source may hold more head rows per token than are moved (Hs >= H rows, of
// which rows h0..h0+H-1 are taken): one third of a fused projection output, say.
struct PadMap {
  const int32_t *cu;
  int H, S, R, Hs, h0, zero;
  // without the zero fill, tiles that lie wholly in the padding of their sequence have nothing to write
  __device__ bool active(int tx, int b) const { return zero || (tx / H) * R < cu[b + 1] - cu[b]; }
  __device__ void operator()(int tx, int b, int r, int64_t &src, int64_t &dst) const {
    const int h = tx % H;
    const int s = (tx / H) * R + r;
    const int start = cu[b];
    const int len = cu[b + 1] - start;
    dst = (s < S && (zero || s < len)) ? ((int64_t)b * H + h) * S + s : kSkipRow;
    src = (s < len) ? ((int64_t)(start + s)) * Hs + h0 + h : kZeroRow;
  }
};

// transpose_depad: same tiling, opposite direction; tiles past the sequence end exit.
struct DepadHeadsMap {
  const int32_t *cu;
  int H, S, R;
  __device__ bool active(int tx, int b) const { return (tx / H) * R < cu[b + 1] - cu[b]; }
  __device__ void operator()(int tx, int b, int r, int64_t &src, int64_t &dst) const {
    const int h = tx % H;
    const int s = (tx / H) * R + r;
    const int start = cu[b];
    const int len = cu[b + 1] - start;
    src = ((int64_t)b * H + h) * S + s;
    dst = (s < len) ? ((int64_t)(start + s)) * H + h : kSkipRow;
  }
};

// depad: rows of the whole hidden width; grid.x = s_tile, grid.y = b.
struct DepadRowsMap {
  const int32_t *cu;
  int S, R, left;
  __device__ bool active(int tx, int b) const { return tx * R < cu[b + 1] - cu[b]; }
  __device__ void operator()(int tx, int b, int r, int64_t &src, int64_t &dst) const {
    const int s = tx * R + r;
    const int start = cu[b];
    const int len = cu[b + 1] - start;
    src = (int64_t)b * S + s + (left ? S - len : 0);
    dst = (s < len) ? (int64_t)start + s : kSkipRow;
  }
};

// repad: inverse of depad; every row of the padded output is written (copy or zeros).
struct RepadRowsMap {
  const int32_t *cu;
  int S, R, left;
  __device__ bool active(int, int) const { return true; }
  __device__ void operator()(int tx, int b, int r, int64_t &src, int64_t &dst) const {
    const int s = tx * R + r;
    const int start = cu[b];
    const int len = cu[b + 1] - start;
    const int i = s - (left ? S - len : 0);     // position inside the sequence
    dst = (s < S) ? (int64_t)b * S + s : kSkipRow;
    src = (i >= 0 && i < len) ? (int64_t)start + i : kZeroRow;
  }
};

// ft_remove_padding: tgt[t] = src[t + off[t]]; also publishes mask_offset[t].
struct FtRemoveMap {
  const int32_t *tmp_off;
  int32_t *mask_off;
  int valid, R;
  __device__ bool active(int, int) const { return true; }
  __device__ void operator()(int tx, int, int r, int64_t &src, int64_t &dst) const {
    const int t = tx * R + r;
    if (t < valid) {
      const int off = tmp_off[t];
      mask_off[t] = off;
      src = (int64_t)t + off;
      dst = t;
    } else {
      src = kZeroRow;
      dst = kSkipRow;
    }
  }
};

// ft_rebuild_padding: for each output row find the token t with t + off[t] == row
// (t + off[t] is strictly increasing in t), else the row is padding -> zero.
struct FtRebuildMap {
  const int32_t *off;
  int valid, rows_out, R;
  __device__ bool active(int, int) const { return true; }
  __device__ void operator()(int tx, int, int r, int64_t &src, int64_t &dst) const {
    const int row = tx * R + r;
    if (row >= rows_out) {
      src = kZeroRow;
      dst = kSkipRow;
      return;
    }
    int lo = 0, hi = valid;  // first t with t + off[t] >= row
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (mid + off[mid] < row) lo = mid + 1; else hi = mid;
    }
    dst = row;
    src = (lo < valid && lo + off[lo] == row) ? (int64_t)lo : kZeroRow;
  }
};

// ft_transpose_rebuild_padding: [T,H,D] -> [B,H,S,D]; grid.x = head + H * t_tile.
struct FtTransposeRebuildMap {
  const int32_t *off;
  int valid, H, S, R;
  __device__ bool active(int, int) const { return true; }
  __device__ void operator()(int tx, int, int r, int64_t &src, int64_t &dst) const {
    const int h = tx % H;
    const int t = (tx / H) * R + r;
    if (t < valid) {
      const int pos = t + off[t];
      const int b = pos / S, s = pos - b * S;
      src = (int64_t)t * H + h;
      dst = ((int64_t)b * H + h) * S + s;
    } else {
      src = kZeroRow;
      dst = kSkipRow;
    }
  }
};

// ft_transpose_remove_padding: the inverse gather.
struct FtTransposeRemoveMap {
  const int32_t *off;
  int valid, H, S, R;
  __device__ bool active(int, int) const { return true; }
  __device__ void operator()(int tx, int, int r, int64_t &src, int64_t &dst) const {
    const int h = tx % H;
    const int t = (tx / H) * R + r;
    if (t < valid) {
      const int pos = t + off[t];
      const int b = pos / S, s = pos - b * S;
      src = ((int64_t)b * H + h) * S + s;
      dst = (int64_t)t * H + h;
    } else {
      src = kZeroRow;
      dst = kSkipRow;
    }
  }
};

// ---------------------------------------------------------------------------
// the mover
// ---------------------------------------------------------------------------
template <typename Vec> __device__ __forceinline__ Vec zero_vec();
template <> __device__ __forceinline__ uint4 zero_vec<uint4>() { return make_uint4(0, 0, 0, 0); }
template <> __device__ __forceinline__ uint2 zero_vec<uint2>() { return make_uint2(0, 0); }
template <> __device__ __forceinline__ uint32_t zero_vec<uint32_t>() { return 0u; }
template <> __device__ __forceinline__ uint16_t zero_vec<uint16_t>() { return (uint16_t)0; }

// loads and stores of the mover; the 16-byte path has a non-temporal form for tensors too large to stay cached
// (a plain copy of 0.5 GB runs at 5.3 TB/s with the default policy, at 6.4 TB/s with non-temporal loads and stores)
template <typename Vec, bool STREAM> __device__ __forceinline__ void put(Vec *p, const Vec &v) {
  if constexpr (sizeof(Vec) == 16) store16<STREAM>(p, v);
  else *p = v;
}
template <typename Vec, bool STREAM> __device__ __forceinline__ Vec get(const Vec *p) {
  if constexpr (sizeof(Vec) == 16) return load16<STREAM>(p);
  else return *p;
}

// One tile of one operation: the first lanes evaluate the map for the tile's rows, then every lane streams
// 4 x 128-bit loads followed by 4 x 128-bit stores per step, for each of the NT tensors that share the map.
template <typename Vec, typename Map, int NT, bool STREAM, bool STREAM_LD = false>
__device__ __forceinline__ void gather_tile(const Map &map, const Ptrs3 &p, int vpr, int rows_per_block, int tx, int ty) {
  __shared__ int64_t s_src[kMaxTileRows];
  __shared__ int64_t s_dst[kMaxTileRows];
  const int tid = threadIdx.x;
  if (!map.active(tx, ty)) return;
  if (tid < rows_per_block) {
    int64_t so, dn;
    map(tx, ty, tid, so, dn);
    s_src[tid] = so < 0 ? so : so * vpr;
    s_dst[tid] = dn < 0 ? dn : dn * vpr;
  }
  __syncthreads();
  constexpr int U = 4;
  const int n = rows_per_block * vpr;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const Vec *__restrict__ src = reinterpret_cast<const Vec *>(p.src[t]);
    Vec *__restrict__ dst = reinterpret_cast<Vec *>(p.dst[t]);
    for (int i0 = tid; i0 < n; i0 += kBlock * U) {
      Vec v[U];
      int64_t d[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + u * kBlock;
        d[u] = kSkipRow;
        if (i < n) {
          const int r = i / vpr;
          const int c = i - r * vpr;
          const int64_t so = s_src[r];
          const int64_t dn = s_dst[r];
          if (dn >= 0) {
            d[u] = dn + c;
            v[u] = (so >= 0) ? get<Vec, STREAM_LD>(src + so + c) : zero_vec<Vec>();
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (d[u] >= 0) put<Vec, STREAM>(dst + d[u], v[u]);
    }
  }
}

template <typename Vec, typename Map, int NT, bool STREAM, bool STREAM_LD = false>
__global__ __launch_bounds__(kBlock) void row_gather_kernel(Map map, Ptrs3 p, int vpr, int rows_per_block) {
  gather_tile<Vec, Map, NT, STREAM, STREAM_LD>(map, p, vpr, rows_per_block, blockIdx.x, blockIdx.y);
}

// Two independent operations in one launch (128-bit rows, default store policy): workgroups [0, first_blocks)
// run the first operation's tiles, the rest the second's.  Small batches are bound by the fixed cost of a
// launch, and depad depends on nothing the attention chain produces, so it rides along with transpose_pad.
struct GatherPart {
  Ptrs3 p;
  int vpr, rows_per_block;
  unsigned grid_x;      // the operation's own grid is grid_x x grid_y; tiles are numbered x-fastest
};

template <typename MapA, typename MapB>
__global__ __launch_bounds__(kBlock) void row_gather_pair_kernel(MapA map_a, GatherPart a, MapB map_b, GatherPart b,
                                                                 unsigned first_blocks) {
  const unsigned id = blockIdx.x;
  if (id < first_blocks) gather_tile<uint4, MapA, 1, false>(map_a, a.p, a.vpr, a.rows_per_block, id % a.grid_x, id / a.grid_x);
  else gather_tile<uint4, MapB, 1, false>(map_b, b.p, b.vpr, b.rows_per_block, (id - first_blocks) % b.grid_x,
                                          (id - first_blocks) / b.grid_x);
}

// ---------------------------------------------------------------------------
// host-side launch helpers
// ---------------------------------------------------------------------------
static int pick_vec_bytes(int64_t row_bytes, const Ptrs3 &p, int nt) {
  int vb = 16;
  while (vb > 2) {
    bool ok = (row_bytes % vb) == 0;
    for (int t = 0; t < nt && ok; ++t) ok = aligned_to(p.src[t], vb) && aligned_to(p.dst[t], vb);
    if (ok) break;
    vb >>= 1;
  }
  return vb;
}

static int tile_rows(int64_t vpr, int64_t total_rows) {
  int64_t r = kTileVecs / (vpr > 0 ? vpr : 1);
  if (r < 1) r = 1;
  if (r > kMaxTileRows) r = kMaxTileRows;
  if (r > total_rows) r = total_rows > 0 ? total_rows : 1;
  return (int)r;
}

template <typename Map, int NT, typename MakeMap>
static int launch_row_gather(int64_t row_bytes, int64_t tile_dim_rows, int64_t out_bytes, const Ptrs3 &p,
                             MakeMap make_map, hipStream_t stream) {
  const int vb = pick_vec_bytes(row_bytes, p, NT);
  const int64_t vpr64 = row_bytes / vb;
  if (vpr64 > (int64_t)INT32_MAX / kMaxTileRows) return EN_ERR_SHAPE;
  const int vpr = (int)vpr64;
  const int R = tile_rows(vpr, tile_dim_rows);
  dim3 grid;
  const Map map = make_map(R, grid);
  if (grid.x == 0 || grid.y == 0) return EN_OK;
  if (grid.y > 65535u) return EN_ERR_SHAPE;
  switch (vb) {
    case 16:
      if (out_bytes >= kStreamLoadBytes) row_gather_kernel<uint4, Map, NT, true, true><<<grid, kBlock, 0, stream>>>(map, p, vpr, R);
      else if (out_bytes >= kStreamStoreBytes) row_gather_kernel<uint4, Map, NT, true><<<grid, kBlock, 0, stream>>>(map, p, vpr, R);
      else row_gather_kernel<uint4, Map, NT, false><<<grid, kBlock, 0, stream>>>(map, p, vpr, R);
      break;
    case 8: row_gather_kernel<uint2, Map, NT, false><<<grid, kBlock, 0, stream>>>(map, p, vpr, R); break;
    case 4: row_gather_kernel<uint32_t, Map, NT, false><<<grid, kBlock, 0, stream>>>(map, p, vpr, R); break;
    default: row_gather_kernel<uint16_t, Map, NT, false><<<grid, kBlock, 0, stream>>>(map, p, vpr, R); break;
  }
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

// ---------------------------------------------------------------------------
// ft_build_padding_offsets: one workgroup per sequence writes that sequence's
// run of offsets; the exclusive prefix of (S - len) is recomputed per block from
// the (short) length vector, 64 lengths per wave step.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void ft_build_offsets_kernel(const int32_t *__restrict__ lens, int batch,
                                                                  int max_seq_len, int32_t *__restrict__ valid,
                                                                  int32_t *__restrict__ tmp_off, int left_padded) {
  __shared__ int32_t s_tok[kBlock / kWave];
  __shared__ int32_t s_pad[kBlock / kWave];
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  // tokens and padding before sequence b (block 0 of the tail also totals everything)
  const int upto = (b == 0) ? batch : b;
  int32_t tok = 0, pad = 0;
  for (int i = tid; i < upto; i += kBlock) {
    const int32_t n = lens[i];
    tok += n;
    pad += max_seq_len - n;
  }
  for (int off = 32; off > 0; off >>= 1) {
    tok += __shfl_xor(tok, off, kWave);
    pad += __shfl_xor(pad, off, kWave);
  }
  if ((tid & 63) == 0) {
    s_tok[tid >> 6] = tok;
    s_pad[tid >> 6] = pad;
  }
  __syncthreads();
  tok = s_tok[0] + s_tok[1] + s_tok[2] + s_tok[3];
  pad = s_pad[0] + s_pad[1] + s_pad[2] + s_pad[3];
  if (b == 0) {
    if (tid == 0 && valid) valid[0] = tok;
    tok = 0;
    pad = 0;
  }
  const int32_t n = lens[b];
  if (left_padded) pad += max_seq_len - n;   // a left-padded sequence starts behind its own padding as well
  for (int j = tid; j < n; j += kBlock) tmp_off[tok + j] = pad;
}

static int check_elem(int elem_size) { return (elem_size == 2 || elem_size == 4) ? EN_OK : EN_ERR_DTYPE; }

int depad_and_transpose_pad(const void *hidden_padded, void *x_packed, const void *qkv_packed, void *qkv_padded,
                            const int32_t *cu_seqlens, int batch, int max_seq_len, int64_t hidden, int head_num,
                            int size_per_head, int elem_size, int left_padded, int zero_padding, hipStream_t stream) {
  if (!hidden_padded || !x_packed || !qkv_packed || !qkv_padded || !cu_seqlens) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (batch < 1 || max_seq_len < 1 || hidden < 1 || head_num < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  const Ptrs3 pd = {{hidden_padded, nullptr, nullptr}, {x_packed, nullptr, nullptr}};
  const Ptrs3 pt = {{qkv_packed, nullptr, nullptr}, {qkv_padded, nullptr, nullptr}};
  const int64_t rb_d = hidden * elem_size, rb_t = (int64_t)size_per_head * elem_size;
  const int64_t vpr_d = rb_d / 16, vpr_t = rb_t / 16;
  // Large outputs (the ones written with streaming stores) gain nothing from sharing a launch -- measured 1 %
  // slower on a 9 k-token batch of 7168-wide rows -- so only small batches, bound by launch cost, are paired.
  const bool st = (int64_t)batch * max_seq_len * head_num * size_per_head * elem_size >= kStreamStoreBytes;
  const bool sd = (int64_t)batch * max_seq_len * hidden * elem_size / 2 >= kStreamStoreBytes;
  const bool pair = !st && !sd && pick_vec_bytes(rb_d, pd, 1) == 16 && pick_vec_bytes(rb_t, pt, 1) == 16 &&
                    vpr_d <= (int64_t)INT32_MAX / kMaxTileRows && vpr_t <= (int64_t)INT32_MAX / kMaxTileRows;
  if (!pair) {   // the two entry points, one after the other
    const int rc = en_depad(hidden_padded, x_packed, cu_seqlens, batch, max_seq_len, hidden, elem_size, left_padded, stream);
    if (rc) return rc;
    return en_transpose_pad_heads(qkv_packed, qkv_padded, cu_seqlens, batch, max_seq_len, head_num, size_per_head,
                                  head_num, 0, zero_padding, elem_size, stream);
  }
  GatherPart gt{pt, (int)vpr_t, tile_rows(vpr_t, max_seq_len), 0u};
  GatherPart gd{pd, (int)vpr_d, tile_rows(vpr_d, max_seq_len), 0u};
  gt.grid_x = (unsigned)(ceil_div(max_seq_len, gt.rows_per_block) * head_num);
  gd.grid_x = (unsigned)ceil_div(max_seq_len, gd.rows_per_block);
  const int64_t n_t = (int64_t)gt.grid_x * batch, n_d = (int64_t)gd.grid_x * batch;
  if (n_t + n_d > INT32_MAX) return EN_ERR_SHAPE;
  const PadMap mt{cu_seqlens, head_num, max_seq_len, gt.rows_per_block, head_num, 0, zero_padding ? 1 : 0};
  const DepadRowsMap md{cu_seqlens, max_seq_len, gd.rows_per_block, left_padded ? 1 : 0};
  const unsigned grid = (unsigned)(n_t + n_d), first = (unsigned)n_t;   // transpose_pad, the larger one, goes first
  row_gather_pair_kernel<PadMap, DepadRowsMap><<<grid, kBlock, 0, stream>>>(mt, gt, md, gd, first);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

}  // namespace en

using namespace en;


extern "C" {

int en_depad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len, int64_t hidden,
             int elem_size, int left_padded, en_stream_t stream) {
  if (!src || !dst || !cu_seqlens) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (batch < 1 || max_seq_len < 1 || hidden < 1) return EN_ERR_SHAPE;
  if (!aligned_to(src, elem_size) || !aligned_to(dst, elem_size)) return EN_ERR_ALIGN;
  Ptrs3 p = {{src, nullptr, nullptr}, {dst, nullptr, nullptr}};
  return launch_row_gather<DepadRowsMap, 1>(hidden * elem_size, max_seq_len,
                                            (int64_t)batch * max_seq_len * hidden * elem_size / 2, p, [&](int R, dim3 &grid) {
    grid = dim3((unsigned)ceil_div(max_seq_len, R), (unsigned)batch, 1);
    return DepadRowsMap{cu_seqlens, max_seq_len, R, left_padded ? 1 : 0};
  }, (hipStream_t)stream);
}

int en_repad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len, int64_t hidden,
             int elem_size, int left_padded, en_stream_t stream) {
  if (!src || !dst || !cu_seqlens) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (batch < 1 || max_seq_len < 1 || hidden < 1) return EN_ERR_SHAPE;
  if (!aligned_to(src, elem_size) || !aligned_to(dst, elem_size)) return EN_ERR_ALIGN;
  Ptrs3 p = {{src, nullptr, nullptr}, {dst, nullptr, nullptr}};
  return launch_row_gather<RepadRowsMap, 1>(hidden * elem_size, max_seq_len,
                                            (int64_t)batch * max_seq_len * hidden * elem_size, p, [&](int R, dim3 &grid) {
    grid = dim3((unsigned)ceil_div(max_seq_len, R), (unsigned)batch, 1);
    return RepadRowsMap{cu_seqlens, max_seq_len, R, left_padded ? 1 : 0};
  }, (hipStream_t)stream);
}

int en_transpose_pad_heads(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len,
                           int head_num, int size_per_head, int src_head_rows, int src_head_first,
                           int zero_padding, int elem_size, en_stream_t stream) {
  if (!src || !dst || !cu_seqlens) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (batch < 1 || max_seq_len < 1 || head_num < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  if (src_head_first < 0 || src_head_rows < src_head_first + head_num) return EN_ERR_SHAPE;
  if (!aligned_to(src, elem_size) || !aligned_to(dst, elem_size)) return EN_ERR_ALIGN;
  Ptrs3 p = {{src, nullptr, nullptr}, {dst, nullptr, nullptr}};
  return launch_row_gather<PadMap, 1>((int64_t)size_per_head * elem_size, max_seq_len,
                                      (int64_t)batch * max_seq_len * head_num * size_per_head * elem_size, p, [&](int R, dim3 &grid) {
    grid = dim3((unsigned)(ceil_div(max_seq_len, R) * head_num), (unsigned)batch, 1);
    return PadMap{cu_seqlens, head_num, max_seq_len, R, src_head_rows, src_head_first, zero_padding ? 1 : 0};
  }, (hipStream_t)stream);
}

int en_transpose_pad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len, int head_num,
                     int size_per_head, int elem_size, en_stream_t stream) {
  return en_transpose_pad_heads(src, dst, cu_seqlens, batch, max_seq_len, head_num, size_per_head, head_num, 0, 1,
                                elem_size, stream);
}

int en_transpose_depad(const void *src, void *dst, const int32_t *cu_seqlens, int batch, int max_seq_len,
                       int head_num, int size_per_head, int elem_size, en_stream_t stream) {
  if (!src || !dst || !cu_seqlens) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (batch < 1 || max_seq_len < 1 || head_num < 1 || size_per_head < 1) return EN_ERR_SHAPE;
  if (!aligned_to(src, elem_size) || !aligned_to(dst, elem_size)) return EN_ERR_ALIGN;
  Ptrs3 p = {{src, nullptr, nullptr}, {dst, nullptr, nullptr}};
  return launch_row_gather<DepadHeadsMap, 1>((int64_t)size_per_head * elem_size, max_seq_len,
                                             (int64_t)batch * max_seq_len * head_num * size_per_head * elem_size / 2, p,
                                             [&](int R, dim3 &grid) {
    grid = dim3((unsigned)(ceil_div(max_seq_len, R) * head_num), (unsigned)batch, 1);
    return DepadHeadsMap{cu_seqlens, head_num, max_seq_len, R};
  }, (hipStream_t)stream);
}

int en_ft_build_offsets(const int32_t *seq_lens, int batch, int max_seq_len, int32_t *valid_word_num,
                        int32_t *tmp_mask_offset, en_stream_t stream) {
  if (!seq_lens || !valid_word_num || !tmp_mask_offset) return EN_ERR_NULL;
  if (batch < 1 || max_seq_len < 1) return EN_ERR_SHAPE;
  ft_build_offsets_kernel<<<batch, kBlock, 0, (hipStream_t)stream>>>(seq_lens, batch, max_seq_len, valid_word_num,
                                                                      tmp_mask_offset, 0);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_padding_offsets(const int32_t *seq_lens, int batch, int max_seq_len, int left_padded, int32_t *row_offsets,
                       en_stream_t stream) {
  if (!seq_lens || !row_offsets) return EN_ERR_NULL;
  if (batch < 1 || max_seq_len < 1) return EN_ERR_SHAPE;
  ft_build_offsets_kernel<<<batch, kBlock, 0, (hipStream_t)stream>>>(seq_lens, batch, max_seq_len, nullptr, row_offsets,
                                                                      left_padded ? 1 : 0);
  EN_RETURN_IF_LAUNCH_FAILED();
  return EN_OK;
}

int en_ft_remove_padding(const void *src, void *tgt, const int32_t *tmp_mask_offset, int32_t *mask_offset,
                         int valid_word_num, int64_t hidden, int elem_size, en_stream_t stream) {
  if (!src || !tgt || !tmp_mask_offset || !mask_offset) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (valid_word_num < 0 || hidden < 1) return EN_ERR_SHAPE;
  if (valid_word_num == 0) return EN_OK;
  if (!aligned_to(src, elem_size) || !aligned_to(tgt, elem_size)) return EN_ERR_ALIGN;
  Ptrs3 p = {{src, nullptr, nullptr}, {tgt, nullptr, nullptr}};
  return launch_row_gather<FtRemoveMap, 1>(hidden * elem_size, valid_word_num,
                                           (int64_t)valid_word_num * hidden * elem_size, p, [&](int R, dim3 &grid) {
    grid = dim3((unsigned)ceil_div(valid_word_num, R), 1, 1);
    return FtRemoveMap{tmp_mask_offset, mask_offset, valid_word_num, R};
  }, (hipStream_t)stream);
}

int en_ft_rebuild_padding(const void *src, void *tgt, const int32_t *mask_offset, int valid_word_num,
                          int64_t hidden, int batch, int max_seq_len, int elem_size, en_stream_t stream) {
  if (!src || !tgt || !mask_offset) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (valid_word_num < 0 || hidden < 1 || batch < 1 || max_seq_len < 1) return EN_ERR_SHAPE;
  const int64_t rows_out = (int64_t)batch * max_seq_len;
  if (rows_out > INT32_MAX || valid_word_num > rows_out) return EN_ERR_SHAPE;
  if (!aligned_to(src, elem_size) || !aligned_to(tgt, elem_size)) return EN_ERR_ALIGN;
  Ptrs3 p = {{src, nullptr, nullptr}, {tgt, nullptr, nullptr}};
  return launch_row_gather<FtRebuildMap, 1>(hidden * elem_size, rows_out, rows_out * hidden * elem_size, p, [&](int R, dim3 &grid) {
    grid = dim3((unsigned)ceil_div(rows_out, R), 1, 1);
    return FtRebuildMap{mask_offset, valid_word_num, (int)rows_out, R};
  }, (hipStream_t)stream);
}

int en_ft_transpose_rebuild(const void *Q, const void *K, const void *V, void *q_buf, void *k_buf, void *v_buf,
                            int batch, int seq_len, int head_num, int size_per_head, int valid_word_num,
                            const int32_t *mask_offset, int elem_size, en_stream_t stream) {
  if (!Q || !q_buf || !mask_offset) return EN_ERR_NULL;
  if ((K == nullptr) != (k_buf == nullptr) || (V == nullptr) != (v_buf == nullptr)) return EN_ERR_NULL;
  if (V && !K) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (batch < 1 || seq_len < 1 || head_num < 1 || size_per_head < 1 || valid_word_num < 0) return EN_ERR_SHAPE;
  if (valid_word_num == 0) return EN_OK;
  Ptrs3 p = {{Q, K, V}, {q_buf, k_buf, v_buf}};
  const int nt = V ? 3 : (K ? 2 : 1);
  for (int t = 0; t < nt; ++t)
    if (!aligned_to(p.src[t], elem_size) || !aligned_to(p.dst[t], elem_size)) return EN_ERR_ALIGN;
  auto mk = [&](int R, dim3 &grid) {
    grid = dim3((unsigned)(ceil_div(valid_word_num, R) * head_num), 1, 1);
    return FtTransposeRebuildMap{mask_offset, valid_word_num, head_num, seq_len, R};
  };
  const int64_t row_bytes = (int64_t)size_per_head * elem_size;
  const int64_t out_bytes = (int64_t)valid_word_num * head_num * row_bytes * nt;
  if (nt == 3) return launch_row_gather<FtTransposeRebuildMap, 3>(row_bytes, valid_word_num, out_bytes, p, mk, (hipStream_t)stream);
  if (nt == 2) return launch_row_gather<FtTransposeRebuildMap, 2>(row_bytes, valid_word_num, out_bytes, p, mk, (hipStream_t)stream);
  return launch_row_gather<FtTransposeRebuildMap, 1>(row_bytes, valid_word_num, out_bytes, p, mk, (hipStream_t)stream);
}

int en_ft_transpose_remove(const void *src, void *dst, int valid_word_num, int batch, int seq_len, int head_num,
                           int size_per_head, const int32_t *mask_offset, int elem_size, en_stream_t stream) {
  if (!src || !dst || !mask_offset) return EN_ERR_NULL;
  if (check_elem(elem_size)) return EN_ERR_DTYPE;
  if (batch < 1 || seq_len < 1 || head_num < 1 || size_per_head < 1 || valid_word_num < 0) return EN_ERR_SHAPE;
  if (valid_word_num == 0) return EN_OK;
  if (!aligned_to(src, elem_size) || !aligned_to(dst, elem_size)) return EN_ERR_ALIGN;
  Ptrs3 p = {{src, nullptr, nullptr}, {dst, nullptr, nullptr}};
  return launch_row_gather<FtTransposeRemoveMap, 1>((int64_t)size_per_head * elem_size, valid_word_num,
                                                    (int64_t)valid_word_num * head_num * size_per_head * elem_size, p,
                                                    [&](int R, dim3 &grid) {
    grid = dim3((unsigned)(ceil_div(valid_word_num, R) * head_num), 1, 1);
    return FtTransposeRemoveMap{mask_offset, valid_word_num, head_num, seq_len, R};
  }, (hipStream_t)stream);
}

}  // extern "C"
