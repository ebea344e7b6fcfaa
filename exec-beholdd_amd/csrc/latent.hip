// Attention over a cached latent: every position keeps one normed vector c [rank] and one rotated key part
// [rot_dim] that all heads share.  A head's score is q_c . (U_k c) + q_r . k_r = (U_k^T q_c) . c + q_r . k_r, and its
// output U_v (sum_j p_j c_j): with the queries carried into the latent's space the attention is the paged
// attention kernels' own case of ONE key/value head of size rank + rot_dim shared by all query heads, whose
// key is [c | k_r] and whose value is [c | 0].  This file holds what stands around that call:
//   latent_write    norm of c, rotation of k_r, and both into the cache pages of (sequence, position)
//   heads_linear    a small matrix per head: y[row, h, :] = W_h x[row, h, :] (queries into the latent's space,
//                   attended latents into the heads' values)
//   rotate_heads    rotation of a slice of every head of a row into a slice of another matrix's heads
// The angle of pair i at position p is the float32 product p * freq[i]; cosine and sine are taken of that float32.
#include "common.h"

// ---- the cached row: c = rms(x[:rank]) * w, k_r = rotate(x[rank:]) --------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_write_kernel(
    const T* __restrict__ down, int row_stride, int offset, const float* __restrict__ w, float eps,
    const float* __restrict__ freq, int turned, const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
    T* __restrict__ k_pages, T* __restrict__ v_pages, const int32_t* __restrict__ page_table, int table_stride, int rank,
    int rot_dim, int kv_order, int write, T* __restrict__ query, long q_row, int q_head, int q_first, int src_head, int src_first,
    int H, const T* __restrict__ q_src, long q_src_row, int neighbours, float magnitude) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const T* x = down + (size_t)row * row_stride + offset;
  const int pos = positions[row], hd = rank + rot_dim;
  const int half = turned / 2;
  if (query != nullptr) {      // the heads' rotated query parts, from the same projected row or from a matrix of their own
    for (int e = threadIdx.x; e < H * rot_dim; e += blockDim.x) {
      const int head = e / rot_dim, i = e % rot_dim;
      const T* from = q_src + (size_t)row * q_src_row + (size_t)head * src_head + src_first;
      float y;
      if (i < turned) {
        // the pair's first and second dimension: i and i + half, or the neighbours 2 pair and 2 pair + 1
        const int pair = neighbours ? i / 2 : (i < half ? i : i - half);
        const bool is_first = neighbours ? (i % 2 == 0) : (i < half);
        const float angle = (float)pos * freq[pair];
        const float c = cosf(angle) * magnitude, s = sinf(angle) * magnitude;
        const float u = to_f32(from[neighbours ? 2 * pair : pair]), v = to_f32(from[neighbours ? 2 * pair + 1 : pair + half]);
        y = is_first ? u * c - v * s : v * c + u * s;
      } else {
        y = to_f32(from[i]);
      }
      query[(size_t)row * q_row + (size_t)head * q_head + q_first + i] = from_f32<T>(y);
    }
  }
  if (!write) return;
  const int page = page_table[(size_t)row_seq[row] * table_stride + pos / BH_PAGE], token = pos % BH_PAGE;
  T* keys = k_pages + (size_t)page * BH_PAGE * hd;
  T* values = v_pages + (size_t)page * BH_PAGE * hd;
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = to_f32(x[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const T c = from_f32<T>(to_f32(x[i]) * inv * (w ? w[i] : 1.f));
    keys[bh_key_index(kv_order, token, i, hd)] = c;
    values[bh_value_index(kv_order, token, i, hd)] = c;
  }
  for (int i = threadIdx.x; i < rot_dim; i += blockDim.x) {
    float y;
    if (i < turned) {
      const int pair = neighbours ? i / 2 : (i < half ? i : i - half);
      const bool is_first = neighbours ? (i % 2 == 0) : (i < half);
      const float angle = (float)pos * freq[pair];
      const float c = cosf(angle) * magnitude, s = sinf(angle) * magnitude;
      const float u = to_f32(x[rank + (neighbours ? 2 * pair : pair)]), v = to_f32(x[rank + (neighbours ? 2 * pair + 1 : pair + half)]);
      y = is_first ? u * c - v * s : v * c + u * s;
    } else {
      y = to_f32(x[rank + i]);
    }
    keys[bh_key_index(kv_order, token, rank + i, hd)] = from_f32<T>(y);
    values[bh_value_index(kv_order, token, rank + i, hd)] = from_f32<T>(0.f);
  }
}

// down [n_rows][row_stride]: a row holds, from `offset`, rank latent elements and rot_dim key elements.
// Pages as the attention kernels take them for one kv head of size rank + rot_dim (written when `write` is set).
// With `query`, the same launch rotates the rot_dim elements at src_first of each of the H heads (src_head apart) of the
// same row into query[row][head * q_head + q_first ..]: the heads' rotated query parts, beside the key's.  With `q_src`
// (rows of q_src_row elements) the heads' parts are read from that matrix instead of `down`.  `neighbours`: a pair is
// dimensions 2i and 2i + 1 instead of i and i + turned/2; `magnitude` multiplies every cosine and sine.
extern "C" int bh_latent_write(const void* down, int dtype, int row_stride, int offset, const float* w, float eps,
                               const float* freq, int turned, const int32_t* positions, const int32_t* row_seq,
                               void* k_pages, void* v_pages, const int32_t* page_table, int table_stride, int n_rows,
                               int rank, int rot_dim, int kv_order, int write, void* query, long q_row, int q_head, int q_first,
                               int src_head, int src_first, int H, const void* q_src, long q_src_row, int neighbours,
                               float magnitude, hipStream_t stream) {
  BH_REQUIRE(write || query != nullptr, "latent_write: nothing to do");
  if (q_src == nullptr) {
    q_src = down;
    q_src_row = row_stride;
  }
  BH_REQUIRE(query == nullptr || (H > 0 && q_first >= 0 && src_first >= 0 && q_first + rot_dim <= q_head && src_first + rot_dim <= src_head &&
                                  (long)H * q_head <= q_row && (long)H * src_head <= q_src_row),
             "latent_write: the heads' rotated slices do not lie inside their rows");
  BH_REQUIRE(n_rows > 0 && rank > 0 && rot_dim >= 0, "latent_write: sizes must be positive (the rotated part may be absent)");
  BH_REQUIRE(turned >= 0 && turned % 2 == 0 && turned <= rot_dim, "latent_write: %d turned dimensions of %d", turned, rot_dim);
  BH_REQUIRE(turned == 0 || freq != nullptr, "latent_write: a rotation needs its frequencies");
  BH_REQUIRE(offset >= 0 && offset + rank + rot_dim <= row_stride, "latent_write: the latent does not lie inside a row of %d", row_stride);
  BH_REQUIRE(kv_order == BH_KV_ROWS || (kv_order == BH_KV_PIECES && (rank + rot_dim) % 32 == 0),
             "latent_write: cache order %d does not exist for head size %d", kv_order, rank + rot_dim);
#define BH_LW(T)                                                                                                      \
  latent_write_kernel<T><<<dim3(n_rows), dim3(256), 0, stream>>>((const T*)down, row_stride, offset, w, eps, freq, turned, \
                                                                 positions, row_seq, (T*)k_pages, (T*)v_pages, page_table, \
                                                                 table_stride, rank, rot_dim, kv_order, write, (T*)query, q_row, q_head, \
                                                                 q_first, src_head, src_first, H, (const T*)q_src, q_src_row, \
                                                                 neighbours, magnitude)
  if (dtype == BH_F32) BH_LW(float);
  else if (dtype == BH_BF16) BH_LW(bf16_t);
  else return bh_fail("latent_write: unknown dtype %d", dtype);
#undef BH_LW
  return bh_check_launch("latent_write");
}

// ---- a small matrix per head ---------------------------------------------------------------------------------
// y[row][h][o] = sum_i w[h][i][o] * x[row][h][i] for o < n_out, i < n_in; x and y are slices of the heads of wider rows
// (row stride, head stride and first element given for each); w [H][n_in][n_out], the output index running fastest,
// so that the lanes of a wave read neighbouring weights.  Float32 sums; a workgroup takes HL_ROWS rows of one head
// and up to 256 outputs, the rows' inputs going through LDS once.  y's rows lie one after the other, or, for the
// product that reads them next, in blocks of rows (bh_rows_index; y_row is then the matrix's width).
#define HL_ROWS 16

template <typename T>
__global__ __launch_bounds__(256) void heads_linear_kernel(const T* __restrict__ x, long x_row, int x_head, int x_first,
                                                           const T* __restrict__ w, T* __restrict__ y, long y_row, int y_head,
                                                           int y_first, int n_rows, int n_in, int n_out, int y_block_rows) {
  extern __shared__ __align__(16) float xs[];      // [n_in][HL_ROWS]: the rows' values of one input side by side
  const int row0 = blockIdx.x * HL_ROWS, head = blockIdx.y, o = blockIdx.z * 256 + threadIdx.x;
  const int rows = n_rows - row0 < HL_ROWS ? n_rows - row0 : HL_ROWS;
  for (int e = threadIdx.x; e < HL_ROWS * n_in; e += 256) {
    const int r = e / n_in, i = e % n_in;      // neighbouring threads read neighbouring inputs of a row
    xs[i * HL_ROWS + r] = r < rows ? to_f32(x[(size_t)(row0 + r) * x_row + (size_t)head * x_head + x_first + i]) : 0.f;
  }
  __syncthreads();
  if (o >= n_out) return;
  const T* wh = w + (size_t)head * n_in * n_out + o;
  float acc[HL_ROWS] = {};
  for (int i = 0; i < n_in; ++i) {
    const float wv = to_f32(wh[(size_t)i * n_out]);
#pragma unroll
    for (int r = 0; r < HL_ROWS; r += 4) {      // four rows a read of LDS, the same address for every lane
      const float4 x4 = *reinterpret_cast<const float4*>(xs + i * HL_ROWS + r);
      acc[r] = fmaf(x4.x, wv, acc[r]);
      acc[r + 1] = fmaf(x4.y, wv, acc[r + 1]);
      acc[r + 2] = fmaf(x4.z, wv, acc[r + 2]);
      acc[r + 3] = fmaf(x4.w, wv, acc[r + 3]);
    }
  }
#pragma unroll
  for (int r = 0; r < HL_ROWS; ++r)
    if (r < rows) y[bh_rows_index(y_block_rows, row0 + r, head * y_head + y_first + o, (int)y_row)] = from_f32<T>(acc[r]);
}

// The same for a step of at most HL_ROWS rows (decoding): a workgroup takes 64 outputs of one head and its four waves
// a quarter of the inputs each, so that a head's weights are streamed by several workgroups and no thread walks all the
// inputs alone; the quarters' sums are added through LDS in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void heads_linear_few_kernel(const T* __restrict__ x, long x_row, int x_head, int x_first,
                                                               const T* __restrict__ w, T* __restrict__ y, long y_row, int y_head,
                                                               int y_first, int n_rows, int n_in, int n_out, int y_block_rows) {
  extern __shared__ __align__(16) float xs[];      // [n_in][HL_ROWS]
  __shared__ float parts[3][64][HL_ROWS + 1];
  const int head = blockIdx.y, lane = threadIdx.x % 64, quarter = threadIdx.x / 64, o = blockIdx.z * 64 + lane;
  for (int e = threadIdx.x; e < HL_ROWS * n_in; e += 256) {
    const int r = e / n_in, i = e % n_in;
    xs[i * HL_ROWS + r] = r < n_rows ? to_f32(x[(size_t)r * x_row + (size_t)head * x_head + x_first + i]) : 0.f;
  }
  __syncthreads();
  const int each = (n_in + 3) / 4, from = quarter * each, to = from + each < n_in ? from + each : n_in;
  const T* wh = w + (size_t)head * n_in * n_out + (o < n_out ? o : n_out - 1);
  float acc[HL_ROWS] = {};
  for (int i = from; i < to; ++i) {
    const float wv = to_f32(wh[(size_t)i * n_out]);
#pragma unroll
    for (int r = 0; r < HL_ROWS; r += 4) {
      const float4 x4 = *reinterpret_cast<const float4*>(xs + i * HL_ROWS + r);
      acc[r] = fmaf(x4.x, wv, acc[r]);
      acc[r + 1] = fmaf(x4.y, wv, acc[r + 1]);
      acc[r + 2] = fmaf(x4.z, wv, acc[r + 2]);
      acc[r + 3] = fmaf(x4.w, wv, acc[r + 3]);
    }
  }
  if (quarter > 0) {
#pragma unroll
    for (int r = 0; r < HL_ROWS; ++r) parts[quarter - 1][lane][r] = acc[r];
  }
  __syncthreads();
  if (quarter > 0 || o >= n_out) return;
#pragma unroll
  for (int r = 0; r < HL_ROWS; ++r) {
    if (r >= n_rows) continue;
    const float total = ((acc[r] + parts[0][lane][r]) + parts[1][lane][r]) + parts[2][lane][r];
    y[bh_rows_index(y_block_rows, r, head * y_head + y_first + o, (int)y_row)] = from_f32<T>(total);
  }
}

extern "C" int bh_heads_linear(const void* x, long x_row, int x_head, int x_first, const void* w, void* y, long y_row,
                               int y_head, int y_first, int dtype, int n_rows, int H, int n_in, int n_out, int y_block_rows,
                               hipStream_t stream) {
  BH_REQUIRE(y_block_rows == 0 || ((y_block_rows == 8 || y_block_rows == 16) && dtype == BH_BF16 && y_row % 32 == 0 && y_row < (1L << 31)),
             "heads_linear: an output in blocks of %d rows needs bfloat16 and rows of a multiple of 32 elements (got %ld)",
             y_block_rows, y_row);
  BH_REQUIRE(n_rows > 0 && H > 0 && n_in > 0 && n_out > 0, "heads_linear: sizes must be positive");
  BH_REQUIRE(H <= 65535 && (n_out + 255) / 256 <= 65535, "heads_linear: too many heads or outputs");
  BH_REQUIRE(x_first >= 0 && y_first >= 0 && x_first + n_in <= x_head && y_first + n_out <= y_head &&
                 (long)H * x_head <= x_row && (long)H * y_head <= y_row,
             "heads_linear: the heads' slices do not lie inside their rows");
  const size_t smem = (size_t)HL_ROWS * n_in * sizeof(float);
  BH_REQUIRE(smem <= 64 * 1024, "heads_linear: %d inputs a head are above the limit of %d", n_in, 64 * 1024 / 4 / HL_ROWS);
  if (n_rows <= HL_ROWS && smem + sizeof(float) * 3 * 64 * (HL_ROWS + 1) <= 64 * 1024) {      // (its partial sums need LDS too)
    dim3 few(1, H, (n_out + 63) / 64);
#define BH_HL_FEW(T)                                                                                                      \
  heads_linear_few_kernel<T><<<few, dim3(256), smem, stream>>>((const T*)x, x_row, x_head, x_first, (const T*)w, (T*)y, y_row, \
                                                               y_head, y_first, n_rows, n_in, n_out, y_block_rows)
    if (dtype == BH_F32) BH_HL_FEW(float);
    else if (dtype == BH_BF16) BH_HL_FEW(bf16_t);
    else return bh_fail("heads_linear: unknown dtype %d", dtype);
#undef BH_HL_FEW
    return bh_check_launch("heads_linear_few");
  }
  dim3 grid((n_rows + HL_ROWS - 1) / HL_ROWS, H, (n_out + 255) / 256), block(256);
#define BH_HL(T)                                                                                                         \
  heads_linear_kernel<T><<<grid, block, smem, stream>>>((const T*)x, x_row, x_head, x_first, (const T*)w, (T*)y, y_row, y_head, \
                                                        y_first, n_rows, n_in, n_out, y_block_rows)
  if (dtype == BH_F32) BH_HL(float);
  else if (dtype == BH_BF16) BH_HL(bf16_t);
  else return bh_fail("heads_linear: unknown dtype %d", dtype);
#undef BH_HL
  return bh_check_launch("heads_linear");
}

// ---- rotation of a slice of every head ------------------------------------------------------------------------
// y[row][h][y_first + i] = rotated x[row][h][x_first + i] for i < width: the first `turned` of them in pairs
// (i, i + turned/2) by the angle position[row] * freq[i], the rest as they are.
template <typename T>
__global__ void rotate_heads_kernel(const T* __restrict__ x, long x_row, int x_head, int x_first, T* __restrict__ y,
                                    long y_row, int y_head, int y_first, const float* __restrict__ freq, int turned,
                                    const int32_t* __restrict__ positions, int H, int width) {
  const int row = blockIdx.x;
  const float pos = (float)positions[row];
  const int half = turned / 2;
  for (int e = threadIdx.x; e < H * width; e += blockDim.x) {
    const int head = e / width, i = e % width;
    const T* from = x + (size_t)row * x_row + (size_t)head * x_head + x_first;
    float v;
    if (i < turned) {
      const int pair = i < half ? i : i - half;
      const float angle = pos * freq[pair];
      const float c = cosf(angle), s = sinf(angle);
      const float a = to_f32(from[pair]), b = to_f32(from[pair + half]);
      v = i < half ? a * c - b * s : b * c + a * s;
    } else {
      v = to_f32(from[i]);
    }
    y[(size_t)row * y_row + (size_t)head * y_head + y_first + i] = from_f32<T>(v);
  }
}

extern "C" int bh_rotate_heads(const void* x, long x_row, int x_head, int x_first, void* y, long y_row, int y_head,
                               int y_first, int dtype, const float* freq, int turned, const int32_t* positions, int n_rows,
                               int H, int width, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && width > 0, "rotate_heads: sizes must be positive");
  BH_REQUIRE(turned >= 0 && turned % 2 == 0 && turned <= width, "rotate_heads: %d turned dimensions of %d", turned, width);
  BH_REQUIRE(turned == 0 || freq != nullptr, "rotate_heads: a rotation needs its frequencies");
  BH_REQUIRE(x_first >= 0 && y_first >= 0 && x_first + width <= x_head && y_first + width <= y_head &&
                 (long)H * x_head <= x_row && (long)H * y_head <= y_row,
             "rotate_heads: the heads' slices do not lie inside their rows");
#define BH_RH(T)                                                                                                          \
  rotate_heads_kernel<T><<<dim3(n_rows), dim3(256), 0, stream>>>((const T*)x, x_row, x_head, x_first, (T*)y, y_row, y_head, \
                                                                 y_first, freq, turned, positions, H, width)
  if (dtype == BH_F32) BH_RH(float);
  else if (dtype == BH_BF16) BH_RH(bf16_t);
  else return bh_fail("rotate_heads: unknown dtype %d", dtype);
#undef BH_RH
  return bh_check_launch("rotate_heads");
}
