// Small row-wise operations on the float32 residual and on logits:
//   layernorm        (x - mean) / sqrt(var + eps) * w + b per row, optional row gather, rows or blocks of rows out
//   sum_layernorm    h <- layernorm(alpha h + y) per row in place, and the same rounded for the product that reads it next
//   gelu_tanh        out = gelu(x), tanh form, elementwise into rows or blocks of rows
//   cast_concat      [a | b] per row from float32 into the activation type (b optional): the input of a product
//   softcap          x <- cap * tanh(x / cap) in place
//   rms_scale_add    h <- h + y / sqrt(mean(y^2) + eps) * w per row
//   gelu_gate_table  out[r][i] = gelu_tanh(gate[r][i]) * table[token of r][first + i]
// All statistics are float32.
#include "common.h"

// One workgroup a row.  The mean first, then the mean of the squared deviations (not E[x^2] - mean^2, which
// loses digits where the mean is large beside the spread).
template <typename TO>
__global__ __launch_bounds__(256) void layernorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                                        const float* __restrict__ w, const float* __restrict__ b,
                                                        TO* __restrict__ out, int width, float eps, int out_block_rows) {
  __shared__ float scratch[8];
  const int r = blockIdx.x;
  const float* src = x + (size_t)(rows ? rows[r] : r) * width;
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) sum += src[i];
  const float mean = block_sum(sum, scratch) / (float)width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float d = src[i] - mean;
    ss += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float y = (src[i] - mean) * inv * w[i] + (b ? b[i] : 0.f);
    out[bh_rows_index(out_block_rows, r, i, width)] = from_f32<TO>(y);
  }
}

extern "C" int bh_layernorm(const float* x, const int32_t* rows, const float* w, const float* b, void* out, int out_dtype,
                            int n_rows, int width, float eps, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "layernorm: sizes must be positive");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && width % 32 == 0 && out_dtype == BH_BF16),
             "layernorm: rows in blocks of %d of width %d are not written", out_block_rows, width);
  if (out_dtype == BH_F32)
    layernorm_kernel<float><<<n_rows, 256, 0, stream>>>(x, rows, w, b, (float*)out, width, eps, out_block_rows);
  else if (out_dtype == BH_BF16)
    layernorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(x, rows, w, b, (bf16_t*)out, width, eps, out_block_rows);
  else
    return bh_fail("layernorm: unknown dtype %d", out_dtype);
  return bh_check_launch("layernorm");
}

// h <- ((s - mean) / sqrt(var + eps)) * w + b with s = alpha * h + y: the norm stands behind the sum.  One workgroup a
// row; a thread meets the same elements in all three passes, so the sum can stand in h's own place between them.  With
// `rounded` the result also goes out in the activation type (rows or blocks of rows), for the product that reads it next.
template <typename TO>
__global__ __launch_bounds__(256) void sum_layernorm_kernel(float* __restrict__ h, const float* __restrict__ y, float alpha,
                                                            const float* __restrict__ w, const float* __restrict__ b,
                                                            TO* __restrict__ rounded, int width, float eps, int out_block_rows) {
  __shared__ float scratch[8];
  const int r = blockIdx.x;
  float* row = h + (size_t)r * width;
  const float* add = y + (size_t)r * width;
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float s = fmaf(alpha, row[i], add[i]);
    row[i] = s;
    sum += s;
  }
  const float mean = block_sum(sum, scratch) / (float)width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float d = row[i] - mean;
    ss += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = (row[i] - mean) * inv * w[i] + (b ? b[i] : 0.f);
    row[i] = v;
    if (rounded) rounded[bh_rows_index(out_block_rows, r, i, width)] = from_f32<TO>(v);
  }
}

// The same for rows of up to THREADS * PER elements: a thread keeps its PER elements of the sum in registers, so the row is read
// once and written once and nothing waits for its own stores (a step of few rows is three trips to memory shorter).
template <typename TO, int PER, int THREADS>
__global__ __launch_bounds__(THREADS) void sum_layernorm_held_kernel(float* __restrict__ h, const float* __restrict__ y, float alpha,
                                                                 const float* __restrict__ w, const float* __restrict__ b,
                                                                 TO* __restrict__ rounded, int width, float eps, int out_block_rows) {
  __shared__ float scratch[THREADS / BH_WAVE];
  const int r = blockIdx.x;
  float* row = h + (size_t)r * width;
  const float* add = y + (size_t)r * width;
  float held[PER];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * THREADS;
    held[k] = i < width ? fmaf(alpha, row[i], add[i]) : 0.f;
    sum += held[k];
  }
  const float mean = block_sum(sum, scratch) / (float)width;
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const float d = threadIdx.x + k * THREADS < width ? held[k] - mean : 0.f;
    ss += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * THREADS;
    if (i < width) {
      const float v = (held[k] - mean) * inv * w[i] + (b ? b[i] : 0.f);
      row[i] = v;
      if (rounded) rounded[bh_rows_index(out_block_rows, r, i, width)] = from_f32<TO>(v);
    }
  }
}

template <typename TO>
static void sum_layernorm_launch(float* h, const float* y, float alpha, const float* w, const float* b, TO* rounded, int n_rows,
                                 int width, float eps, int out_block_rows, hipStream_t stream) {
#define BH_SL(PER, THREADS) \
  sum_layernorm_held_kernel<TO, PER, THREADS><<<n_rows, THREADS, 0, stream>>>(h, y, alpha, w, b, rounded, width, eps, out_block_rows)
  if (n_rows <= 64 && width > 1024 && width <= 1024 * 8) {      // few rows: a row on sixteen waves, a few elements a thread
    if (width <= 1024 * 4) BH_SL(4, 1024);
    else BH_SL(8, 1024);
  } else if (width <= 256 * 4) {
    BH_SL(4, 256);
  } else if (width <= 256 * 16) {
    BH_SL(16, 256);
  } else if (width <= 256 * 32) {
    BH_SL(32, 256);
  } else {
    sum_layernorm_kernel<TO><<<n_rows, 256, 0, stream>>>(h, y, alpha, w, b, rounded, width, eps, out_block_rows);
  }
#undef BH_SL
}

extern "C" int bh_sum_layernorm(float* h, const float* y, float alpha, const float* w, const float* b, void* rounded,
                                int out_dtype, int n_rows, int width, float eps, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "sum_layernorm: sizes must be positive");
  BH_REQUIRE(h != y, "sum_layernorm: the sublayer's result stands apart from the residual");
  BH_REQUIRE(out_block_rows == 0 || (rounded && (out_block_rows == 8 || out_block_rows == 16) && width % 32 == 0 && out_dtype == BH_BF16),
             "sum_layernorm: rows in blocks of %d of width %d are not written", out_block_rows, width);
  if (rounded == nullptr || out_dtype == BH_F32)
    sum_layernorm_launch<float>(h, y, alpha, w, b, (float*)rounded, n_rows, width, eps, out_block_rows, stream);
  else if (out_dtype == BH_BF16)
    sum_layernorm_launch<bf16_t>(h, y, alpha, w, b, (bf16_t*)rounded, n_rows, width, eps, out_block_rows, stream);
  else
    return bh_fail("sum_layernorm: unknown dtype %d", out_dtype);
  return bh_check_launch("sum_layernorm");
}

template <typename TO>
__global__ __launch_bounds__(256) void cast_concat_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          TO* __restrict__ out, int n_rows, int width, int out_block_rows) {
  const int total = b ? 2 * width : width;
  const size_t n = (size_t)n_rows * total;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const int r = (int)(e / total), i = (int)(e % total);
    const float v = i < width ? a[(size_t)r * width + i] : b[(size_t)r * width + i - width];
    out[bh_rows_index(out_block_rows, r, i, total)] = from_f32<TO>(v);
  }
}

extern "C" int bh_cast_concat(const float* a, const float* b, void* out, int out_dtype, int n_rows, int width,
                              int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "cast_concat: sizes must be positive");
  const int total = b ? 2 * width : width;
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && total % 32 == 0 && out_dtype == BH_BF16),
             "cast_concat: rows in blocks of %d of width %d are not written", out_block_rows, total);
  const size_t n = (size_t)n_rows * total;
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  if (out_dtype == BH_F32)
    cast_concat_kernel<float><<<blocks, 256, 0, stream>>>(a, b, (float*)out, n_rows, width, out_block_rows);
  else if (out_dtype == BH_BF16)
    cast_concat_kernel<bf16_t><<<blocks, 256, 0, stream>>>(a, b, (bf16_t*)out, n_rows, width, out_block_rows);
  else
    return bh_fail("cast_concat: unknown dtype %d", out_dtype);
  return bh_check_launch("cast_concat");
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, long n, float cap) {
  const float inv = 1.0f / cap;
  for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long)gridDim.x * blockDim.x)
    x[e] = cap * tanhf(x[e] * inv);
}

extern "C" int bh_softcap(float* x, long n, float cap, hipStream_t stream) {
  BH_REQUIRE(n > 0 && cap > 0.f, "softcap: a positive count and a positive cap");
  const long blocks = (n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096;
  softcap_kernel<<<(int)blocks, 256, 0, stream>>>(x, n, cap);
  return bh_check_launch("softcap");
}

__global__ __launch_bounds__(256) void rms_scale_add_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                            const float* __restrict__ w, int width, float eps) {
  __shared__ float scratch[8];
  const float* src = y + (size_t)blockIdx.x * width;
  float* dst = h + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) ss += src[i] * src[i];
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] += src[i] * inv * w[i];
}

extern "C" int bh_rms_scale_add(float* h, const float* y, const float* w, int n_rows, int width, float eps, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "rms_scale_add: sizes must be positive");
  rms_scale_add_kernel<<<n_rows, 256, 0, stream>>>(h, y, w, width, eps);
  return bh_check_launch("rms_scale_add");
}

__device__ inline float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_kernel(const T* __restrict__ x, T* __restrict__ out, int width, size_t total, int block_rows) {
  const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (at >= total) return;
  const size_t to = block_rows ? (size_t)bh_rows_index(block_rows, (int)(at / width), (int)(at % width), width) : at;
  out[to] = from_f32<T>(gelu_tanh(to_f32(x[at])));
}

extern "C" int bh_gelu_tanh(const void* x, void* out, int dtype, int n_rows, int width, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "gelu_tanh: nothing to do");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && dtype == BH_BF16 && width % 32 == 0 && x != out),
             "gelu_tanh: rows in blocks of %d need bfloat16, a width that is a multiple of 32 (got %d) and an output of their own",
             out_block_rows, width);
  const size_t total = (size_t)n_rows * width;
  const size_t blocks = (total + 255) / 256;
  BH_REQUIRE(blocks <= 2147483647u, "gelu_tanh: too many elements");
  if (dtype == BH_F32)
    gelu_tanh_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>((const float*)x, (float*)out, width, total, out_block_rows);
  else if (dtype == BH_BF16)
    gelu_tanh_kernel<bf16_t><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>((const bf16_t*)x, (bf16_t*)out, width, total, out_block_rows);
  else return bh_fail("gelu_tanh: unknown dtype %d", dtype);
  return bh_check_launch("gelu_tanh");
}

// A row's token is tokens[row], or fed[token_src[row]] where token_src is given and not negative (a token chosen on the
// device that the host has not read yet).
template <typename T>
__global__ __launch_bounds__(256) void gelu_gate_table_kernel(const T* __restrict__ gate, const int32_t* __restrict__ tokens,
                                                              const int32_t* __restrict__ token_src, const int32_t* __restrict__ fed,
                                                              const T* __restrict__ table, int table_width, int first, int vocab,
                                                              T* __restrict__ out, int n_rows, int dim, int out_block_rows) {
  const size_t n = (size_t)n_rows * dim;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const int r = (int)(e / dim), i = (int)(e % dim);
    int token = tokens[r];
    if (token_src != nullptr && token_src[r] >= 0) token = fed[token_src[r]];
    token = token < 0 ? 0 : (token >= vocab ? vocab - 1 : token);
    const float g = gelu_tanh(to_f32(gate[(size_t)r * dim + i])) * to_f32(table[(size_t)token * table_width + first + i]);
    out[bh_rows_index(out_block_rows, r, i, dim)] = from_f32<T>(g);
  }
}

extern "C" int bh_gelu_gate_table(const void* gate, int dtype, const int32_t* tokens, const int32_t* token_src,
                                  const int32_t* fed, const void* table, int table_width, int first, int vocab, void* out,
                                  int n_rows, int dim, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && dim > 0 && vocab > 0, "gelu_gate_table: sizes must be positive");
  BH_REQUIRE(first >= 0 && first + dim <= table_width, "gelu_gate_table: columns %d..%d lie outside a table row of %d", first,
             first + dim, table_width);
  BH_REQUIRE((token_src == nullptr) == (fed == nullptr), "gelu_gate_table: fed tokens come with their source indices");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && dim % 32 == 0 && dtype == BH_BF16),
             "gelu_gate_table: rows in blocks of %d of width %d are not written", out_block_rows, dim);
  const size_t n = (size_t)n_rows * dim;
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  if (dtype == BH_F32)
    gelu_gate_table_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate, tokens, token_src, fed, (const float*)table,
                                                            table_width, first, vocab, (float*)out, n_rows, dim, out_block_rows);
  else if (dtype == BH_BF16)
    gelu_gate_table_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gate, tokens, token_src, fed, (const bf16_t*)table,
                                                             table_width, first, vocab, (bf16_t*)out, n_rows, dim, out_block_rows);
  else
    return bh_fail("gelu_gate_table: unknown dtype %d", dtype);
  return bh_check_launch("gelu_gate_table");
}

// ---- a norm over a slice of wider rows, and a weighted sum of two matrices ---------------------------------------------
//   slice_rmsnorm   out[row][i] = x[row][first + i] / sqrt(mean_i(x^2) + eps) * w[i] for i < width (x in the activations'
//                   type, statistic and weight float32): a low-rank projection's share of a stacked product, normed
//   weighted_sum    out = a x + b y, float32 (out may be x or y)
template <typename T>
__global__ __launch_bounds__(256) void slice_rmsnorm_kernel(const T* __restrict__ x, int row_stride, int first, const float* __restrict__ w,
                                                            float eps, T* __restrict__ out, int width, int out_block_rows) {
  __shared__ float scratch[8];
  const int row = blockIdx.x;
  const T* src = x + (size_t)row * row_stride + first;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = to_f32(src[i]);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    out[bh_rows_index(out_block_rows, row, i, width)] = from_f32<T>(to_f32(src[i]) * inv * (w ? w[i] : 1.f));
}

extern "C" int bh_slice_rmsnorm(const void* x, int dtype, int row_stride, int first, const float* w, float eps, void* out, int n_rows,
                                int width, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0 && first >= 0 && first + width <= row_stride, "slice_rmsnorm: the slice lies outside a row of %d", row_stride);
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && width % 32 == 0 && dtype == BH_BF16),
             "slice_rmsnorm: rows in blocks of %d of width %d are not written", out_block_rows, width);
  if (dtype == BH_F32)
    slice_rmsnorm_kernel<float><<<n_rows, 256, 0, stream>>>((const float*)x, row_stride, first, w, eps, (float*)out, width, out_block_rows);
  else if (dtype == BH_BF16)
    slice_rmsnorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>((const bf16_t*)x, row_stride, first, w, eps, (bf16_t*)out, width, out_block_rows);
  else
    return bh_fail("slice_rmsnorm: unknown dtype %d", dtype);
  return bh_check_launch("slice_rmsnorm");
}

__global__ __launch_bounds__(256) void weighted_sum_kernel(float* out, const float* x, float a, const float* y, float b, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) out[e] = a * x[e] + b * y[e];
}

extern "C" int bh_weighted_sum(float* out, const float* x, float a, const float* y, float b, long n, hipStream_t stream) {
  BH_REQUIRE(n > 0, "weighted_sum: nothing to add");
  const int blocks = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  weighted_sum_kernel<<<blocks, 256, 0, stream>>>(out, x, a, y, b, (size_t)n);
  return bh_check_launch("weighted_sum");
}
