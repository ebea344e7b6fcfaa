// What stands around the paged attention kernels for an attention whose queries and keys are normed over the whole
// projection (all heads of a row together), turned in neighbouring pairs on the first dimensions of each head, and
// whose heads are gated before the output projection:
//   whole_norm_rope_write   per row of [q | k | v] (float32): q <- rms(q over all its channels) * wq, k likewise;
//                           dimensions 2i and 2i+1 (i < turned/2) of every head of q and k turned by
//                           position * freq[i]; q into a matrix of heads of `pad` dimensions, k and v into the cache
//                           pages of (sequence, position) as heads of `pad` (zeros beyond dim and vdim), so that keys of
//                           one size and values of another go through kernels that know one head size
//   conv_norm_rope_write    the same from the projected rows, the short convolution made on the way
//   gate_heads              out[row][h][i] = attended[row][h][i] * sigmoid(gate[row][h][i]) for i < vdim; the gate may be one
//                           number a head (gate[row][h]) or absent (the heads' first vdim elements are put side by side)
// Statistics, angles, cosines and sines are float32; the angle is the float32 product position * freq[i].
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void whole_norm_rope_write_kernel(
    const float* __restrict__ qkv, const float* __restrict__ wq, const float* __restrict__ wk, float eps,
    const float* __restrict__ freq, int turned, const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
    T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages, const int32_t* __restrict__ page_table,
    int table_stride, int H, int G, int dim, int vdim, int pad, int kv_order, int write) {
  extern __shared__ float turns[];      // the cosines, then the sines, of the row's turned pairs: one of each a pair and row
  __shared__ float scratch[8];
  const int row = blockIdx.x;
  const int q_width = H * dim, k_width = G * dim, v_width = G * vdim;
  const float* q = qkv + (size_t)row * (q_width + k_width + v_width);
  const float* k = q + q_width;
  const float* v = k + k_width;
  const int pos = positions[row];
  float* cosines = turns;
  float* sines = turns + turned / 2;
  for (int i = threadIdx.x; i < turned / 2; i += blockDim.x) {
    const float angle = (float)pos * freq[i];
    cosines[i] = cosf(angle);
    sines[i] = sinf(angle);
  }
  float ss_q = 0.f, ss_k = 0.f;
  for (int e = threadIdx.x; e < q_width + k_width; e += blockDim.x) {
    const float x = q[e];
    if (e < q_width) ss_q += x * x;
    else ss_k += x * x;
  }
  const float inv_q = 1.0f / sqrtf(block_sum(ss_q, scratch) / (float)q_width + eps);
  const float inv_k = 1.0f / sqrtf(block_sum(ss_k, scratch) / (float)k_width + eps);
  // a thread takes a pair of neighbouring dimensions: both of a turned pair come from the same two loads
  const int half = pad / 2;
  for (int e = threadIdx.x; e < H * half; e += blockDim.x) {
    const int head = e / half, i = 2 * (e % half);
    float y0 = 0.f, y1 = 0.f;
    if (i < dim) {
      const int at = head * dim + i;
      y0 = q[at] * inv_q * wq[at];
      if (i + 1 < dim) y1 = q[at + 1] * inv_q * wq[at + 1];
      if (i < turned) {
        const float c = cosines[i >> 1], s = sines[i >> 1], u = y0, w = y1;
        y0 = u * c - w * s;
        y1 = w * c + u * s;
      }
    }
    T* out = q_out + (size_t)row * H * pad + head * pad + i;
    out[0] = from_f32<T>(y0);
    out[1] = from_f32<T>(y1);
  }
  if (!write) return;
  const int page = page_table[(size_t)row_seq[row] * table_stride + pos / BH_PAGE], token = pos % BH_PAGE;
  for (int e = threadIdx.x; e < G * half; e += blockDim.x) {
    const int head = e / half, i = 2 * (e % half);
    float y0 = 0.f, y1 = 0.f;
    if (i < dim) {
      const int at = head * dim + i;
      y0 = k[at] * inv_k * wk[at];
      if (i + 1 < dim) y1 = k[at + 1] * inv_k * wk[at + 1];
      if (i < turned) {
        const float c = cosines[i >> 1], s = sines[i >> 1], u = y0, w = y1;
        y0 = u * c - w * s;
        y1 = w * c + u * s;
      }
    }
    T* keys = k_pages + ((size_t)page * G + head) * BH_PAGE * pad;
    T* values = v_pages + ((size_t)page * G + head) * BH_PAGE * pad;
    keys[bh_key_index(kv_order, token, i, pad)] = from_f32<T>(y0);
    keys[bh_key_index(kv_order, token, i + 1, pad)] = from_f32<T>(y1);
    values[bh_value_index(kv_order, token, i, pad)] = from_f32<T>(i < vdim ? v[head * vdim + i] : 0.f);
    values[bh_value_index(kv_order, token, i + 1, pad)] = from_f32<T>(i + 1 < vdim ? v[head * vdim + i + 1] : 0.f);
  }
}

extern "C" int bh_whole_norm_rope_write(const float* qkv, const float* wq, const float* wk, float eps, const float* freq,
                                        int turned, const int32_t* positions, const int32_t* row_seq, void* q_out, int dtype,
                                        void* k_pages, void* v_pages, const int32_t* page_table, int table_stride, int n_rows,
                                        int H, int G, int dim, int vdim, int pad, int kv_order, int write, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && G > 0 && dim > 0 && vdim > 0, "whole_norm_rope_write: sizes must be positive");
  BH_REQUIRE(pad >= dim && pad >= vdim, "whole_norm_rope_write: heads of %d do not hold keys of %d and values of %d", pad, dim, vdim);
  BH_REQUIRE(turned >= 0 && turned % 2 == 0 && turned <= dim && dim % 2 == 0 || turned == 0,
             "whole_norm_rope_write: %d turned dimensions of %d", turned, dim);
  BH_REQUIRE(turned == 0 || freq != nullptr, "whole_norm_rope_write: a rotation needs its frequencies");
  BH_REQUIRE(kv_order == BH_KV_ROWS || (kv_order == BH_KV_PIECES && pad % 32 == 0),
             "whole_norm_rope_write: cache order %d does not exist for head size %d", kv_order, pad);
  BH_REQUIRE(pad % 2 == 0, "whole_norm_rope_write: heads of an even size, got %d", pad);
  const size_t lds = (size_t)(turned > 0 ? turned : 1) * sizeof(float);
  if (dtype == BH_F32)
    whole_norm_rope_write_kernel<float><<<n_rows, 256, lds, stream>>>(qkv, wq, wk, eps, freq, turned, positions, row_seq, (float*)q_out,
                                                                  (float*)k_pages, (float*)v_pages, page_table, table_stride, H, G,
                                                                  dim, vdim, pad, kv_order, write);
  else if (dtype == BH_BF16)
    whole_norm_rope_write_kernel<bf16_t><<<n_rows, 256, lds, stream>>>(qkv, wq, wk, eps, freq, turned, positions, row_seq,
                                                                   (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, page_table,
                                                                   table_stride, H, G, dim, vdim, pad, kv_order, write);
  else
    return bh_fail("whole_norm_rope_write: unknown dtype %d", dtype);
  return bh_check_launch("whole_norm_rope_write");
}

// The same from the projected rows themselves: the short convolution over time (csrc/short_conv.hip has its definition and
// its state) is made on the way, a row's convolved channels stand in LDS as float32 and are never written to memory.
// proj [n_rows][row_stride]: a row holds, from `first`, q, k and v; w_conv [q + k + v channels][taps] (taps 0: no convolution).
template <typename T>
__global__ __launch_bounds__(1024) void conv_norm_rope_write_kernel(
    const T* __restrict__ proj, int row_stride, int first, const float* __restrict__ w_conv, int taps, const float* __restrict__ state,
    long slot_stride, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const float* __restrict__ freq, int turned, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_seq, T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int32_t* __restrict__ page_table, int table_stride, int H, int G, int dim, int vdim, int pad, int kv_order, int write) {
  extern __shared__ float conv[];      // [q | k | v] of this row, then the cosines and sines of the row's turned pairs
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int q_width = H * dim, k_width = G * dim, v_width = G * vdim, channels = q_width + k_width + v_width;
  float* cosines = conv + channels;
  float* sines = cosines + turned / 2;
  const int seq = row_seq[row], pos = positions[row];
  const int t = row - seq_start[seq];
  const float* old = state ? state + (size_t)seq_slot[seq] * slot_stride : nullptr;
  for (int i = threadIdx.x; i < turned / 2; i += blockDim.x) {
    const float angle = (float)pos * freq[i];
    cosines[i] = cosf(angle);
    sines[i] = sinf(angle);
  }
  float ss_q = 0.f, ss_k = 0.f;
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float acc;
    if (taps <= 1) {
      acc = to_f32(proj[(size_t)row * row_stride + first + c]) * (taps ? w_conv[c] : 1.f);
    } else {
      acc = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;
        const float u = back <= t ? to_f32(proj[(size_t)(row - back) * row_stride + first + c])
                                  : old[(size_t)(taps - 1 + t - back) * channels + c];
        acc = fmaf(w_conv[(size_t)c * taps + j], u, acc);
      }
    }
    conv[c] = acc;
    if (c < q_width) ss_q += acc * acc;
    else if (c < q_width + k_width) ss_k += acc * acc;
  }
  const float inv_q = 1.0f / sqrtf(block_sum(ss_q, scratch) / (float)q_width + eps);
  const float inv_k = 1.0f / sqrtf(block_sum(ss_k, scratch) / (float)k_width + eps);
  const float* q = conv;
  const float* k = conv + q_width;
  const float* v = k + k_width;
  for (int e = threadIdx.x; e < H * pad; e += blockDim.x) {
    const int head = e / pad, i = e % pad;
    float y = 0.f;
    if (i < dim) {
      const int at = head * dim + i;
      y = q[at] * inv_q * wq[at];
      if (i < turned) {
        const int mate = at ^ 1;
        const float other = q[mate] * inv_q * wq[mate];
        const float c = cosines[i >> 1], s = sines[i >> 1];
        y = (i & 1) ? y * c + other * s : y * c - other * s;
      }
    }
    q_out[(size_t)row * H * pad + e] = from_f32<T>(y);
  }
  if (!write) return;
  const int page = page_table[(size_t)seq * table_stride + pos / BH_PAGE], token = pos % BH_PAGE;
  for (int e = threadIdx.x; e < G * pad; e += blockDim.x) {
    const int head = e / pad, i = e % pad;
    float y = 0.f;
    if (i < dim) {
      const int at = head * dim + i;
      y = k[at] * inv_k * wk[at];
      if (i < turned) {
        const int mate = at ^ 1;
        const float other = k[mate] * inv_k * wk[mate];
        const float c = cosines[i >> 1], s = sines[i >> 1];
        y = (i & 1) ? y * c + other * s : y * c - other * s;
      }
    }
    T* keys = k_pages + ((size_t)page * G + head) * BH_PAGE * pad;
    T* values = v_pages + ((size_t)page * G + head) * BH_PAGE * pad;
    keys[bh_key_index(kv_order, token, i, pad)] = from_f32<T>(y);
    values[bh_value_index(kv_order, token, i, pad)] = from_f32<T>(i < vdim ? v[head * vdim + i] : 0.f);
  }
}

extern "C" int bh_conv_norm_rope_write(const void* proj, int dtype, int row_stride, int first, const float* w_conv, int taps,
                                       const float* state, long slot_stride, const int32_t* seq_start, const int32_t* seq_slot,
                                       const float* wq, const float* wk, float eps, const float* freq, int turned,
                                       const int32_t* positions, const int32_t* row_seq, void* q_out, void* k_pages, void* v_pages,
                                       const int32_t* page_table, int table_stride, int n_rows, int H, int G, int dim, int vdim, int pad,
                                       int kv_order, int write, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && G > 0 && dim > 0 && vdim > 0, "conv_norm_rope_write: sizes must be positive");
  BH_REQUIRE(pad >= dim && pad >= vdim, "conv_norm_rope_write: heads of %d do not hold keys of %d and values of %d", pad, dim, vdim);
  BH_REQUIRE(turned == 0 || (turned % 2 == 0 && turned <= dim && dim % 2 == 0 && freq != nullptr),
             "conv_norm_rope_write: %d turned dimensions of %d", turned, dim);
  BH_REQUIRE(taps >= 0 && taps <= 16 && (taps <= 1 || state != nullptr) && (taps == 0 || w_conv != nullptr),
             "conv_norm_rope_write: %d taps need their weights and, beyond one, a state", taps);
  const int channels = (H + G) * dim + G * vdim;
  BH_REQUIRE(first >= 0 && first + channels <= row_stride, "conv_norm_rope_write: q, k and v lie outside a row of %d", row_stride);
  BH_REQUIRE(kv_order == BH_KV_ROWS || (kv_order == BH_KV_PIECES && pad % 32 == 0),
             "conv_norm_rope_write: cache order %d does not exist for head size %d", kv_order, pad);
  const size_t lds = (size_t)(channels + turned) * sizeof(float);
  BH_REQUIRE(lds <= 128 * 1024, "conv_norm_rope_write: %d channels do not fit the local memory", channels);
  const int threads = n_rows < 2 * bh_compute_units() && channels >= 2048 ? 1024 : 256;      // few rows: more of the chip a row
#define BH_CW(T)                                                                                                                   \
  do {                                                                                                                             \
    bh_allow_lds<conv_norm_rope_write_kernel<T>>(lds);                                                                             \
    conv_norm_rope_write_kernel<T><<<n_rows, threads, lds, stream>>>((const T*)proj, row_stride, first, w_conv, taps, state, slot_stride,  \
                                                                 seq_start, seq_slot, wq, wk, eps, freq, turned, positions, row_seq, \
                                                                 (T*)q_out, (T*)k_pages, (T*)v_pages, page_table, table_stride, H, G, \
                                                                 dim, vdim, pad, kv_order, write);                                  \
  } while (0)
  if (dtype == BH_F32) BH_CW(float);
  else if (dtype == BH_BF16) BH_CW(bf16_t);
  else return bh_fail("conv_norm_rope_write: unknown dtype %d", dtype);
#undef BH_CW
  return bh_check_launch("conv_norm_rope_write");
}

template <typename T>
__global__ __launch_bounds__(256) void gate_heads_kernel(const T* __restrict__ attended, int pad, const T* __restrict__ gate,
                                                         int gate_stride, int gate_first, T* __restrict__ out, int n_rows, int H,
                                                         int vdim, int out_block_rows, int gate_per_head) {
  const int width = H * vdim;
  const size_t n = (size_t)n_rows * width;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const int r = (int)(e / width), c = (int)(e % width), head = c / vdim, i = c % vdim;
    const float a = to_f32(attended[((size_t)r * H + head) * pad + i]);
    if (gate == nullptr) {      // no gate: the heads' first vdim elements, side by side
      out[bh_rows_index(out_block_rows, r, c, width)] = from_f32<T>(a);
      continue;
    }
    const float g = to_f32(gate[(size_t)r * gate_stride + gate_first + (gate_per_head ? head : c)]);
    out[bh_rows_index(out_block_rows, r, c, width)] = from_f32<T>(a / (1.0f + expf(-g)));
  }
}

extern "C" int bh_gate_heads(const void* attended, int dtype, int pad, const void* gate, int gate_stride, int gate_first,
                             void* out, int n_rows, int H, int vdim, int out_block_rows, int gate_per_head, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && vdim > 0 && pad >= vdim, "gate_heads: sizes do not fit");
  BH_REQUIRE(gate == nullptr || (gate_first >= 0 && gate_first + (gate_per_head ? H : H * vdim) <= gate_stride),
             "gate_heads: the gate lies outside its row");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && (H * vdim) % 32 == 0 && dtype == BH_BF16),
             "gate_heads: rows in blocks of %d of width %d are not written", out_block_rows, H * vdim);
  const size_t n = (size_t)n_rows * H * vdim;
  const int blocks = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  if (dtype == BH_F32)
    gate_heads_kernel<float><<<blocks, 256, 0, stream>>>((const float*)attended, pad, (const float*)gate, gate_stride, gate_first,
                                                       (float*)out, n_rows, H, vdim, out_block_rows, gate_per_head);
  else if (dtype == BH_BF16)
    gate_heads_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)attended, pad, (const bf16_t*)gate, gate_stride, gate_first,
                                                        (bf16_t*)out, n_rows, H, vdim, out_block_rows, gate_per_head);
  else
    return bh_fail("gate_heads: unknown dtype %d", dtype);
  return bh_check_launch("gate_heads");
}
