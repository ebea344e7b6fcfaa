// What stands ahead of the paged attention kernels for an attention whose projections carry biases, whose queries and
// keys are normed head by head with one weight for all heads, and whose rotation turns the first dimensions of a head,
// dimension i with dimension i + turned/2:
//   head_norm_rope_write   per row of the stacked projection [q | k | v] (from column `first` of a wider row):
//                          x <- x + bias;  every head of q and k: x / sqrt(mean(x^2 over the head's dim) + eps) * w  (w [dim],
//                          the same for all heads; without w no norm);  dimensions i and i + turned/2 (i < turned/2) of every
//                          head of q and k turned by position * freq[i];  q into a matrix of heads of `pad` dimensions, k and v
//                          into the cache pages of (sequence, position) as heads of `pad` (zeros beyond dim and vdim), so that
//                          keys of one size and values of another go through kernels that know one head size.
// Sums, statistics, angles, cosines and sines are float32; the angle is the float32 product position * freq[i].
#include "common.h"

#define HN_WAVES 4

// A workgroup a row and a stretch of `per_group` heads (the heads of q, then those of k, then those of v, numbered through), a
// wave a head at a time.  The head stands in the wave's own stretch of LDS between the statistic and the rotation, which
// needs a dimension's mate.  Few rows: a stretch is one head a wave, so that a decode step's heads run side by side.
template <typename T>
__global__ __launch_bounds__(HN_WAVES * BH_WAVE) void head_norm_rope_write_kernel(
    const T* __restrict__ proj, int row_stride, int first, const float* __restrict__ bias, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const float* __restrict__ freq, int turned, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_seq, T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int32_t* __restrict__ page_table, int table_stride, int H, int G, int dim, int vdim, int pad, int kv_order, int write,
    int per_group, int neighbours, float magnitude) {
  extern __shared__ float lds[];      // the cosines and sines of the row's turned pairs, then a head of `dim` floats a wave
  const int row = blockIdx.x, wave = threadIdx.x / BH_WAVE, lane = threadIdx.x % BH_WAVE;
  const int half = turned / 2;
  float* cosines = lds;
  float* sines = lds + half;
  float* mine = lds + turned + wave * dim;
  const int pos = positions[row];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float angle = (float)pos * freq[i];
    cosines[i] = cosf(angle) * magnitude;
    sines[i] = sinf(angle) * magnitude;
  }
  __syncthreads();
  const T* x = proj + (size_t)row * row_stride + first;
  const int q_width = H * dim, k_width = G * dim;
  int page = 0;
  const int token = pos % BH_PAGE;
  if (write) page = page_table[(size_t)row_seq[row] * table_stride + pos / BH_PAGE];
  const int heads = write ? H + 2 * G : H;
  const int stretch_end = ((int)blockIdx.y + 1) * per_group < heads ? ((int)blockIdx.y + 1) * per_group : heads;
  for (int unit = blockIdx.y * per_group + wave; unit < stretch_end; unit += HN_WAVES) {
    if (unit >= H + G) {      // a head of values: the bias, and zeros beyond vdim
      const int head = unit - H - G, at = q_width + k_width + head * vdim;
      T* values = v_pages + ((size_t)page * G + head) * BH_PAGE * pad;
      for (int i = lane; i < pad; i += BH_WAVE) {
        const float v = i < vdim ? to_f32(x[at + i]) + (bias ? bias[at + i] : 0.f) : 0.f;
        values[bh_value_index(kv_order, token, i, pad)] = from_f32<T>(v);
      }
      continue;
    }
    const bool is_key = unit >= H;
    const int head = is_key ? unit - H : unit, at = (is_key ? q_width : 0) + head * dim;
    const float* w = is_key ? wk : wq;
    float ss = 0.f;
    for (int i = lane; i < dim; i += BH_WAVE) {
      const float v = to_f32(x[at + i]) + (bias ? bias[at + i] : 0.f);
      mine[i] = v;
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = w ? 1.0f / sqrtf(ss / (float)dim + eps) : 1.0f;
    // (a wave's lanes run together: what the lanes wrote above is there for all of them below)
    __builtin_amdgcn_wave_barrier();
    T* keys = is_key ? k_pages + ((size_t)page * G + head) * BH_PAGE * pad : nullptr;
    T* queries = q_out + ((size_t)row * H + head) * pad;
    for (int i = lane; i < pad; i += BH_WAVE) {
      float y = 0.f;
      if (i < dim) {
        y = mine[i] * inv * (w ? w[i] : 1.f);
        if (i < turned) {
          // the pair's mate: i + half and i - half, or the neighbour (2 pair, 2 pair + 1)
          const int pair = neighbours ? i / 2 : (i < half ? i : i - half);
          const bool is_first = neighbours ? (i % 2 == 0) : (i < half);
          const int mate = neighbours ? (i ^ 1) : (i < half ? i + half : i - half);
          const float other = mine[mate] * inv * (w ? w[mate] : 1.f);
          const float c = cosines[pair], s = sines[pair];
          y = is_first ? y * c - other * s : y * c + other * s;
        }
      }
      if (is_key) keys[bh_key_index(kv_order, token, i, pad)] = from_f32<T>(y);
      else queries[i] = from_f32<T>(y);
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// proj [n_rows][row_stride]: a row holds, from `first`, H heads of q and G heads of k of `dim` and G heads of v of `vdim`;
// bias f32 over those channels, or null; wq, wk f32 [dim], both or neither.  Pages as the attention kernels take them for G
// kv heads of size `pad` (written when `write` is set); q_out [n_rows][H * pad].  `neighbours`: a turned pair is
// dimensions 2i and 2i + 1 instead of i and i + turned/2; `magnitude` multiplies every cosine and sine.
extern "C" int bh_head_norm_rope_write(const void* proj, int dtype, int row_stride, int first, const float* bias, const float* wq,
                                       const float* wk, float eps, const float* freq, int turned, const int32_t* positions,
                                       const int32_t* row_seq, void* q_out, void* k_pages, void* v_pages, const int32_t* page_table,
                                       int table_stride, int n_rows, int H, int G, int dim, int vdim, int pad, int kv_order, int write,
                                       int neighbours, float magnitude, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && G > 0 && dim > 0 && vdim > 0, "head_norm_rope_write: sizes must be positive");
  BH_REQUIRE(pad >= dim && pad >= vdim, "head_norm_rope_write: heads of %d do not hold keys of %d and values of %d", pad, dim, vdim);
  BH_REQUIRE(turned >= 0 && turned % 2 == 0 && turned <= dim, "head_norm_rope_write: %d turned dimensions of %d", turned, dim);
  BH_REQUIRE(turned == 0 || freq != nullptr, "head_norm_rope_write: a rotation needs its frequencies");
  BH_REQUIRE((wq == nullptr) == (wk == nullptr), "head_norm_rope_write: give both norm weights or neither");
  BH_REQUIRE(first >= 0 && first + (H + G) * dim + G * vdim <= row_stride, "head_norm_rope_write: q, k and v lie outside a row of %d", row_stride);
  BH_REQUIRE(kv_order == BH_KV_ROWS || (kv_order == BH_KV_PIECES && pad % 32 == 0),
             "head_norm_rope_write: cache order %d does not exist for head size %d", kv_order, pad);
  const size_t lds = (size_t)(turned + HN_WAVES * dim) * sizeof(float);
  BH_REQUIRE(lds <= 48 * 1024, "head_norm_rope_write: heads of %d dimensions do not fit the local memory", dim);
  const int heads = write ? H + 2 * G : H;
  const int per_group = n_rows >= 4 * bh_compute_units() ? 4 * HN_WAVES : HN_WAVES;      // many rows fill the chip by themselves
  const dim3 grid(n_rows, (heads + per_group - 1) / per_group);
  BH_REQUIRE(grid.y <= 65535, "head_norm_rope_write: too many heads");
#define BH_HN(T)                                                                                                                  \
  head_norm_rope_write_kernel<T><<<grid, HN_WAVES * BH_WAVE, lds, stream>>>((const T*)proj, row_stride, first, bias, wq, wk, eps, freq, \
                                                                           turned, positions, row_seq, (T*)q_out, (T*)k_pages,    \
                                                                           (T*)v_pages, page_table, table_stride, H, G, dim, vdim, \
                                                                           pad, kv_order, write, per_group, neighbours, magnitude)
  if (dtype == BH_F32) BH_HN(float);
  else if (dtype == BH_BF16) BH_HN(bf16_t);
  else return bh_fail("head_norm_rope_write: unknown dtype %d", dtype);
#undef BH_HN
  return bh_check_launch("head_norm_rope_write");
}
