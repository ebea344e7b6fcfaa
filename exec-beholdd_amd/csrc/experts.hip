// Routed experts: each row chooses `top` of E small gated feed-forward layers by the largest router logits and
// adds their outputs, weighted by the softmax over the chosen logits alone.
//   route_top_k        chosen [rows][top] (int32, largest first, ties to the lower index) and weights [rows][top]
//   experts_gate_up    per (row, chosen expert): inner = act(Wg_e h, Wu_e h)             (weights read per pair: the
//   experts_down       per row: h_res += sum_j weight_j * Wd_ej inner_j, j in order       form for steps of few rows)
//   clamped_glu        act over a stacked [gate | up] matrix (the shared expert, and experts run as products of rows)
//   act(g, u) = g' * sigmoid(alpha g') * (u' + shift),  g' = min(g, limit),  u' = clamp(u, -limit, limit)
//               (an infinite limit, alpha 1 and shift 0 give silu(g) * u)
// A router may score by the sigmoid of every chosen logit instead (`scoring` 1), and a pair's weight may multiply the
// expert's input instead of its output: W (w h) = w (W h), so the gate and up sums are multiplied ahead of the activation.
// Router logits, the softmax and all sums are float32.
#include "common.h"

__device__ inline float clamped_glu(float g, float u, float limit, float alpha, float shift) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + shift);
}

#define ROUTE_MAX_TOP 32
#define ROUTE_PER_LANE 16      // experts a lane holds: up to 1024 experts

// One wave a row: a lane holds the logits of experts lane, lane + 64, ...; the largest is found `top` times over, each time
// without those already taken (ties go to the lower index).
__global__ __launch_bounds__(256) void route_top_k_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                         int32_t* __restrict__ chosen, float* __restrict__ weights, int n_rows,
                                                         int E, int top, int scoring) {
  const int lane = threadIdx.x & (BH_WAVE - 1), row = blockIdx.x * (blockDim.x / BH_WAVE) + threadIdx.x / BH_WAVE;
  if (row >= n_rows) return;
  const float* z = logits + (size_t)row * E;
  float v[ROUTE_PER_LANE];
#pragma unroll
  for (int i = 0; i < ROUTE_PER_LANE; ++i) {
    const int e = lane + i * BH_WAVE;
    v[i] = e < E ? z[e] + (bias ? bias[e] : 0.f) : -INFINITY;
  }
  unsigned taken = 0;      // bit i: this lane's expert lane + 64 i was chosen
  float largest = 0.f, sum = 0.f, mine = 0.f;      // lane j keeps the j-th choice's exponential
  int mine_index = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
      const int e = lane + i * BH_WAVE;
      if (e < E && !((taken >> i) & 1u) && (v[i] > best || best_e == 0x7fffffff)) {
        best = v[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int off = BH_WAVE / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, BH_WAVE);
      const int other_e = __shfl_xor(best_e, off, BH_WAVE);
      if (other_e != 0x7fffffff && (best_e == 0x7fffffff || other > best || (other == best && other_e < best_e))) {
        best = other;
        best_e = other_e;
      }
    }
    if ((best_e & (BH_WAVE - 1)) == lane) taken |= 1u << (best_e / BH_WAVE);
    if (j == 0) largest = best;
    const float p = scoring ? 1.0f / (1.0f + expf(-best)) : expf(best - largest);
    sum += p;
    if (lane == j) {
      mine = p;
      mine_index = best_e;
    }
  }
  if (lane < top) {
    chosen[(size_t)row * top + lane] = mine_index;
    weights[(size_t)row * top + lane] = scoring ? mine : mine / sum;
  }
}

extern "C" int bh_route_top_k(const float* logits, const float* bias, int32_t* chosen, float* weights, int n_rows, int E, int top,
                              int scoring, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && E > 0 && E <= BH_WAVE * ROUTE_PER_LANE, "route_top_k: 1 to %d experts, got %d", BH_WAVE * ROUTE_PER_LANE, E);
  BH_REQUIRE(top >= 1 && top <= E && top <= ROUTE_MAX_TOP, "route_top_k: 1 to min(%d, %d) experts a row, got %d", E, ROUTE_MAX_TOP, top);
  route_top_k_kernel<<<(n_rows + 3) / 4, 256, 0, stream>>>(logits, bias, chosen, weights, n_rows, E, top, scoring);
  return bh_check_launch("route_top_k");
}

// A wave's dot product of a weight row with a vector kept in LDS as float32; every lane gets the sum.
template <typename T>
__device__ inline float wave_dot(const T* __restrict__ w, const float* __restrict__ x, int K, int lane) {
  float acc = 0.f;
  if (K % 4 == 0) {
    for (int k = lane * 4; k < K; k += BH_WAVE * 4) {
      acc = fmaf(to_f32(w[k]), x[k], acc);
      acc = fmaf(to_f32(w[k + 1]), x[k + 1], acc);
      acc = fmaf(to_f32(w[k + 2]), x[k + 2], acc);
      acc = fmaf(to_f32(w[k + 3]), x[k + 3], acc);
    }
  } else {
    for (int k = lane; k < K; k += BH_WAVE) acc = fmaf(to_f32(w[k]), x[k], acc);
  }
  return wave_sum(acc);
}

#define EX_WAVES 4
#define EX_OUTS 16      // outputs a workgroup computes

// grid (pairs, ceil(ff / EX_OUTS)); w_gu [E][2 ff][K]: an expert's gate rows, then its up rows.
template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const T* __restrict__ h, const int32_t* __restrict__ chosen,
                                                              const T* __restrict__ w_gu, T* __restrict__ inner, int top, int K, int ff,
                                                              float limit, float alpha, float shift,
                                                              const float* __restrict__ in_weights) {
  extern __shared__ float xs[];
  const int pair = blockIdx.x, row = pair / top, e = chosen[pair];
  for (int k = threadIdx.x; k < K; k += blockDim.x) xs[k] = to_f32(h[(size_t)row * K + k]);
  __syncthreads();
  const int lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  const T* base = w_gu + (size_t)e * 2 * ff * K;
  for (int i = wave; i < EX_OUTS; i += EX_WAVES) {
    const int o = blockIdx.y * EX_OUTS + i;
    if (o >= ff) break;
    const float g = wave_dot(base + (size_t)o * K, xs, K, lane);
    const float u = wave_dot(base + (size_t)(ff + o) * K, xs, K, lane);
    const float wgt = in_weights ? in_weights[pair] : 1.0f;
    if (lane == 0) inner[(size_t)pair * ff + o] = from_f32<T>(clamped_glu(g * wgt, u * wgt, limit, alpha, shift));
  }
}

extern "C" int bh_experts_gate_up(const void* h, int dtype, const int32_t* chosen, const void* w_gu, void* inner, int n_rows, int top,
                                  int K, int ff, float limit, float alpha, float shift, const float* in_weights, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && top > 0 && K > 0 && ff > 0, "experts_gate_up: sizes must be positive");
  BH_REQUIRE((size_t)K * sizeof(float) <= 64 * 1024, "experts_gate_up: rows of up to 16384 inputs, got %d", K);
  dim3 grid(n_rows * top, (ff + EX_OUTS - 1) / EX_OUTS);
  const size_t lds = (size_t)K * sizeof(float);
  if (dtype == BH_F32) bh_allow_lds<experts_gate_up_kernel<float>>(lds);
  if (dtype == BH_BF16) bh_allow_lds<experts_gate_up_kernel<bf16_t>>(lds);
  if (dtype == BH_F32)
    experts_gate_up_kernel<float><<<grid, 64 * EX_WAVES, lds, stream>>>((const float*)h, chosen, (const float*)w_gu, (float*)inner, top, K, ff,
                                                                       limit, alpha, shift, in_weights);
  else if (dtype == BH_BF16)
    experts_gate_up_kernel<bf16_t><<<grid, 64 * EX_WAVES, lds, stream>>>((const bf16_t*)h, chosen, (const bf16_t*)w_gu, (bf16_t*)inner, top, K,
                                                                        ff, limit, alpha, shift, in_weights);
  else
    return bh_fail("experts_gate_up: unknown dtype %d", dtype);
  return bh_check_launch("experts_gate_up");
}

// grid (rows, ceil(D / EX_OUTS)); w_d [E][D][ff].  The chosen experts' shares of an output are added in their order.
template <typename T>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ inner, const int32_t* __restrict__ chosen,
                                                           const float* __restrict__ weights, const T* __restrict__ w_d,
                                                           float* __restrict__ hidden, int top, int ff, int D) {
  extern __shared__ float xs[];      // [top][ff]
  const int row = blockIdx.x;
  for (int k = threadIdx.x; k < top * ff; k += blockDim.x) xs[k] = to_f32(inner[(size_t)row * top * ff + k]);
  __syncthreads();
  const int lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  for (int i = wave; i < EX_OUTS; i += EX_WAVES) {
    const int o = blockIdx.y * EX_OUTS + i;
    if (o >= D) break;
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = chosen[(size_t)row * top + j];
      total = fmaf(weights ? weights[(size_t)row * top + j] : 1.0f, wave_dot(w_d + ((size_t)e * D + o) * ff, xs + (size_t)j * ff, ff, lane), total);
    }
    if (lane == 0) hidden[(size_t)row * D + o] += total;
  }
}

extern "C" int bh_experts_down(const void* inner, int dtype, const int32_t* chosen, const float* weights, const void* w_d, float* hidden,
                               int n_rows, int top, int ff, int D, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && top > 0 && ff > 0 && D > 0, "experts_down: sizes must be positive");
  const size_t lds = (size_t)top * ff * sizeof(float);
  BH_REQUIRE(lds <= 64 * 1024, "experts_down: %d experts a row of %d inner values do not fit the local memory", top, ff);
  dim3 grid(n_rows, (D + EX_OUTS - 1) / EX_OUTS);
  if (dtype == BH_F32) bh_allow_lds<experts_down_kernel<float>>(lds);
  if (dtype == BH_BF16) bh_allow_lds<experts_down_kernel<bf16_t>>(lds);
  if (dtype == BH_F32)
    experts_down_kernel<float><<<grid, 64 * EX_WAVES, lds, stream>>>((const float*)inner, chosen, weights, (const float*)w_d, hidden, top, ff, D);
  else if (dtype == BH_BF16)
    experts_down_kernel<bf16_t><<<grid, 64 * EX_WAVES, lds, stream>>>((const bf16_t*)inner, chosen, weights, (const bf16_t*)w_d, hidden, top, ff,
                                                                     D);
  else
    return bh_fail("experts_down: unknown dtype %d", dtype);
  return bh_check_launch("experts_down");
}

template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_rows, int ff, float limit,
                                                          float alpha, int out_block_rows, float shift) {
  const size_t n = (size_t)n_rows * ff;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const int r = (int)(e / ff), i = (int)(e % ff);
    const float g = to_f32(gu[(size_t)r * 2 * ff + i]), u = to_f32(gu[(size_t)r * 2 * ff + ff + i]);
    out[bh_rows_index(out_block_rows, r, i, ff)] = from_f32<T>(clamped_glu(g, u, limit, alpha, shift));
  }
}

extern "C" int bh_clamped_glu(const void* gu, int dtype, void* out, int n_rows, int ff, float limit, float alpha, int out_block_rows,
                              float shift, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && ff > 0, "clamped_glu: sizes must be positive");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && ff % 32 == 0 && dtype == BH_BF16),
             "clamped_glu: rows in blocks of %d of width %d are not written", out_block_rows, ff);
  const size_t n = (size_t)n_rows * ff;
  const int blocks = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  if (dtype == BH_F32)
    clamped_glu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, n_rows, ff, limit, alpha, out_block_rows, shift);
  else if (dtype == BH_BF16)
    clamped_glu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n_rows, ff, limit, alpha, out_block_rows, shift);
  else
    return bh_fail("clamped_glu: unknown dtype %d", dtype);
  return bh_check_launch("clamped_glu");
}

// ---- the experts' work grouped by expert ----------------------------------------------------------------------
//   experts_group     for every expert the (row, choice) pairs that chose it, in the pairs' order, and their count
//   experts_rows      per expert, for its pairs: a product with that expert's matrix, the matrix read from memory once per
//                     workgroup whatever the number of pairs (gated: two rows an output and the activation; plain: float32
//                     results for experts_combine)
//   experts_gather    the pairs' input rows side by side, expert after expert, for products of many rows
//   experts_combine   h_res[row] += sum_j weight_j * y[place of pair (row, j)], j in order

// One workgroup an expert: it walks over all pairs in order and keeps those that chose it.
__global__ __launch_bounds__(256) void experts_group_kernel(const int32_t* __restrict__ chosen, int n_pairs, int32_t* __restrict__ list,
                                                            int capacity, int32_t* __restrict__ counts) {
  __shared__ int wave_count[4];
  const int e = blockIdx.x, lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  int base = 0;
  for (int p0 = 0; p0 < n_pairs; p0 += 256) {
    const int p = p0 + threadIdx.x;
    const bool mine = p < n_pairs && chosen[p] == e;
    const unsigned long long mask = __ballot(mine);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    if (lane == 0) wave_count[wave] = __popcll(mask);
    __syncthreads();
    int offset = base, total = 0;
    for (int w = 0; w < 4; ++w) {
      if (w < wave) offset += wave_count[w];
      total += wave_count[w];
    }
    if (mine) list[(size_t)e * capacity + offset + before] = p;
    base += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) counts[e] = base;
}

extern "C" int bh_experts_group(const int32_t* chosen, int n_pairs, int32_t* list, int capacity, int32_t* counts, int E, hipStream_t stream) {
  BH_REQUIRE(n_pairs > 0 && E > 0 && capacity > 0, "experts_group: sizes must be positive");
  experts_group_kernel<<<E, 256, 0, stream>>>(chosen, n_pairs, list, capacity, counts);
  return bh_check_launch("experts_group");
}

template <typename T>
__device__ inline void load8(const T* __restrict__ p, float (&v)[8]);
template <>
__device__ inline void load8<float>(const float* __restrict__ p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}
template <>
__device__ inline void load8<bf16_t>(const bf16_t* __restrict__ p, float (&v)[8]) {
  const uint4 raw = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = bf16_bits_to_f32((uint16_t)(w[i] & 0xffffu));
    v[2 * i + 1] = bf16_bits_to_f32((uint16_t)(w[i] >> 16));
  }
}

#define ER_PAIRS 8      // pairs whose sums a wave keeps at a time
#define ER_OUTS 16      // outputs a workgroup computes

// grid (E, ceil(N / ER_OUTS)).  in [*][K]: the input of pair p is row p / in_div.  w [E][GATED ? 2 N : N][K].
// GATED: out (T) [pairs][N] = act(gate row . x, up row . x);  otherwise out (float) [pairs][N] = row . x.
// A wave takes U outputs at a time, so that the loads of U (gated: 2 U) weight rows are in flight together.
// K must be a multiple of 8 (16-byte loads).
template <typename T, bool GATED, int U>
__global__ __launch_bounds__(256) void experts_rows_kernel(const T* __restrict__ in, int in_div, const int32_t* __restrict__ list, int capacity,
                                                           const int32_t* __restrict__ counts, const T* __restrict__ w, void* __restrict__ out_raw,
                                                           int K, int N, float limit, float alpha, float shift,
                                                           const float* __restrict__ in_weights) {
  const int e = blockIdx.x, count = counts[e];
  if (count == 0) return;
  const int lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  const int32_t* mine = list + (size_t)e * capacity;
  const T* base = w + (size_t)e * (GATED ? 2 : 1) * N * K;
  for (int i = wave * U; i < ER_OUTS; i += 4 * U) {
    const int o0 = blockIdx.y * ER_OUTS + i;
    if (o0 >= N) break;
    const T* row_a[U];
    const T* row_b[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int o = o0 + u < N ? o0 + u : N - 1;      // a row beyond the last is computed again and not stored
      row_a[u] = base + (size_t)o * K;
      row_b[u] = base + (size_t)(N + o) * K;
    }
    for (int p0 = 0; p0 < count; p0 += ER_PAIRS) {
      const int n_pairs = count - p0 < ER_PAIRS ? count - p0 : ER_PAIRS;
      const T* x[ER_PAIRS];
#pragma unroll
      for (int j = 0; j < ER_PAIRS; ++j) x[j] = in + (size_t)(mine[p0 + (j < n_pairs ? j : 0)] / in_div) * K;
      float acc_a[U][ER_PAIRS] = {}, acc_b[U][ER_PAIRS] = {};
      for (int k = lane * 8; k < K; k += BH_WAVE * 8) {
        float wa[U][8], wb[U][8], xv[8];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          load8<T>(row_a[u] + k, wa[u]);
          if (GATED) load8<T>(row_b[u] + k, wb[u]);
        }
#pragma unroll
        for (int j = 0; j < ER_PAIRS; ++j) {
          if (j < n_pairs) {
            load8<T>(x[j] + k, xv);
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
              for (int t = 0; t < 8; ++t) {
                acc_a[u][j] = fmaf(wa[u][t], xv[t], acc_a[u][j]);
                if (GATED) acc_b[u][j] = fmaf(wb[u][t], xv[t], acc_b[u][j]);
              }
            }
          }
        }
      }
#pragma unroll
      for (int j = 0; j < ER_PAIRS; ++j) {
        if (j >= n_pairs) break;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const float a = wave_sum(acc_a[u][j]);
          const float b = GATED ? wave_sum(acc_b[u][j]) : 0.f;
          if (lane == 0 && o0 + u < N) {
            const size_t at = (size_t)mine[p0 + j] * N + o0 + u;
            const float wgt = (GATED && in_weights) ? in_weights[mine[p0 + j]] : 1.0f;
            if (GATED) reinterpret_cast<T*>(out_raw)[at] = from_f32<T>(clamped_glu(a * wgt, b * wgt, limit, alpha, shift));
            else reinterpret_cast<float*>(out_raw)[at] = a;
          }
        }
      }
    }
  }
}

extern "C" int bh_experts_rows(const void* in, int dtype, int in_div, const int32_t* list, int capacity, const int32_t* counts, const void* w,
                               void* out, int E, int K, int N, int gated, float limit, float alpha, float shift, const float* in_weights,
                               hipStream_t stream) {
  BH_REQUIRE(E > 0 && K > 0 && N > 0 && in_div > 0 && capacity > 0, "experts_rows: sizes must be positive");
  BH_REQUIRE(K % 8 == 0, "experts_rows: rows of a multiple of 8 inputs, got %d", K);
  dim3 grid(E, (N + ER_OUTS - 1) / ER_OUTS);
#define BH_ER(T, G, U) experts_rows_kernel<T, G, U><<<grid, 256, 0, stream>>>((const T*)in, in_div, list, capacity, counts, (const T*)w, out, K, N, limit, alpha, shift, in_weights)
  if (dtype == BH_F32) {
    if (gated) BH_ER(float, true, 2);
    else BH_ER(float, false, 4);
  } else if (dtype == BH_BF16) {
    if (gated) BH_ER(bf16_t, true, 2);
    else BH_ER(bf16_t, false, 4);
  } else {
    return bh_fail("experts_rows: unknown dtype %d", dtype);
  }
#undef BH_ER
  return bh_check_launch("experts_rows");
}

// grid (E, rows of the grid's second axis walk an expert's pairs).  offsets [E]: where an expert's rows start in `sorted`.
template <typename T>
__global__ __launch_bounds__(256) void experts_gather_kernel(const T* __restrict__ x, int top, const int32_t* __restrict__ list, int capacity,
                                                             const int32_t* __restrict__ counts, const int32_t* __restrict__ offsets,
                                                             T* __restrict__ sorted, int32_t* __restrict__ place, int K,
                                                             const float* __restrict__ in_weights) {
  const int e = blockIdx.x, count = counts[e], first = offsets[e];
  for (int i = blockIdx.y; i < count; i += gridDim.y) {
    const int pair = list[(size_t)e * capacity + i];
    const T* from = x + (size_t)(pair / top) * K;
    T* to = sorted + (size_t)(first + i) * K;
    if (in_weights) {      // the pair's weight on the expert's input
      const float wgt = in_weights[pair];
      for (int k = threadIdx.x; k < K; k += blockDim.x) to[k] = from_f32<T>(to_f32(from[k]) * wgt);
    } else {
      for (int k = threadIdx.x; k < K; k += blockDim.x) to[k] = from[k];
    }
    if (threadIdx.x == 0) place[pair] = first + i;
  }
}

extern "C" int bh_experts_gather(const void* x, int dtype, int top, const int32_t* list, int capacity, const int32_t* counts,
                                 const int32_t* offsets, void* sorted, int32_t* place, int E, int K, int n_rows, const float* in_weights,
                                 hipStream_t stream) {
  BH_REQUIRE(E > 0 && K > 0 && top > 0 && n_rows > 0, "experts_gather: sizes must be positive");
  dim3 grid(E, n_rows < 256 ? n_rows : 256);
  if (dtype == BH_F32)
    experts_gather_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, top, list, capacity, counts, offsets, (float*)sorted, place, K, in_weights);
  else if (dtype == BH_BF16)
    experts_gather_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, top, list, capacity, counts, offsets, (bf16_t*)sorted, place, K, in_weights);
  else
    return bh_fail("experts_gather: unknown dtype %d", dtype);
  return bh_check_launch("experts_gather");
}

// y [*][D] float32: the result of pair p lies at row place[p] (or p where no places are given).
__global__ __launch_bounds__(256) void experts_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ place,
                                                              const float* __restrict__ weights, float* __restrict__ hidden, int top, int D) {
  const int row = blockIdx.x, d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    const int pair = row * top + j;
    total = fmaf(weights ? weights[pair] : 1.0f, y[(size_t)(place ? place[pair] : pair) * D + d], total);
  }
  hidden[(size_t)row * D + d] += total;
}

extern "C" int bh_experts_combine(const float* y, const int32_t* place, const float* weights, float* hidden, int n_rows, int top, int D,
                                  hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && top > 0 && D > 0, "experts_combine: sizes must be positive");
  BH_REQUIRE((D + 255) / 256 <= 65535, "experts_combine: rows of up to 16 million outputs");
  experts_combine_kernel<<<dim3(n_rows, (D + 255) / 256), 256, 0, stream>>>(y, place, weights, hidden, top, D);
  return bh_check_launch("experts_combine");
}
