// A selective state-space recurrence with a scalar decay per head (the "state-space duality" form), kept as a
// recurrent state, and the gated norm behind it:
//   ssm_scan            per (sequence, head): dt = softplus(dt_raw + dt_bias);  S <- exp(-exp(A_log) dt) S + dt B x^T;
//                       y = S^T C + D x.   S is [N][vdim] float32 and lives in the sequence's state region.
//   gated_group_rmsnorm out = rms_g(y * silu(z)) * w, the root mean square taken in `groups` equal parts of a row; with
//                       `gate_after` the statistic is y's alone: out = rms_g(y) * w * silu(z)
// Everything but the reading of dt_raw and z is float32.
#include "common.h"

__device__ inline float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// One workgroup a (sequence, head): thread (p, s) owns column p of the state for the rows n of slice s; the state
// stays in LDS over the rows of the step, a thread touching only its own elements.  A row's B, C, x and dt go
// through LDS once; the slices' shares of y are added in slice order.
template <typename T>
__global__ __launch_bounds__(256) void ssm_scan_kernel(const float* __restrict__ xbc, int xbc_stride, const T* __restrict__ proj,
                                                       int proj_stride, int dt_first, const float* __restrict__ dt_bias,
                                                       const float* __restrict__ a_log, const float* __restrict__ d_skip,
                                                       float* __restrict__ state, long slot_stride,
                                                       const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                                       float* __restrict__ y, int H, int vdim, int N, int G, int slices) {
  extern __shared__ float lds[];
  float* S = lds;                          // [N][vdim]
  float* bc = S + (size_t)N * vdim;        // B [N], C [N]
  float* xs = bc + 2 * N;                  // x [vdim]
  float* part = xs + vdim;                 // [slices][vdim]
  __shared__ float step[2];                // decay, dt
  const int seq = blockIdx.x, head = blockIdx.y, group = head / (H / G);
  const int inner = H * vdim;
  const int start = seq_start[seq], stop = seq_start[seq + 1];
  float* mine = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * N * vdim;
  for (int e = threadIdx.x; e < N * vdim; e += blockDim.x) S[e] = mine[e];
  const int p = threadIdx.x % vdim, s = threadIdx.x / vdim;
  const bool works = s < slices;
  const int per = (N + slices - 1) / slices;
  const int n0 = s * per, n1 = (n0 + per < N) ? n0 + per : N;
  const float rate = expf(a_log[head]), skip = d_skip[head], bias = dt_bias[head];
  __syncthreads();
  for (int row = start; row < stop; ++row) {
    const float* in = xbc + (size_t)row * xbc_stride;
    for (int e = threadIdx.x; e < 2 * N; e += blockDim.x)
      bc[e] = in[inner + (e < N ? 0 : G * N) + group * N + (e < N ? e : e - N)];
    for (int e = threadIdx.x; e < vdim; e += blockDim.x) xs[e] = in[head * vdim + e];
    if (threadIdx.x == 0) {
      const float dt = softplus_f32(to_f32(proj[(size_t)row * proj_stride + dt_first + head]) + bias);
      step[0] = expf(-rate * dt);
      step[1] = dt;
    }
    __syncthreads();
    if (works) {
      const float decay = step[0], dtx = step[1] * xs[p];
      float acc = 0.f;
      for (int n = n0; n < n1; ++n) {
        const float v = fmaf(decay, S[n * vdim + p], bc[n] * dtx);
        S[n * vdim + p] = v;
        acc = fmaf(v, bc[N + n], acc);
      }
      part[s * vdim + p] = acc;
    }
    __syncthreads();
    if (threadIdx.x < vdim) {
      float total = skip * xs[threadIdx.x];
      for (int k = 0; k < slices; ++k) total += part[k * vdim + threadIdx.x];
      y[(size_t)row * inner + head * vdim + threadIdx.x] = total;
    }
    __syncthreads();
  }
  for (int e = threadIdx.x; e < N * vdim; e += blockDim.x) mine[e] = S[e];
}

extern "C" int bh_ssm_scan(const float* xbc, int xbc_stride, const void* proj, int dtype, int proj_stride, int dt_first,
                           const float* dt_bias, const float* a_log, const float* d_skip, float* state, long slot_stride,
                           const int32_t* seq_start, const int32_t* seq_slot, float* y, int n_seqs, int H, int vdim, int N, int G,
                           hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && vdim > 0 && N > 0 && G > 0, "ssm_scan: sizes must be positive");
  BH_REQUIRE(H % G == 0, "ssm_scan: %d heads do not fall into %d groups evenly", H, G);
  BH_REQUIRE(vdim <= 256, "ssm_scan: heads of up to 256 values, got %d", vdim);
  BH_REQUIRE(xbc_stride >= H * vdim + 2 * G * N, "ssm_scan: a row of %d does not hold x, B and C", xbc_stride);
  BH_REQUIRE(dt_first >= 0 && dt_first + H <= proj_stride, "ssm_scan: the step sizes lie outside their row");
  int slices = 256 / vdim;
  if (slices > N) slices = N;
  const size_t lds_bytes = ((size_t)N * vdim + 2 * N + vdim + (size_t)slices * vdim) * sizeof(float);
  BH_REQUIRE(lds_bytes <= 160 * 1024 - 64, "ssm_scan: a state of %d x %d does not fit the local memory", N, vdim);
  dim3 grid(n_seqs, H);
  if (dtype == BH_F32) {
    bh_allow_lds<ssm_scan_kernel<float>>(lds_bytes);
    ssm_scan_kernel<float><<<grid, 256, lds_bytes, stream>>>(xbc, xbc_stride, (const float*)proj, proj_stride, dt_first, dt_bias, a_log,
                                                             d_skip, state, slot_stride, seq_start, seq_slot, y, H, vdim, N, G, slices);
  } else if (dtype == BH_BF16) {
    bh_allow_lds<ssm_scan_kernel<bf16_t>>(lds_bytes);
    ssm_scan_kernel<bf16_t><<<grid, 256, lds_bytes, stream>>>(xbc, xbc_stride, (const bf16_t*)proj, proj_stride, dt_first, dt_bias,
                                                              a_log, d_skip, state, slot_stride, seq_start, seq_slot, y, H, vdim, N, G,
                                                              slices);
  } else {
    return bh_fail("ssm_scan: unknown dtype %d", dtype);
  }
  return bh_check_launch("ssm_scan");
}

// ---- the same recurrence with the state in registers ------------------------------------------------------------
// Thread (p, s) keeps its NPT state rows of column p in registers; SS_STAGE rows of B, C, x and the step sizes go through
// LDS at a time, and the slices' shares of those rows' outputs are added in slice order.  A long sequence is cut into
// chunks of rows that run side by side:
//   MODE 1  every chunk walks its rows from a zero state, leaves its rows' outputs, its final state and, for every row,
//           the logarithm of the decay from the chunk's start up to and including that row
//   ssm_combine  goes through a sequence's chunks in order: the state a chunk truly starts from replaces the chunk's own
//           in the scratch memory, and the state after the last chunk goes to the sequence's region
//   MODE 2  every chunk adds to its rows what its true starting state owes them: y_t += exp(cum_t) S_in^T C_t
// MODE 0 is a sequence in one piece, from and to its region (decode steps, short prompts).
#define SS_STAGE 16

template <typename T, int NPT, int MODE>
__global__ __launch_bounds__(256) void ssm_chunk_kernel(const float* __restrict__ xbc, int xbc_stride, const T* __restrict__ proj,
                                                        int proj_stride, int dt_first, const float* __restrict__ dt_bias,
                                                        const float* __restrict__ a_log, const float* __restrict__ d_skip,
                                                        float* __restrict__ state, long slot_stride, float* __restrict__ chunk_states,
                                                        float* __restrict__ chunk_decay, float* __restrict__ cum,
                                                        const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                                        float* __restrict__ y, int H, int vdim, int N, int G, int slices, int chunk_rows,
                                                        int chunks_per_seq) {
  extern __shared__ __align__(16) float lds[];
  float* bc = lds;                                 // [SS_STAGE][2 N]: B, C of a row
  float* xs = bc + SS_STAGE * 2 * N;               // [SS_STAGE][vdim]
  float* part = xs + SS_STAGE * vdim;              // [SS_STAGE][slices][vdim]
  float* fac = part + SS_STAGE * slices * vdim;    // [SS_STAGE][2]: log decay (MODE 2: the decay since the chunk's start), dt
  const int seq = blockIdx.x / chunks_per_seq, chunk = blockIdx.x % chunks_per_seq, head = blockIdx.y;
  const int seq_stop = seq_start[seq + 1];
  const int start = seq_start[seq] + chunk * chunk_rows;
  if (start >= seq_stop) return;
  const int stop = start + chunk_rows < seq_stop ? start + chunk_rows : seq_stop;
  const int group = head / (H / G), inner = H * vdim;
  const int p = threadIdx.x % vdim, s = threadIdx.x / vdim;
  const bool works = s < slices;
  const int per = (N + slices - 1) / slices;
  const int n0 = s * per, n1 = n0 + per < N ? n0 + per : N;
  float* home = MODE == 0 ? state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * N * vdim
                          : chunk_states + ((size_t)blockIdx.x * H + head) * N * vdim;
  float S[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) S[i] = (MODE != 1 && works && n0 + i < n1) ? home[(size_t)(n0 + i) * vdim + p] : 0.f;
  const float rate = expf(a_log[head]), skip = d_skip[head], bias = dt_bias[head];
  float run = 0.f;
  const int staged = 2 * N + vdim;      // a row's B, C and x, as they are asked for: eight loads a thread in flight
  const bool by_four = per % 4 == 0 && N % 4 == 0;
  for (int r0 = start; r0 < stop; r0 += SS_STAGE) {
    const int rows = stop - r0 < SS_STAGE ? stop - r0 : SS_STAGE;
    for (int e0 = threadIdx.x; e0 < rows * staged; e0 += 8 * blockDim.x) {
      float got[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = e0 + u * blockDim.x;
        if (e < rows * staged) {
          const int r = e / staged, j = e % staged;
          const int column = j < N ? inner + group * N + j : (j < 2 * N ? inner + (G + group) * N + j - N : head * vdim + j - 2 * N);
          got[u] = xbc[(size_t)(r0 + r) * xbc_stride + column];
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = e0 + u * blockDim.x;
        if (e < rows * staged) {
          const int r = e / staged, j = e % staged;
          if (j < 2 * N) bc[r * 2 * N + j] = got[u];
          else xs[r * vdim + j - 2 * N] = got[u];
        }
      }
    }
    if (threadIdx.x < rows) {
      if (MODE == 2) {
        fac[2 * threadIdx.x] = expf(cum[(size_t)(r0 + threadIdx.x) * H + head]);
      } else {
        const float dt = softplus_f32(to_f32(proj[(size_t)(r0 + threadIdx.x) * proj_stride + dt_first + head]) + bias);
        fac[2 * threadIdx.x] = -rate * dt;
        fac[2 * threadIdx.x + 1] = dt;
      }
    }
    __syncthreads();
    if (MODE == 1 && threadIdx.x == 0) {
      for (int r = 0; r < rows; ++r) {
        run += fac[2 * r];
        cum[(size_t)(r0 + r) * H + head] = run;
      }
    }
    if (works) {
      for (int r = 0; r < rows; ++r) {
        const float* b = bc + r * 2 * N;
        const float* c = b + N;
        float acc = 0.f;
        const float decay = MODE == 2 ? 0.f : expf(fac[2 * r]), dtx = MODE == 2 ? 0.f : fac[2 * r + 1] * xs[r * vdim + p];
        if (by_four) {      // four state rows a read of LDS
#pragma unroll
          for (int i = 0; i < NPT; i += 4) {
            if (n0 + i < n1) {
              const float4 c4 = *reinterpret_cast<const float4*>(c + n0 + i);
              if (MODE != 2) {
                const float4 b4 = *reinterpret_cast<const float4*>(b + n0 + i);
                S[i] = fmaf(decay, S[i], b4.x * dtx);
                S[i + 1] = fmaf(decay, S[i + 1], b4.y * dtx);
                S[i + 2] = fmaf(decay, S[i + 2], b4.z * dtx);
                S[i + 3] = fmaf(decay, S[i + 3], b4.w * dtx);
              }
              acc = fmaf(S[i], c4.x, acc);
              acc = fmaf(S[i + 1], c4.y, acc);
              acc = fmaf(S[i + 2], c4.z, acc);
              acc = fmaf(S[i + 3], c4.w, acc);
            }
          }
        } else {
#pragma unroll
          for (int i = 0; i < NPT; ++i) {
            if (n0 + i < n1) {
              if (MODE != 2) S[i] = fmaf(decay, S[i], b[n0 + i] * dtx);
              acc = fmaf(S[i], c[n0 + i], acc);
            }
          }
        }
        part[(r * slices + s) * vdim + p] = acc;
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < rows * vdim; e += blockDim.x) {
      const int r = e / vdim, i = e % vdim;
      float total = 0.f;
      for (int k = 0; k < slices; ++k) total += part[(r * slices + k) * vdim + i];
      float* out = y + (size_t)(r0 + r) * inner + head * vdim + i;
      if (MODE == 2) *out += fac[2 * r] * total;
      else *out = total + skip * xs[e];
    }
    __syncthreads();
  }
  if (MODE != 2 && works) {
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      if (n0 + i < n1) home[(size_t)(n0 + i) * vdim + p] = S[i];
  }
  if (MODE == 1 && threadIdx.x == 0) chunk_decay[(size_t)blockIdx.x * H + head] = run;
}

// grid (sequences, heads): a thread per state element walks the sequence's chunks in order.
__global__ __launch_bounds__(256) void ssm_combine_kernel(float* __restrict__ state, long slot_stride, float* __restrict__ chunk_states,
                                                          const float* __restrict__ chunk_decay, const int32_t* __restrict__ seq_start,
                                                          const int32_t* __restrict__ seq_slot, int H, int elements, int chunk_rows,
                                                          int chunks_per_seq) {
  const int seq = blockIdx.x, head = blockIdx.y;
  const int n_rows = seq_start[seq + 1] - seq_start[seq];
  const int chunks = (n_rows + chunk_rows - 1) / chunk_rows;
  float* home = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * elements;
  for (int e = threadIdx.x; e < elements; e += blockDim.x) {
    float S = home[e];
    for (int c = 0; c < chunks; ++c) {
      const size_t at = (size_t)seq * chunks_per_seq + c;
      float* slot = chunk_states + (at * H + head) * elements + e;
      const float local = *slot;
      *slot = S;
      S = fmaf(expf(chunk_decay[at * H + head]), S, local);
    }
    home[e] = S;
  }
}

// How a step's sequences are cut: rows a chunk (a multiple of SS_STAGE) for sequences of up to max_rows rows, so that the
// chip has about two workgroups a compute unit where the rows allow it, and no chunk is shorter than 64 rows.
extern "C" int bh_ssm_chunk_rows(int n_seqs, int max_rows, int H) {
  if (max_rows <= 128) return max_rows < 1 ? 1 : max_rows;
  long wanted = (2L * bh_compute_units() + (long)n_seqs * H - 1) / ((long)n_seqs * H);
  const int most = max_rows / 64;
  if (wanted > most) wanted = most;
  if (wanted < 1) wanted = 1;
  const int rows = (int)((max_rows + wanted - 1) / wanted);
  return (rows + SS_STAGE - 1) / SS_STAGE * SS_STAGE;
}

// Whether the recurrence with the state in registers takes these sizes (otherwise bh_ssm_scan walks with the state in LDS).
extern "C" int bh_ssm_fast_takes(int vdim, int N) {
  if (vdim > 256 || vdim < 1 || N < 1) return 0;
  int slices = 256 / vdim;
  if (slices > N) slices = N;
  const int per = (N + slices - 1) / slices;
  const size_t lds = ((size_t)SS_STAGE * (2 * N + vdim + slices * vdim + 2)) * sizeof(float);
  return per <= 128 && lds <= 150 * 1024;
}

template <typename T, int NPT>
static int ssm_fast_launch(const float* xbc, int xbc_stride, const T* proj, int proj_stride, int dt_first, const float* dt_bias,
                           const float* a_log, const float* d_skip, float* state, long slot_stride, float* chunk_states,
                           float* chunk_decay, float* cum, const int32_t* seq_start, const int32_t* seq_slot, float* y, int n_seqs, int H,
                           int vdim, int N, int G, int slices, int chunk_rows, int chunks_per_seq, size_t lds, hipStream_t stream) {
  dim3 grid(n_seqs * chunks_per_seq, H);
#define BH_SS(MODE)                                                                                                                 \
  do {                                                                                                                              \
    bh_allow_lds<ssm_chunk_kernel<T, NPT, MODE>>(lds);                                                                              \
    ssm_chunk_kernel<T, NPT, MODE><<<grid, 256, lds, stream>>>(xbc, xbc_stride, proj, proj_stride, dt_first, dt_bias, a_log, d_skip,   \
                                                               state, slot_stride, chunk_states, chunk_decay, cum, seq_start, seq_slot, \
                                                               y, H, vdim, N, G, slices, chunk_rows, chunks_per_seq);                \
  } while (0)
  if (chunks_per_seq == 1) {
    BH_SS(0);
    return bh_check_launch("ssm_scan");
  }
  BH_SS(1);
  ssm_combine_kernel<<<dim3(n_seqs, H), 256, 0, stream>>>(state, slot_stride, chunk_states, chunk_decay, seq_start, seq_slot, H, N * vdim,
                                                         chunk_rows, chunks_per_seq);
  BH_SS(2);
#undef BH_SS
  return bh_check_launch("ssm_scan in chunks");
}

// chunk_states [n_seqs * chunks_per_seq][H][N][vdim], chunk_decay [n_seqs * chunks_per_seq][H] and cum [rows][H] are scratch
// memory of the call (unused, and may be null, with one chunk a sequence).
extern "C" int bh_ssm_scan_fast(const float* xbc, int xbc_stride, const void* proj, int dtype, int proj_stride, int dt_first,
                                const float* dt_bias, const float* a_log, const float* d_skip, float* state, long slot_stride,
                                float* chunk_states, float* chunk_decay, float* cum, const int32_t* seq_start, const int32_t* seq_slot,
                                float* y, int n_seqs, int H, int vdim, int N, int G, int chunk_rows, int chunks_per_seq,
                                hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && G > 0 && H % G == 0, "ssm_scan: %d heads in %d groups", H, G);
  BH_REQUIRE(bh_ssm_fast_takes(vdim, N), "ssm_scan: the form with the state in registers does not take heads of %d with %d rows", vdim, N);
  BH_REQUIRE(xbc_stride >= H * vdim + 2 * G * N, "ssm_scan: a row of %d does not hold x, B and C", xbc_stride);
  BH_REQUIRE(dt_first >= 0 && dt_first + H <= proj_stride, "ssm_scan: the step sizes lie outside their row");
  BH_REQUIRE(chunk_rows > 0 && chunks_per_seq > 0 && (chunks_per_seq == 1 || (chunk_rows % SS_STAGE == 0 && chunk_states && chunk_decay && cum)),
             "ssm_scan: chunks of a multiple of %d rows with their scratch memory", SS_STAGE);
  int slices = 256 / vdim;
  if (slices > N) slices = N;
  const int per = (N + slices - 1) / slices;
  const size_t lds = ((size_t)SS_STAGE * (2 * N + vdim + slices * vdim + 2)) * sizeof(float);
#define BH_SF(T, NPT)                                                                                                              \
  return ssm_fast_launch<T, NPT>(xbc, xbc_stride, (const T*)proj, proj_stride, dt_first, dt_bias, a_log, d_skip, state, slot_stride, \
                                 chunk_states, chunk_decay, cum, seq_start, seq_slot, y, n_seqs, H, vdim, N, G, slices, chunk_rows,   \
                                 chunks_per_seq, lds, stream)
  if (dtype == BH_F32) {
    if (per <= 8) BH_SF(float, 8);
    if (per <= 32) BH_SF(float, 32);
    BH_SF(float, 128);
  } else if (dtype == BH_BF16) {
    if (per <= 8) BH_SF(bf16_t, 8);
    if (per <= 32) BH_SF(bf16_t, 32);
    BH_SF(bf16_t, 128);
  }
#undef BH_SF
  return bh_fail("ssm_scan: unknown dtype %d", dtype);
}

// One workgroup a (row, group).
template <typename T>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(const float* __restrict__ y, const T* __restrict__ z, int z_stride,
                                                                  int z_first, const float* __restrict__ w, float eps,
                                                                  T* __restrict__ out, int width, int groups, int out_block_rows,
                                                                  int gate_after) {
  __shared__ float scratch[8];
  const int row = blockIdx.x, per = width / groups, c0 = blockIdx.y * per;
  const float* src = y + (size_t)row * width + c0;
  const T* gate = z + (size_t)row * z_stride + z_first + c0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < per; i += blockDim.x) {
    const float g = to_f32(gate[i]);
    const float v = gate_after ? src[i] : src[i] * (g / (1.0f + expf(-g)));
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)per + eps);
  for (int i = threadIdx.x; i < per; i += blockDim.x) {
    const float g = to_f32(gate[i]);
    const float v = src[i] * (g / (1.0f + expf(-g)));      // the gate's factor commutes with the norm's
    out[bh_rows_index(out_block_rows, row, c0 + i, width)] = from_f32<T>(v * inv * w[c0 + i]);
  }
}

// The same with a wave a group, for groups of up to 512 elements (the heads of a row normed one by one): a workgroup takes a
// row, its four waves the row's groups in turn, a lane keeps its elements in registers between the statistic and the write.
template <typename T>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_waves_kernel(const float* __restrict__ y, const T* __restrict__ z, int z_stride,
                                                                        int z_first, const float* __restrict__ w, float eps,
                                                                        T* __restrict__ out, int width, int groups, int out_block_rows,
                                                                        int gate_after) {
  const int row = blockIdx.x, per = width / groups, lane = threadIdx.x % BH_WAVE;
  for (int group = threadIdx.x / BH_WAVE; group < groups; group += 4) {
    const int c0 = group * per;
    const float* src = y + (size_t)row * width + c0;
    const T* gate = z + (size_t)row * z_stride + z_first + c0;
    float held[8], gates[8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = lane + i * BH_WAVE;
      held[i] = gates[i] = 0.f;
      if (c < per) {
        const float g = to_f32(gate[c]);
        gates[i] = g / (1.0f + expf(-g));
        held[i] = gate_after ? src[c] : src[c] * gates[i];
        ss += held[i] * held[i];
      }
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)per + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = lane + i * BH_WAVE;
      if (c < per) out[bh_rows_index(out_block_rows, row, c0 + c, width)] = from_f32<T>(held[i] * (gate_after ? gates[i] : 1.0f) * inv * w[c0 + c]);
    }
  }
}

extern "C" int bh_gated_group_rmsnorm(const float* y, const void* z, int dtype, int z_stride, int z_first, const float* w, float eps,
                                      void* out, int n_rows, int width, int groups, int out_block_rows, int gate_after,
                                      hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0 && groups > 0 && width % groups == 0, "gated_group_rmsnorm: %d columns in %d equal parts", width,
             groups);
  BH_REQUIRE(z_first >= 0 && z_first + width <= z_stride, "gated_group_rmsnorm: the gate lies outside its row");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && width % 32 == 0 && dtype == BH_BF16),
             "gated_group_rmsnorm: rows in blocks of %d of width %d are not written", out_block_rows, width);
  dim3 grid(n_rows, groups);
  if (groups > 1 && width / groups <= 8 * BH_WAVE && n_rows >= bh_compute_units() / 2) {      // many rows of small groups: a wave a group
    if (dtype == BH_F32)
      gated_group_rmsnorm_waves_kernel<float><<<n_rows, 256, 0, stream>>>(y, (const float*)z, z_stride, z_first, w, eps, (float*)out, width,
                                                                          groups, out_block_rows, gate_after);
    else if (dtype == BH_BF16)
      gated_group_rmsnorm_waves_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(y, (const bf16_t*)z, z_stride, z_first, w, eps, (bf16_t*)out, width,
                                                                           groups, out_block_rows, gate_after);
    else
      return bh_fail("gated_group_rmsnorm: unknown dtype %d", dtype);
    return bh_check_launch("gated_group_rmsnorm");
  }
  if (dtype == BH_F32)
    gated_group_rmsnorm_kernel<float><<<grid, 256, 0, stream>>>(y, (const float*)z, z_stride, z_first, w, eps, (float*)out, width, groups,
                                                                out_block_rows, gate_after);
  else if (dtype == BH_BF16)
    gated_group_rmsnorm_kernel<bf16_t><<<grid, 256, 0, stream>>>(y, (const bf16_t*)z, z_stride, z_first, w, eps, (bf16_t*)out, width,
                                                                 groups, out_block_rows, gate_after);
  else
    return bh_fail("gated_group_rmsnorm: unknown dtype %d", dtype);
  return bh_check_launch("gated_group_rmsnorm");
}
