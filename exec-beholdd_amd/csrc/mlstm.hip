// A matrix memory with exponential gates (mLSTM), walked as a recurrence over a float32 state.  Per sequence and head:
//   i_t = cap tanh(x_i / cap),  f_t = logsigmoid(cap tanh(x_f / cap))        the gates' logarithms, from their pre-activations
//   m_t = max(f_t + m_(t-1), i_t)                                            m starts at 0
//   a_t = exp(f_t + m_(t-1) - m_t),  b_t = exp(i_t - m_t)
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,   n_t = a_t n_(t-1) + b_t k_t           S [dim][vdim], n [dim], zero at the start
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// n is S's column for a value that is always one, so the state of a head is kept as vdim + 1 columns of dim floats (the
// last one n), then m: (vdim + 1) * dim + 1 floats a head, heads one after the other in a slot's row of the cache.
//   mlstm_gates    a_t, b_t and m_t of every row and head, the rows of a sequence in order from the slot's m, which it moves on
//   mlstm_scan     the recurrence over the columns: S^T q and n . q of every row and head, from the slot's state, which it moves on
//   mlstm_finish   the division, the heads' RMS norm (no mean taken off), the weight and the sigmoid gate, for the output projection
//   mlstm_step     all three for a step of one row a sequence (a decode step), one launch
// Everything here is float32 but the projected q, k, v and the gate's pre-activation, which come in the activation type.
#include "common.h"

#define ML_BESIDE 4      // floats a row and head beside the read-out: a_t, b_t, m_t, n_t . q_t

// ---- the gates -------------------------------------------------------------------------------------------------
// A wave a (sequence, head), 64 rows at a time, a lane a row.  A step of the maximum is the map x -> max(x + f, i); two steps
// in a row are again such a map, (f1, i1) then (f2, i2) = (f1 + f2, max(i1 + f2, i2)), so the 64 maps are put together by a
// prefix over the lanes in six exchanges and every lane applies its own to the m the block started from.  The sums of f
// are added up in another order than one step after the other would; m only says by how much the state is scaled, and the
// factors a and b are made from the same m's that are stored, so the state times exp(m) does not feel it.
__global__ __launch_bounds__(BH_WAVE) void mlstm_gates_kernel(const float* __restrict__ pre, const float* __restrict__ bias, float cap,
                                                              float* __restrict__ state, long slot_stride, int head_floats,
                                                              const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                                              float* __restrict__ beside, int H) {
  const int seq = blockIdx.x / H, head = blockIdx.x % H, lane = threadIdx.x;
  const int row0 = seq_start[seq], rows = seq_start[seq + 1] - row0;
  float* m_at = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * head_floats + head_floats - 1;
  float m = *m_at;
  const float bias_i = bias ? bias[head] : 0.f, bias_f = bias ? bias[H + head] : 0.f, inv_cap = 1.0f / cap;
  for (int base = 0; base < rows; base += BH_WAVE) {
    const int t = base + lane;
    float gate_i = -INFINITY, gate_f = 0.f;      // a row beyond the end is the map that changes nothing
    if (t < rows) {
      const float* x = pre + (size_t)(row0 + t) * 2 * H;
      gate_i = cap * tanhf((x[head] + bias_i) * inv_cap);
      const float z = cap * tanhf((x[H + head] + bias_f) * inv_cap);
      gate_f = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));      // log(sigmoid(z)) without overflow
    }
    float sum_f = gate_f, top_i = gate_i;      // the map of rows base .. t put together
#pragma unroll
    for (int off = 1; off < BH_WAVE; off <<= 1) {
      const float f_before = __shfl_up(sum_f, off, BH_WAVE), i_before = __shfl_up(top_i, off, BH_WAVE);
      if (lane >= off) {
        top_i = fmaxf(i_before + sum_f, top_i);
        sum_f = f_before + sum_f;
      }
    }
    const float mine = fmaxf(m + sum_f, top_i);
    float before = __shfl_up(mine, 1, BH_WAVE);
    if (lane == 0) before = m;
    if (t < rows) {
      float* out = beside + ((size_t)(row0 + t) * H + head) * ML_BESIDE;
      out[0] = expf(gate_f + before - mine);
      out[1] = expf(gate_i - mine);
      out[2] = mine;
    }
    m = __shfl(mine, BH_WAVE - 1, BH_WAVE);
  }
  if (lane == 0 && rows > 0) *m_at = m;
}

// pre f32 [n_rows][2 H]: the input gates' pre-activations of the H heads, then the forget gates'; bias f32 [2 H] or null.
extern "C" int bh_mlstm_gates(const float* pre, const float* bias, float cap, float* state, long slot_stride, int head_floats,
                              const int32_t* seq_start, const int32_t* seq_slot, float* beside, int n_seqs, int H, hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && head_floats > 0 && cap > 0.f, "mlstm_gates: sizes and the cap must be positive");
  BH_REQUIRE((long)H * head_floats <= slot_stride, "mlstm_gates: %d heads of %d floats do not fit a slot's %ld", H, head_floats, slot_stride);
  mlstm_gates_kernel<<<n_seqs * H, BH_WAVE, 0, stream>>>(pre, bias, cap, state, slot_stride, head_floats, seq_start, seq_slot, beside, H);
  return bh_check_launch("mlstm_gates");
}

// ---- the recurrence --------------------------------------------------------------------------------------------
// A workgroup a (sequence, head, tile of 16 columns).  Thread (column c, slice s) keeps rows s R .. s R + R - 1 of column c in
// registers; the 16 slices of a column are neighbouring lanes.  16 rows of q, k (times b_t), the tile's values and the a_t go
// through LDS at a time, the next 16 asked for before these are walked (two stages in flight brought nothing and cost 70
// registers; a stage that asks every row whether it is there, so that a decode step walks one row and not sixteen, was
// slower on prompts and no faster in decode steps).  The walk over a stage's rows is unrolled and keeps
// every row's share of the read-out in a register; the 16 shares of 16 lanes are then added up crosswise in 15 exchanges
// (each lane ends with one row's sum, always in the same order), so no row waits for an exchange.
#define ML_COLS 16
#define ML_SLICES 16
#define ML_STAGE 16

// x of another lane of the same row of 16 lanes, by a data-parallel move: CTRL 0x140 the row mirrored (lane ^ 15), 0x141 its
// halves mirrored (lane ^ 7), 0x1B quads reversed (lane ^ 3), 0xB1 neighbours swapped (lane ^ 1).
template <int CTRL>
__device__ inline float lanes_moved(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}

// One exchange of the crosswise sum: acc[0 .. 2 SPAN) are the shares of 2 SPAN rows; the lane keeps the SPAN rows whose bit
// SPAN is its own, adds what its partner (CTRL) held of them, and leaves them in acc[0 .. SPAN).
template <int SPAN, int CTRL>
__device__ inline void hand_over(float (&acc)[ML_STAGE], int lane) {
  const bool upper = (lane & SPAN) != 0;
#pragma unroll
  for (int i = 0; i < SPAN; ++i) {
    const float give = upper ? acc[i] : acc[i + SPAN], keep = upper ? acc[i + SPAN] : acc[i];
    acc[i] = keep + lanes_moved<CTRL>(give);
  }
}

template <typename T, int R>
__global__ __launch_bounds__(ML_COLS * ML_SLICES) void mlstm_scan_kernel(
    const T* __restrict__ proj, int row_stride, int q_off, int k_off, int v_off, const float* beside_in,
    float* __restrict__ state, long slot_stride, const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
    float* __restrict__ read, float* beside, int H, int dim, int vdim, int tiles, float q_scale) {
  constexpr int DIM = ML_SLICES * R;      // the rows of a column that the registers hold (dim <= DIM)
  __shared__ __attribute__((aligned(16))) float s_q[ML_STAGE][DIM];
  __shared__ __attribute__((aligned(16))) float s_k[ML_STAGE][DIM];    // times b_t already
  __shared__ float s_v[ML_STAGE][ML_COLS];
  __shared__ float s_a[ML_STAGE];
  const int tile = blockIdx.x % tiles, unit = blockIdx.x / tiles;
  const int head = unit % H, seq = unit / H;
  const int row0 = seq_start[seq], rows = seq_start[seq + 1] - row0;
  if (rows <= 0) return;
  const int tid = threadIdx.x, c = tid / ML_SLICES, s = tid % ML_SLICES;
  const int column = tile * ML_COLS + c;      // vdim is n's
  const int head_floats = (vdim + 1) * dim + 1;
  float* mine = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * head_floats + (size_t)column * dim;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = s * R + r;
    S[r] = (column <= vdim && d < dim) ? mine[d] : 0.f;
  }
  // what this thread brings into a stage: row `c` of it, dimensions s R + r of q and k; the tile's value (c, s as row, column)
  float next_q[R], next_k[R], next_v = 0.f, next_a = 1.f, next_b = 0.f;
  auto ask = [&](int base) {
    const int t = base + c;
    const bool live = t < rows;
    const T* x = proj + (size_t)(row0 + (live ? t : 0)) * row_stride + (size_t)head * dim;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = s * R + r;
      const bool there = live && d < dim;
      next_q[r] = there ? to_f32(x[q_off + d]) : 0.f;
      next_k[r] = there ? to_f32(x[k_off + d]) : 0.f;
    }
    const float* g = beside_in + ((size_t)(row0 + (live ? t : 0)) * H + head) * ML_BESIDE;
    next_a = live ? g[0] : 1.f;
    next_b = live ? g[1] : 0.f;
    const int value = tile * ML_COLS + s;
    next_v = 0.f;
    if (live && value < vdim) next_v = to_f32(proj[(size_t)(row0 + t) * row_stride + v_off + (size_t)head * vdim + value]);
    else if (live && value == vdim) next_v = 1.f;
  };
  ask(0);
  for (int base = 0; base < rows; base += ML_STAGE) {
    __syncthreads();      // the stage before has been walked by all
#pragma unroll
    for (int r = 0; r < R; ++r) {
      s_q[c][s * R + r] = next_q[r] * q_scale;
      s_k[c][s * R + r] = next_k[r] * next_b;
    }
    s_v[c][s] = next_v;
    if (s == 0) s_a[c] = next_a;
    __syncthreads();
    if (base + ML_STAGE < rows) ask(base + ML_STAGE);
    // (rows beyond the end stand in LDS as a = 1, k = 0: they change nothing and their sums are not stored)
    float acc[ML_STAGE];
#pragma unroll
    for (int t = 0; t < ML_STAGE; ++t) {
      const float a = s_a[t], v = s_v[t][c];
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        S[r] = fmaf(a, S[r], s_k[t][s * R + r] * v);
        sum = fmaf(S[r], s_q[t][s * R + r], sum);
      }
      acc[t] = sum;
    }
    // Lane s of a column's 16 ends with row s's sum.  Four exchanges with the lane whose number differs in all four bits, in
    // the lower three, two and one (a row of 16 lanes mirrored, its halves mirrored, quads reversed, neighbours swapped: the
    // data-parallel moves of the vector unit): each time a lane keeps the rows whose bit is its own and hands over the
    // others' shares.  (Written out by templates: a loop over the spans is not unrolled, its registers are then found by
    // number at run time, and that took more time than everything else in this kernel.)
    hand_over<8, 0x140>(acc, s);
    hand_over<4, 0x141>(acc, s);
    hand_over<2, 0x1B>(acc, s);
    hand_over<1, 0xB1>(acc, s);
    if (base + s < rows) {
      const size_t row = (size_t)(row0 + base + s);
      if (column < vdim) read[row * H * vdim + (size_t)head * vdim + column] = acc[0];
      else if (column == vdim) beside[(row * H + head) * ML_BESIDE + 3] = acc[0];
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = s * R + r;
    if (column <= vdim && d < dim) mine[d] = S[r];
  }
}

// proj [n_rows][row_stride] holds a row's q and k (H heads of dim) and v (H heads of vdim) from q_off, k_off, v_off; beside
// f32 [n_rows][H][4] as mlstm_gates left it (its fourth number, n . q, is written here); read f32 [n_rows][H * vdim].
extern "C" int bh_mlstm_scan(const void* proj, int dtype, int row_stride, int q_off, int k_off, int v_off, float* beside, float* state,
                             long slot_stride, const int32_t* seq_start, const int32_t* seq_slot, float* read, int n_seqs, int H, int dim,
                             int vdim, hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && dim > 0 && vdim > 0, "mlstm_scan: sizes must be positive");
  BH_REQUIRE(dim <= ML_SLICES * 32, "mlstm_scan: heads of %d key dimensions are above the limit of %d", dim, ML_SLICES * 32);
  BH_REQUIRE((long)H * ((long)(vdim + 1) * dim + 1) <= slot_stride, "mlstm_scan: %d heads of %d x %d do not fit a slot's %ld floats", H, dim,
             vdim, slot_stride);
  BH_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + H * dim <= row_stride && k_off + H * dim <= row_stride &&
                 v_off + H * vdim <= row_stride, "mlstm_scan: q, k and v lie outside a row of %d", row_stride);
  const int tiles = (vdim + 1 + ML_COLS - 1) / ML_COLS;
  BH_REQUIRE((long)n_seqs * H * tiles < (1L << 31), "mlstm_scan: too many workgroups");
  const float q_scale = 1.0f / sqrtf((float)dim);
  const int per = (dim + ML_SLICES - 1) / ML_SLICES;
#define BH_ML(T, R)                                                                                                              \
  mlstm_scan_kernel<T, R><<<n_seqs * H * tiles, ML_COLS * ML_SLICES, 0, stream>>>((const T*)proj, row_stride, q_off, k_off, v_off, beside, \
                                                                               state, slot_stride, seq_start, seq_slot, read, beside, H, \
                                                                               dim, vdim, tiles, q_scale)
#define BH_ML_SIZES(T)              \
  do {                              \
    if (per <= 1) BH_ML(T, 1);      \
    else if (per <= 2) BH_ML(T, 2); \
    else if (per <= 4) BH_ML(T, 4); \
    else if (per <= 8) BH_ML(T, 8); \
    else if (per <= 16) BH_ML(T, 16); \
    else BH_ML(T, 32);              \
  } while (0)
  if (dtype == BH_F32) BH_ML_SIZES(float);
  else if (dtype == BH_BF16) BH_ML_SIZES(bf16_t);
  else return bh_fail("mlstm_scan: unknown dtype %d", dtype);
#undef BH_ML_SIZES
#undef BH_ML
  return bh_check_launch("mlstm_scan");
}

// ---- the read-out: division, norm of each head, weight, gate ----------------------------------------------------------
// A wave a (row, head).
template <typename T>
__global__ __launch_bounds__(256) void mlstm_finish_kernel(const float* __restrict__ read, const float* __restrict__ beside,
                                                           const T* __restrict__ gate, int gate_stride, int gate_first,
                                                           const float* __restrict__ w, float eps, T* __restrict__ out, int n_rows, int H,
                                                           int vdim, int out_block_rows) {
  const int unit = blockIdx.x * (blockDim.x / BH_WAVE) + threadIdx.x / BH_WAVE, lane = threadIdx.x % BH_WAVE;
  if (unit >= n_rows * H) return;
  const int row = unit / H, head = unit % H;
  const float* b = beside + (size_t)unit * ML_BESIDE;
  const float inv = 1.0f / (fmaxf(fabsf(b[3]), expf(-b[2])) + 1e-6f);
  const float* o = read + (size_t)row * H * vdim + (size_t)head * vdim;
  float ss = 0.f;
  for (int e = lane; e < vdim; e += BH_WAVE) {
    const float v = o[e] * inv;
    ss += v * v;
  }
  const float norm = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  for (int e = lane; e < vdim; e += BH_WAVE) {
    const int column = head * vdim + e;
    const float g = to_f32(gate[(size_t)row * gate_stride + gate_first + column]);
    const float y = o[e] * inv * norm * (w ? w[column] : 1.f) / (1.0f + expf(-g));
    out[bh_rows_index(out_block_rows, row, column, H * vdim)] = from_f32<T>(y);
  }
}

extern "C" int bh_mlstm_finish(const float* read, const float* beside, const void* gate, int dtype, int gate_stride, int gate_first,
                               const float* w, float eps, void* out, int n_rows, int H, int vdim, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && vdim > 0, "mlstm_finish: sizes must be positive");
  BH_REQUIRE(gate_first >= 0 && gate_first + H * vdim <= gate_stride, "mlstm_finish: the gate lies outside its row");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && (H * vdim) % 32 == 0 && dtype == BH_BF16),
             "mlstm_finish: rows in blocks of %d of width %d are not written", out_block_rows, H * vdim);
  const long units = (long)n_rows * H;
  BH_REQUIRE((units + 3) / 4 < (1L << 31), "mlstm_finish: too many rows");
  const int blocks = (int)((units + 3) / 4);
  if (dtype == BH_F32)
    mlstm_finish_kernel<float><<<blocks, 256, 0, stream>>>(read, beside, (const float*)gate, gate_stride, gate_first, w, eps, (float*)out,
                                                         n_rows, H, vdim, out_block_rows);
  else if (dtype == BH_BF16)
    mlstm_finish_kernel<bf16_t><<<blocks, 256, 0, stream>>>(read, beside, (const bf16_t*)gate, gate_stride, gate_first, w, eps,
                                                          (bf16_t*)out, n_rows, H, vdim, out_block_rows);
  else
    return bh_fail("mlstm_finish: unknown dtype %d", dtype);
  return bh_check_launch("mlstm_finish");
}

// ---- a decode step: gates, one step of the recurrence and the read-out in one launch ------------------------------------
// A workgroup a (sequence, head); the sequence brings one row.  Every thread makes the gates' numbers for itself (a handful of
// operations), q and b k stand in LDS, the columns are walked 16 at a time by the scan's threads (column c, slice s), each
// column's read-out is added up across its 16 lanes and left in LDS, and the workgroup then divides, norms and gates its head.
template <typename T, int R>
__global__ __launch_bounds__(ML_COLS * ML_SLICES) void mlstm_step_kernel(
    const T* __restrict__ proj, int row_stride, int q_off, int k_off, int v_off, int g_off, const float* __restrict__ pre,
    const float* __restrict__ bias, float cap, float* __restrict__ state, long slot_stride, const int32_t* __restrict__ seq_slot,
    const float* __restrict__ w, float eps, T* __restrict__ out, int H, int dim, int vdim, float q_scale, int out_block_rows) {
  constexpr int DIM = ML_SLICES * R;
  extern __shared__ float s_o[];      // vdim + 1 read-outs: the values' columns, then n . q
  __shared__ float s_q[DIM];
  __shared__ float s_k[DIM];
  __shared__ float scratch[ML_COLS * ML_SLICES / BH_WAVE];
  const int seq = blockIdx.x / H, head = blockIdx.x % H, row = seq;
  const int tid = threadIdx.x, c = tid / ML_SLICES, s = tid % ML_SLICES;
  const int head_floats = (vdim + 1) * dim + 1;
  float* held = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * head_floats;
  const T* x = proj + (size_t)row * row_stride;
  // the gates (mlstm_gates_kernel's numbers for one row)
  const float inv_cap = 1.0f / cap;
  const float* gate_in = pre + (size_t)row * 2 * H;
  const float gate_i = cap * tanhf((gate_in[head] + (bias ? bias[head] : 0.f)) * inv_cap);
  const float z = cap * tanhf((gate_in[H + head] + (bias ? bias[H + head] : 0.f)) * inv_cap);
  const float gate_f = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
  const float m_before = held[head_floats - 1];
  const float m = fmaxf(gate_f + m_before, gate_i);
  const float a = expf(gate_f + m_before - m), b = expf(gate_i - m);
  for (int d = tid; d < DIM; d += blockDim.x) {
    s_q[d] = d < dim ? to_f32(x[q_off + head * dim + d]) * q_scale : 0.f;
    s_k[d] = d < dim ? to_f32(x[k_off + head * dim + d]) * b : 0.f;
  }
  __syncthreads();
  for (int first = 0; first <= vdim; first += ML_COLS) {
    const int column = first + c;
    float* mine = held + (size_t)column * dim;
    const float v = column < vdim ? to_f32(x[v_off + head * vdim + column]) : 1.f;
    float sum = 0.f;
    if (column <= vdim) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int d = s * R + r;
        if (d < dim) {
          const float now = fmaf(a, mine[d], s_k[d] * v);
          mine[d] = now;
          sum = fmaf(now, s_q[d], sum);
        }
      }
    }
    sum += lanes_moved<0x140>(sum);      // across the column's 16 lanes: every lane ends with the whole
    sum += lanes_moved<0x141>(sum);
    sum += lanes_moved<0x1B>(sum);
    sum += lanes_moved<0xB1>(sum);
    if (s == 0 && column <= vdim) s_o[column] = sum;
  }
  __syncthreads();
  if (tid == 0) held[head_floats - 1] = m;
  const float under = 1.0f / (fmaxf(fabsf(s_o[vdim]), expf(-m)) + 1e-6f);
  float ss = 0.f;
  for (int e = tid; e < vdim; e += blockDim.x) {
    const float o = s_o[e] * under;
    ss += o * o;
  }
  const float norm = 1.0f / sqrtf(block_sum(ss, scratch) / (float)vdim + eps);
  for (int e = tid; e < vdim; e += blockDim.x) {
    const int at = head * vdim + e;
    const float g = to_f32(x[g_off + at]);
    const float y = s_o[e] * under * norm * (w ? w[at] : 1.f) / (1.0f + expf(-g));
    out[bh_rows_index(out_block_rows, row, at, H * vdim)] = from_f32<T>(y);
  }
}

// A step in which sequence b brings the one row b: proj, pre, bias as for mlstm_gates and mlstm_scan, w and out as for
// mlstm_finish; the slots' states are moved on.
extern "C" int bh_mlstm_step(const void* proj, int dtype, int row_stride, int q_off, int k_off, int v_off, int g_off, const float* pre,
                             const float* bias, float cap, float* state, long slot_stride, const int32_t* seq_slot, const float* w,
                             float eps, void* out, int n_seqs, int H, int dim, int vdim, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && dim > 0 && vdim > 0 && cap > 0.f, "mlstm_step: sizes and the cap must be positive");
  BH_REQUIRE(dim <= ML_SLICES * 32, "mlstm_step: heads of %d key dimensions are above the limit of %d", dim, ML_SLICES * 32);
  BH_REQUIRE((long)H * ((long)(vdim + 1) * dim + 1) <= slot_stride, "mlstm_step: %d heads of %d x %d do not fit a slot's %ld floats", H, dim,
             vdim, slot_stride);
  BH_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && g_off >= 0 && q_off + H * dim <= row_stride && k_off + H * dim <= row_stride &&
                 v_off + H * vdim <= row_stride && g_off + H * vdim <= row_stride, "mlstm_step: q, k, v and the gate lie outside a row of %d", row_stride);
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && (H * vdim) % 32 == 0 && dtype == BH_BF16),
             "mlstm_step: rows in blocks of %d of width %d are not written", out_block_rows, H * vdim);
  const size_t lds = (size_t)(vdim + 1) * sizeof(float);
  BH_REQUIRE(lds <= 32 * 1024, "mlstm_step: heads of %d values do not fit the local memory", vdim);
  BH_REQUIRE((long)n_seqs * H < (1L << 31), "mlstm_step: too many workgroups");
  const float q_scale = 1.0f / sqrtf((float)dim);
  const int per = (dim + ML_SLICES - 1) / ML_SLICES;
#define BH_MS(T, R)                                                                                                                 \
  mlstm_step_kernel<T, R><<<n_seqs * H, ML_COLS * ML_SLICES, lds, stream>>>((const T*)proj, row_stride, q_off, k_off, v_off, g_off, pre, \
                                                                          bias, cap, state, slot_stride, seq_slot, w, eps, (T*)out, H, \
                                                                          dim, vdim, q_scale, out_block_rows)
#define BH_MS_SIZES(T)              \
  do {                              \
    if (per <= 1) BH_MS(T, 1);      \
    else if (per <= 2) BH_MS(T, 2); \
    else if (per <= 4) BH_MS(T, 4); \
    else if (per <= 8) BH_MS(T, 8); \
    else if (per <= 16) BH_MS(T, 16); \
    else BH_MS(T, 32);              \
  } while (0)
  if (dtype == BH_F32) BH_MS_SIZES(float);
  else if (dtype == BH_BF16) BH_MS_SIZES(bf16_t);
  else return bh_fail("mlstm_step: unknown dtype %d", dtype);
#undef BH_MS_SIZES
#undef BH_MS
  return bh_check_launch("mlstm_step");
}
