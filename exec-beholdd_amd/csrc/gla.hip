// Gated linear attention: a matrix state per (sequence, head) whose rows decay each by a factor of its own that the
// token sets,
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   alpha_t = sigmoid(z_t + b)^(1/tau)   (one per key channel)
//   gla_scan   walks a sequence's rows of the step in order from the state that the sequence's slot holds and leaves the
//              state after the last row there; prompts, portions of prompts and decode steps are the same walk.
// S is [dim][vdim] float32.  Decays (through the logarithm of the sigmoid, so that 1/tau is a factor), the state, both
// products and the read-out are float32; only q, k and v are read in the activations' type.
#include "common.h"

#define GLA_STAGE 16      // rows that go through LDS at a time

// A barrier between the waves of a workgroup that orders their LDS traffic only: a wave waits for its own LDS operations,
// not for the global loads it has in flight (__syncthreads waits for those too, which would end every read-ahead at the
// next barrier; here the next stage's loads stay on their way across the barriers of this stage).
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ inline float log_sigmoid_f32(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// A workgroup takes a (sequence, head, tile of VT value columns).  Thread (column, slice) keeps rows slice * R .. + R - 1 of its
// column of S in registers.  GLA_STAGE rows' decays, keys, queries (LDS rows of SL * R floats, zeros beyond dim) and the tile's
// values are staged at a time; a row's shares of o are added over a wave's slices by lane exchanges and over the waves through
// LDS, in a fixed order.  The next stage's numbers are asked for (into registers, GLA_AHEAD elements a thread and array; what a
// stage has beyond that is read when it is staged) before this stage's rows are walked, so that the walk hides their way from
// memory.
#define GLA_AHEAD 4
#define GLA_GROUP 4
#define GLA_KEPT 8        // key channels a thread keeps a product of decays for: heads of up to 2,048 key dimensions

// Long sequences in chunks of `rows` rows (0: whole sequences), `count` chunks for the longest; scratch memory for a chunk's last
// state [n_seqs][count][H][dim][vdim], its decays' product [n_seqs][count][H][dim] and a row's decayed query [rows][H][dim].
struct GlaChunks {
  int rows, count;
  float* states;
  float* decays;
  float* queries;
};

template <typename T, int R>
__global__ __launch_bounds__(256) void gla_scan_kernel(const T* __restrict__ proj, int proj_stride, int q_off, int k_off, int v_off,
                                                       const float* __restrict__ z, int z_stride, const float* __restrict__ bias,
                                                       float inv_tau, float q_scale, float* __restrict__ state, long slot_stride,
                                                       const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                                       float* __restrict__ out, int H, int dim, int vdim, int VT, GlaChunks chunks) {
  extern __shared__ __align__(16) float lds[];
  const int SL = 256 / VT, DP = SL * R;      // VT and R are powers of two, so are SL and DP: shifts and masks below
  const int dp_shift = __builtin_ctz(DP), vt_shift = __builtin_ctz(VT);
  float* a_s = lds;                          // [GLA_STAGE][DP]
  float* k_s = a_s + GLA_STAGE * DP;
  float* q_s = k_s + GLA_STAGE * DP;
  float* v_s = q_s + GLA_STAGE * DP;         // [GLA_STAGE][VT]
  float* part = v_s + GLA_STAGE * VT;        // [GLA_STAGE][PARTS][VT]: a wave's slices' shares added up (VT < 64), or a slice's own
  const int PARTS = VT >= BH_WAVE ? SL : 256 / BH_WAVE;
  const int seq = blockIdx.x / chunks.count, chunk = blockIdx.x % chunks.count, head = blockIdx.y, v0 = blockIdx.z * VT;
  const int col = threadIdx.x & (VT - 1), slice = threadIdx.x >> vt_shift, d0 = slice * R;
  const bool has_column = v0 + col < vdim;
  // A sequence of more than chunks.rows rows is walked in chunks side by side: the first from the slot's state, the others
  // from nothing; a chunk leaves its last state, the product of its decays and, row by row, its queries times the decays up
  // to that row, from which gla_combine and gla_carry make up what the later chunks' rows owe the state they started from.
  const int seq_first = seq_start[seq], seq_stop = seq_start[seq + 1];
  const int in_chunks = chunks.rows > 0 ? (seq_stop - seq_first + chunks.rows - 1) / chunks.rows : 1;      // chunks this sequence has
  const int start = seq_first + chunk * chunks.rows;
  const int stop = (chunks.rows > 0 && start + chunks.rows < seq_stop) ? start + chunks.rows : seq_stop;
  if (chunk > 0 && chunk >= in_chunks) return;      // a shorter sequence has fewer chunks
  const bool apart = in_chunks > 1;
  float* mine = apart ? chunks.states + ((size_t)(seq * chunks.count + chunk) * H + head) * dim * vdim + v0 + col
                      : state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * dim * vdim + v0 + col;
  const float* from = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * dim * vdim + v0 + col;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = (chunk == 0 && has_column && d0 + r < dim) ? from[(size_t)(d0 + r) * vdim] : 0.f;
  float kept[GLA_KEPT];      // the decays' products so far, of key channels threadIdx.x, + 256, ... (first tile's workgroup only)
#pragma unroll
  for (int j = 0; j < GLA_KEPT; ++j) kept[j] = 1.0f;
  const bool keeps = apart && blockIdx.z == 0;
  const int width = H * vdim;
  float ahead_z[GLA_AHEAD], ahead_k[GLA_AHEAD], ahead_q[GLA_AHEAD], ahead_v[GLA_AHEAD];
  // a stage's element e of the decays, keys and queries is (row e / DP, key channel e % DP); of the values (row e / VT, column e % VT)
  auto ask = [&](int row0, int n) {
#pragma unroll
    for (int i = 0; i < GLA_AHEAD; ++i) {
      const int e = threadIdx.x + 256 * i, t = e >> dp_shift, d = e & (DP - 1);
      ahead_z[i] = ahead_k[i] = ahead_q[i] = ahead_v[i] = 0.f;
      if (e < n * DP && d < dim) {
        const T* x = proj + (size_t)(row0 + t) * proj_stride + head * dim + d;
        ahead_z[i] = z[(size_t)(row0 + t) * z_stride + head * dim + d] + bias[head * dim + d];
        ahead_k[i] = to_f32(x[k_off]);
        ahead_q[i] = to_f32(x[q_off]);
      }
      const int tv = e >> vt_shift, c = e & (VT - 1);
      if (e < n * VT && v0 + c < vdim) ahead_v[i] = to_f32(proj[(size_t)(row0 + tv) * proj_stride + v_off + head * vdim + v0 + c]);
    }
  };
  if (start < stop) ask(start, stop - start < GLA_STAGE ? stop - start : GLA_STAGE);
  for (int row0 = start; row0 < stop; row0 += GLA_STAGE) {
    const int n = stop - row0 < GLA_STAGE ? stop - row0 : GLA_STAGE;
#pragma unroll
    for (int i = 0; i < GLA_AHEAD; ++i) {
      const int e = threadIdx.x + 256 * i;
      if (e < n * DP) {
        const bool real = (e & (DP - 1)) < dim;
        a_s[e] = real ? expf(log_sigmoid_f32(ahead_z[i]) * inv_tau) : 0.f;
        k_s[e] = ahead_k[i];
        q_s[e] = ahead_q[i] * q_scale;
      }
      if (e < n * VT) v_s[e] = ahead_v[i];
    }
    for (int e = threadIdx.x + 256 * GLA_AHEAD; e < n * DP; e += 256) {      // wide heads: what the registers did not hold
      const int t = e >> dp_shift, d = e & (DP - 1);
      float a = 0.f, kk = 0.f, qq = 0.f;
      if (d < dim) {
        const T* x = proj + (size_t)(row0 + t) * proj_stride + head * dim + d;
        a = expf(log_sigmoid_f32(z[(size_t)(row0 + t) * z_stride + head * dim + d] + bias[head * dim + d]) * inv_tau);
        kk = to_f32(x[k_off]);
        qq = to_f32(x[q_off]) * q_scale;
      }
      a_s[e] = a;
      k_s[e] = kk;
      q_s[e] = qq;
    }
    lds_barrier();
    if (row0 + GLA_STAGE < stop) ask(row0 + GLA_STAGE, stop - row0 - GLA_STAGE < GLA_STAGE ? stop - row0 - GLA_STAGE : GLA_STAGE);
    if (keeps) {
#pragma unroll
      for (int j = 0; j < GLA_KEPT; ++j) {
        const int d = threadIdx.x + 256 * j;
        if (d >= dim) break;
        for (int t = 0; t < n; ++t) {
          kept[j] *= a_s[t * DP + d];
          if (chunk > 0) chunks.queries[(size_t)(row0 + t) * H * dim + head * dim + d] = kept[j] * q_s[t * DP + d];
        }
      }
    }
    // GLA_GROUP rows at a time: their operands are read from LDS with no store in between (the compiler may ask for all of
    // them at once), the slices of a wave add their shares up by lane exchanges, and one lane a column and wave stores them
#pragma unroll 1
    for (int t0 = 0; t0 < n; t0 += GLA_GROUP) {
      float acc[GLA_GROUP];
#pragma unroll
      for (int j = 0; j < GLA_GROUP; ++j) {
        const int t = t0 + j < n ? t0 + j : n - 1;      // a row beyond the last is walked on a copy of the state and dropped
        const float vv = v_s[t * VT + col];
        const float* a_row = a_s + t * DP + d0;
        const float* k_row = k_s + t * DP + d0;
        const float* q_row = q_s + t * DP + d0;
        const bool real = t0 + j < n;
        float sum = 0.f;
        if (R % 4 == 0) {
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            const float4 a4 = *reinterpret_cast<const float4*>(a_row + r), k4 = *reinterpret_cast<const float4*>(k_row + r),
                         q4 = *reinterpret_cast<const float4*>(q_row + r);
            const float s0 = fmaf(a4.x, S[r], k4.x * vv), s1 = fmaf(a4.y, S[r + 1], k4.y * vv);
            const float s2 = fmaf(a4.z, S[r + 2], k4.z * vv), s3 = fmaf(a4.w, S[r + 3], k4.w * vv);
            sum = fmaf(s0, q4.x, sum);
            sum = fmaf(s1, q4.y, sum);
            sum = fmaf(s2, q4.z, sum);
            sum = fmaf(s3, q4.w, sum);
            if (real) S[r] = s0, S[r + 1] = s1, S[r + 2] = s2, S[r + 3] = s3;
          }
        } else {
#pragma unroll
          for (int r = 0; r < R; ++r) {
            const float s0 = fmaf(a_row[r], S[r], k_row[r] * vv);
            sum = fmaf(s0, q_row[r], sum);
            if (real) S[r] = s0;
          }
        }
        acc[j] = sum;
      }
      for (int off = VT; off < BH_WAVE; off <<= 1) {
#pragma unroll
        for (int j = 0; j < GLA_GROUP; ++j) acc[j] += __shfl_xor(acc[j], off, BH_WAVE);
      }
      if ((threadIdx.x % BH_WAVE) < VT || VT >= BH_WAVE) {
        const int share = VT >= BH_WAVE ? slice : threadIdx.x / BH_WAVE;
#pragma unroll
        for (int j = 0; j < GLA_GROUP; ++j)
          if (t0 + j < n) part[((t0 + j) * PARTS + share) * VT + col] = acc[j];
      }
    }
    lds_barrier();
    for (int e = threadIdx.x; e < n * VT; e += 256) {
      const int t = e >> vt_shift, c = e & (VT - 1);
      if (v0 + c >= vdim) continue;
      float total = 0.f;
      for (int s = 0; s < PARTS; ++s) total += part[(t * PARTS + s) * VT + c];
      out[(size_t)(row0 + t) * width + head * vdim + v0 + c] = total;
    }
    lds_barrier();      // the stage's LDS is written again
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (has_column && d0 + r < dim) mine[(size_t)(d0 + r) * vdim] = S[r];
  if (keeps) {
#pragma unroll
    for (int j = 0; j < GLA_KEPT; ++j) {
      const int d = threadIdx.x + 256 * j;
      if (d < dim) chunks.decays[((size_t)(seq * chunks.count + chunk) * H + head) * dim + d] = kept[j];
    }
  }
}

// One thread a state element (sequence, head, key channel, value column): through the sequence's chunks in order,
// S_in(c + 1) = A(c) S_in(c) + S_loc(c), A(c) the chunk's product of decays; a chunk's place in `states` then holds the state
// it started from (for gla_carry), and the state after the last chunk goes to the sequence's slot.
__global__ __launch_bounds__(256) void gla_combine_kernel(GlaChunks chunks, float* __restrict__ state, long slot_stride,
                                                          const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot, int H,
                                                          int dim, int vdim) {
  const int seq = blockIdx.y;
  const size_t per = (size_t)H * dim * vdim, e = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= per) return;
  const int in_chunks = (seq_start[seq + 1] - seq_start[seq] + chunks.rows - 1) / chunks.rows;
  if (in_chunks <= 1) return;      // the walk itself wrote the slot
  const size_t channel = e / vdim;      // (head, key channel)
  float run = 0.f;
  for (int c = 0; c < in_chunks; ++c) {
    float* place = chunks.states + (size_t)(seq * chunks.count + c) * per + e;
    const float local = *place;
    *place = run;
    run = c == 0 ? local : fmaf(chunks.decays[(size_t)(seq * chunks.count + c) * H * dim + channel], run, local);
  }
  state[(size_t)seq_slot[seq] * slot_stride + e] = run;
}

// out[row] += (decayed query of the row) . S_in(the row's chunk), for the rows of every chunk but a sequence's first: a workgroup
// takes a (sequence, chunk, head, 64 value columns); thread (column, row group) keeps 16 rows' sums, 64 key channels of the
// state's tile and of 64 rows' queries go through LDS at a time.
__global__ __launch_bounds__(256) void gla_carry_kernel(GlaChunks chunks, const int32_t* __restrict__ seq_start, float* __restrict__ out, int H,
                                                        int dim, int vdim) {
  __shared__ float s_tile[64][64 + 1];      // [key channel][column]
  __shared__ float b_tile[64][64];          // [row][key channel]
  const int seq = blockIdx.x / chunks.count, chunk = blockIdx.x % chunks.count, head = blockIdx.y, v0 = blockIdx.z * 64;
  if (chunk == 0) return;
  const int first = seq_start[seq] + chunk * chunks.rows, seq_stop = seq_start[seq + 1];
  if (first >= seq_stop) return;
  const int stop = first + chunks.rows < seq_stop ? first + chunks.rows : seq_stop;
  const int col = threadIdx.x & 63, group = threadIdx.x >> 6;
  const float* began = chunks.states + ((size_t)(seq * chunks.count + chunk) * H + head) * dim * vdim;
  for (int row0 = first; row0 < stop; row0 += 64) {
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    for (int dd = 0; dd < dim; dd += 64) {
      __syncthreads();      // the tiles are written again
      for (int e = threadIdx.x; e < 64 * 64; e += 256) {
        const int a = e >> 6, b = e & 63;      // a tile's (row, column): neighbours in memory are neighbouring threads
        s_tile[a][b] = (dd + a < dim && v0 + b < vdim) ? began[(size_t)(dd + a) * vdim + v0 + b] : 0.f;
        b_tile[a][b] = (row0 + a < stop && dd + b < dim) ? chunks.queries[(size_t)(row0 + a) * H * dim + head * dim + dd + b] : 0.f;
      }
      __syncthreads();
#pragma unroll 4
      for (int d = 0; d < 64; ++d) {
        const float s = s_tile[d][col];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = fmaf(b_tile[group * 16 + i][d], s, acc[i]);
      }
    }
    if (v0 + col < vdim) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = row0 + group * 16 + i;
        if (row < stop) out[(size_t)row * H * vdim + head * vdim + v0 + col] += acc[i];
      }
    }
  }
}

// How many value columns a workgroup takes for a step of these sizes.  A stage costs a workgroup about as many instructions
// whatever its tile (the staging of decays, keys and queries is the same for every tile of a head), so narrow tiles multiply
// the work: they pay only while they bring idle compute units in, up to about one workgroup a unit; and never so narrow that
// a thread's slice of a state column exceeds 64 rows.
static int gla_tile(long walks, int H, int dim, int vdim) {
  int tile = 64;
  while (tile > 8 && (tile / 2 >= vdim || walks * H * ((vdim + tile - 1) / tile) < (long)bh_compute_units())) tile /= 2;
  while (tile > 8 && (dim + 256 / tile - 1) / (256 / tile) > 64) tile /= 2;
  return tile;
}

// Rows of a chunk for a step whose longest sequence brings max_rows rows: a walk over a sequence is a chain of stages that one
// workgroup runs at one wave a SIMD, so long sequences are cut until about four workgroups stand on every compute unit, in
// chunks of whole stages and no fewer than 64 rows; max_rows and more: the sequences are walked whole.
extern "C" int bh_gla_chunk_rows(int n_seqs, int max_rows, int H, int dim, int vdim) {
  if (max_rows < 128 || dim > 256 * GLA_KEPT) return max_rows;
  const long whole = (long)n_seqs * H * ((vdim + 63) / 64);
  long wanted = (4L * bh_compute_units() + whole - 1) / whole;
  if (wanted <= 1) return max_rows;
  if (wanted > max_rows / 64) wanted = max_rows / 64;
  int rows = (int)((max_rows + wanted - 1) / wanted);
  rows = (rows + GLA_STAGE - 1) / GLA_STAGE * GLA_STAGE;
  return rows >= max_rows ? max_rows : rows;
}

// proj [rows][proj_stride] (dtype): a row holds H heads of q and of k (dim each) from q_off and k_off and H heads of v (vdim) from
// v_off.  z [rows][z_stride] float32: the decays' pre-activations, H x dim from column 0; bias [H * dim] float32.
// state [slots][slot_stride] float32, a slot's first H * dim * vdim floats being its heads' states; seq_start [n_seqs + 1],
// seq_slot [n_seqs]; out [rows][H * vdim] float32.  chunk_rows: bh_gla_chunk_rows' answer for the step (max_rows: its longest
// sequence's rows); where that is less than max_rows, scratch holds n_seqs * chunks * H * dim * (vdim + 1) + n_rows * H * dim floats.
extern "C" int bh_gla_scan(const void* proj, int dtype, int proj_stride, int q_off, int k_off, int v_off, const float* z, int z_stride,
                           const float* bias, float tau, float q_scale, float* state, long slot_stride, const int32_t* seq_start,
                           const int32_t* seq_slot, float* out, int n_seqs, int H, int dim, int vdim, int n_rows, int max_rows,
                           int chunk_rows, float* scratch, hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && dim > 0 && vdim > 0, "gla_scan: sizes must be positive");
  BH_REQUIRE(tau > 0.f, "gla_scan: tau must be positive, got %f", (double)tau);
  BH_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + H * dim <= proj_stride && k_off + H * dim <= proj_stride &&
                 v_off + H * vdim <= proj_stride, "gla_scan: q, k or v lie outside a row of %d", proj_stride);
  BH_REQUIRE(z_stride >= H * dim, "gla_scan: the decays' rows hold %d numbers, %d are needed", z_stride, H * dim);
  BH_REQUIRE(slot_stride >= (long)H * dim * vdim, "gla_scan: a slot's state is smaller than the heads' states");
  BH_REQUIRE(H <= 65535 && (vdim + 7) / 8 <= 65535, "gla_scan: too many heads or value columns");
  BH_REQUIRE(max_rows > 0 && n_rows >= n_seqs && chunk_rows > 0, "gla_scan: a step has rows, and chunks have rows");
  GlaChunks chunks = {0, 1, nullptr, nullptr, nullptr};
  if (chunk_rows < max_rows) {
    BH_REQUIRE(scratch != nullptr && chunk_rows % GLA_STAGE == 0 && dim <= 256 * GLA_KEPT, "gla_scan: chunks need scratch memory and whole stages");
    chunks.rows = chunk_rows;
    chunks.count = (max_rows + chunk_rows - 1) / chunk_rows;
    chunks.states = scratch;
    chunks.decays = chunks.states + (size_t)n_seqs * chunks.count * H * dim * vdim;
    chunks.queries = chunks.decays + (size_t)n_seqs * chunks.count * H * dim;
  }
  BH_REQUIRE((long)n_seqs * chunks.count < (1L << 31), "gla_scan: too many chunks");
  const int VT = gla_tile((long)n_seqs * chunks.count, H, dim, vdim), SL = 256 / VT;
  int R = 1;
  while (R * SL < dim) R *= 2;
  BH_REQUIRE(R <= 64, "gla_scan: heads of %d key dimensions are above the limit of %d", dim, 64 * 32);
  const size_t lds = (size_t)GLA_STAGE * (3 * SL * R + VT + 256) * sizeof(float);
  BH_REQUIRE(lds <= 160 * 1024, "gla_scan: heads of %d key dimensions do not fit the local memory", dim);
  const dim3 grid(n_seqs * chunks.count, H, (vdim + VT - 1) / VT);
  const float inv_tau = 1.0f / tau;
#define BH_GLA(T, RR)                                                                                                        \
  do {                                                                                                                       \
    bh_allow_lds<gla_scan_kernel<T, RR>>(lds);                                                                               \
    gla_scan_kernel<T, RR><<<grid, 256, lds, stream>>>((const T*)proj, proj_stride, q_off, k_off, v_off, z, z_stride, bias,  \
                                                       inv_tau, q_scale, state, slot_stride, seq_start, seq_slot, out, H, dim, \
                                                       vdim, VT, chunks);                                                    \
  } while (0)
#define BH_GLA_R(T)                  \
  switch (R) {                       \
    case 1: BH_GLA(T, 1); break;     \
    case 2: BH_GLA(T, 2); break;     \
    case 4: BH_GLA(T, 4); break;     \
    case 8: BH_GLA(T, 8); break;     \
    case 16: BH_GLA(T, 16); break;   \
    case 32: BH_GLA(T, 32); break;   \
    default: BH_GLA(T, 64); break;   \
  }
  if (dtype == BH_F32) BH_GLA_R(float)
  else if (dtype == BH_BF16) BH_GLA_R(bf16_t)
  else return bh_fail("gla_scan: unknown dtype %d", dtype);
#undef BH_GLA_R
#undef BH_GLA
  if (int status = bh_check_launch("gla_scan")) return status;
  if (chunks.rows == 0) return 0;
  const size_t per = (size_t)H * dim * vdim;
  gla_combine_kernel<<<dim3((unsigned)((per + 255) / 256), n_seqs), 256, 0, stream>>>(chunks, state, slot_stride, seq_start, seq_slot, H, dim, vdim);
  if (int status = bh_check_launch("gla_combine")) return status;
  gla_carry_kernel<<<dim3(n_seqs * chunks.count, H, (vdim + 63) / 64), 256, 0, stream>>>(chunks, seq_start, out, H, dim, vdim);
  return bh_check_launch("gla_carry");
}
