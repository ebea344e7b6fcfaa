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
// LDS, in a fixed order.  The next stage's
// numbers are asked for (into registers, GLA_AHEAD elements a thread and array; what a stage has beyond that is read when it
// is staged) before this stage's rows are walked, so that the walk hides their way from memory.
#define GLA_AHEAD 4
#define GLA_GROUP 4

template <typename T, int R>
__global__ __launch_bounds__(256) void gla_scan_kernel(const T* __restrict__ proj, int proj_stride, int q_off, int k_off, int v_off,
                                                       const float* __restrict__ z, int z_stride, const float* __restrict__ bias,
                                                       float inv_tau, float q_scale, float* __restrict__ state, long slot_stride,
                                                       const int32_t* __restrict__ seq_start, const int32_t* __restrict__ seq_slot,
                                                       float* __restrict__ out, int H, int dim, int vdim, int VT) {
  extern __shared__ __align__(16) float lds[];
  const int SL = 256 / VT, DP = SL * R;      // VT and R are powers of two, so are SL and DP: shifts and masks below
  const int dp_shift = __builtin_ctz(DP), vt_shift = __builtin_ctz(VT);
  float* a_s = lds;                          // [GLA_STAGE][DP]
  float* k_s = a_s + GLA_STAGE * DP;
  float* q_s = k_s + GLA_STAGE * DP;
  float* v_s = q_s + GLA_STAGE * DP;         // [GLA_STAGE][VT]
  float* part = v_s + GLA_STAGE * VT;        // [GLA_STAGE][PARTS][VT]: a wave's slices' shares added up (VT < 64), or a slice's own
  const int PARTS = VT >= BH_WAVE ? SL : 256 / BH_WAVE;
  const int seq = blockIdx.x, head = blockIdx.y, v0 = blockIdx.z * VT;
  const int col = threadIdx.x & (VT - 1), slice = threadIdx.x >> vt_shift, d0 = slice * R;
  const bool has_column = v0 + col < vdim;
  const int start = seq_start[seq], stop = seq_start[seq + 1];
  float* mine = state + (size_t)seq_slot[seq] * slot_stride + (size_t)head * dim * vdim + v0 + col;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = (has_column && d0 + r < dim) ? mine[(size_t)(d0 + r) * vdim] : 0.f;
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
}

// How many value columns a workgroup takes for a step of these sizes.  A stage costs a workgroup about as many instructions
// whatever its tile (the staging of decays, keys and queries is the same for every tile of a head), so narrow tiles multiply
// the work: they pay only while they bring idle compute units in, up to about one workgroup a unit; and never so narrow that
// a thread's slice of a state column exceeds 64 rows.
static int gla_tile(int n_seqs, int H, int dim, int vdim) {
  int tile = 64;
  while (tile > 8 && (tile / 2 >= vdim || (long)n_seqs * H * ((vdim + tile - 1) / tile) < (long)bh_compute_units())) tile /= 2;
  while (tile > 8 && (dim + 256 / tile - 1) / (256 / tile) > 64) tile /= 2;
  return tile;
}

// proj [rows][proj_stride] (dtype): a row holds H heads of q and of k (dim each) from q_off and k_off and H heads of v (vdim) from
// v_off.  z [rows][z_stride] float32: the decays' pre-activations, H x dim from column 0; bias [H * dim] float32.
// state [slots][slot_stride] float32, a slot's first H * dim * vdim floats being its heads' states; seq_start [n_seqs + 1],
// seq_slot [n_seqs]; out [rows][H * vdim] float32.
extern "C" int bh_gla_scan(const void* proj, int dtype, int proj_stride, int q_off, int k_off, int v_off, const float* z, int z_stride,
                           const float* bias, float tau, float q_scale, float* state, long slot_stride, const int32_t* seq_start,
                           const int32_t* seq_slot, float* out, int n_seqs, int H, int dim, int vdim, hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && H > 0 && dim > 0 && vdim > 0, "gla_scan: sizes must be positive");
  BH_REQUIRE(tau > 0.f, "gla_scan: tau must be positive, got %f", (double)tau);
  BH_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + H * dim <= proj_stride && k_off + H * dim <= proj_stride &&
                 v_off + H * vdim <= proj_stride, "gla_scan: q, k or v lie outside a row of %d", proj_stride);
  BH_REQUIRE(z_stride >= H * dim, "gla_scan: the decays' rows hold %d numbers, %d are needed", z_stride, H * dim);
  BH_REQUIRE(slot_stride >= (long)H * dim * vdim, "gla_scan: a slot's state is smaller than the heads' states");
  BH_REQUIRE(H <= 65535 && (vdim + 7) / 8 <= 65535, "gla_scan: too many heads or value columns");
  const int VT = gla_tile(n_seqs, H, dim, vdim), SL = 256 / VT;
  int R = 1;
  while (R * SL < dim) R *= 2;
  BH_REQUIRE(R <= 64, "gla_scan: heads of %d key dimensions are above the limit of %d", dim, 64 * 32);
  const size_t lds = (size_t)GLA_STAGE * (3 * SL * R + VT + 256) * sizeof(float);
  BH_REQUIRE(lds <= 160 * 1024, "gla_scan: heads of %d key dimensions do not fit the local memory", dim);
  const dim3 grid(n_seqs, H, (vdim + VT - 1) / VT);
  const float inv_tau = 1.0f / tau;
#define BH_GLA(T, RR)                                                                                                        \
  do {                                                                                                                       \
    bh_allow_lds<gla_scan_kernel<T, RR>>(lds);                                                                               \
    gla_scan_kernel<T, RR><<<grid, 256, lds, stream>>>((const T*)proj, proj_stride, q_off, k_off, v_off, z, z_stride, bias,  \
                                                       inv_tau, q_scale, state, slot_stride, seq_start, seq_slot, out, H, dim, \
                                                       vdim, VT);                                                            \
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
  return bh_check_launch("gla_scan");
}
