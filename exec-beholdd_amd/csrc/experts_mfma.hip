// The routed experts' products of a prompt on the matrix cores, all experts in one launch.
// The pairs' inputs lie side by side, expert after expert (experts_gather); a table made from the experts' counts names
// every tile of up to 128 rows: {expert, first row, rows}.  A workgroup of four waves takes one tile of rows and
// 128 weight rows; a wave owns 32 of the tile's rows against all 128 weight rows (four blocks of v_mfma_f32_32x32x16_bf16).
// K goes through LDS in slices of 64 (16-byte pieces, rows padded to 144 bytes).
//   gated:  the 128 weight rows are the gate rows and the up rows of the same 64 outputs, so that a lane holds both
//           sums of an output and applies the activation itself; out bfloat16 [rows][N]
//   plain:  128 outputs; out float32 [rows][N]
// Operands (wave of 64 lanes, l = lane): A row l%32, k 8*(l/32)..+7;  B column l%32, the same k;
// D column l%32, rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15.
#include "common.h"

typedef __bf16 em_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float em_f32x16_t __attribute__((ext_vector_type(16)));

#define EM_TILE 128
#define EM_K 64
#define EM_PITCH 72      // bfloat16 elements from one LDS row to the next

__device__ inline em_bf16x8_t em_operand(const uint16_t* p) {
  union {
    uint4 raw;
    em_bf16x8_t v;
  } u;
  u.raw = *reinterpret_cast<const uint4*>(p);
  return u.v;
}

__device__ inline float em_act(float g, float u, float limit, float alpha, float shift) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + shift);
}

template <bool GATED>
__global__ __launch_bounds__(256) void experts_products_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ w,
                                                               const int32_t* __restrict__ tiles, void* __restrict__ out_raw, int K,
                                                               int N, float limit, float alpha, float shift) {
  __shared__ __align__(16) uint16_t lds_a[EM_TILE * EM_PITCH];
  __shared__ __align__(16) uint16_t lds_b[EM_TILE * EM_PITCH];
  const int expert = tiles[3 * blockIdx.x], first = tiles[3 * blockIdx.x + 1], rows = tiles[3 * blockIdx.x + 2];
  const int outs = GATED ? EM_TILE / 2 : EM_TILE;      // outputs of this workgroup
  const int n0 = blockIdx.y * outs;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint16_t* w_e = w + (size_t)expert * (GATED ? 2 : 1) * N * K;
  // the four 16-byte pieces of each operand that this thread brings per slice: tile row and piece within the row
  const uint16_t* from_a[4];
  const uint16_t* from_b[4];
  int to[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = threadIdx.x + 256 * i, row = q >> 3, piece = q & 7;
    const int a_row = row < rows ? row : rows - 1;      // rows beyond the tile's are read again and not stored
    int w_row;
    if (GATED) {
      const int o = n0 + (row & 63) < N ? n0 + (row & 63) : N - 1;
      w_row = row < 64 ? o : N + o;
    } else {
      w_row = n0 + row < N ? n0 + row : N - 1;
    }
    from_a[i] = a + (size_t)(first + a_row) * K + piece * 8;
    from_b[i] = w_e + (size_t)w_row * K + piece * 8;
    to[i] = row * EM_PITCH + piece * 8;
  }
  em_f32x16_t acc[4];
#pragma unroll
  for (int y = 0; y < 4; ++y)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[y][i] = 0.f;
  const int a_at = (wave * 32 + (lane & 31)) * EM_PITCH + 8 * (lane >> 5);
  const int b_at = (lane & 31) * EM_PITCH + 8 * (lane >> 5);
  uint4 got_a[4], got_b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    got_a[i] = *reinterpret_cast<const uint4*>(from_a[i]);
    got_b[i] = *reinterpret_cast<const uint4*>(from_b[i]);
  }
  for (int k0 = 0; k0 < K; k0 += EM_K) {
    __syncthreads();      // the slice before has been multiplied
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<uint4*>(lds_a + to[i]) = got_a[i];
      *reinterpret_cast<uint4*>(lds_b + to[i]) = got_b[i];
    }
    __syncthreads();
    if (k0 + EM_K < K) {      // the next slice is on its way while this one is multiplied
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        got_a[i] = *reinterpret_cast<const uint4*>(from_a[i] + k0 + EM_K);
        got_b[i] = *reinterpret_cast<const uint4*>(from_b[i] + k0 + EM_K);
      }
    }
#pragma unroll
    for (int kk = 0; kk < EM_K; kk += 16) {
      const em_bf16x8_t av = em_operand(lds_a + a_at + kk);
#pragma unroll
      for (int y = 0; y < 4; ++y)
        acc[y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, em_operand(lds_b + b_at + y * 32 * EM_PITCH + kk), acc[y], 0, 0, 0);
    }
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = wave * 32 + 8 * (i / 4) + 4 * (lane >> 5) + i % 4;
    if (row >= rows) continue;
    if (GATED) {
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        const int n = n0 + y * 32 + (lane & 31);
        if (n < N)
          reinterpret_cast<bf16_t*>(out_raw)[(size_t)(first + row) * N + n] = from_f32<bf16_t>(em_act(acc[y][i], acc[y + 2][i], limit, alpha, shift));
      }
    } else {
#pragma unroll
      for (int y = 0; y < 4; ++y) {
        const int n = n0 + y * 32 + (lane & 31);
        if (n < N) reinterpret_cast<float*>(out_raw)[(size_t)(first + row) * N + n] = acc[y][i];
      }
    }
  }
}

// Whether the one-launch form takes products of these sizes (bfloat16, K in whole slices).
extern "C" int bh_experts_products_takes(int K, int N) { return K > 0 && N > 0 && K % EM_K == 0; }

// a bfloat16 [rows][K]; w bfloat16 [E][gated ? 2 N : N][K]; tiles int32 [n_tiles][3] = {expert, first row, rows (1..128)} on the
// device; out bfloat16 [rows][N] (gated) or float32 [rows][N].
extern "C" int bh_experts_products(const void* a, const void* w, const int32_t* tiles, int n_tiles, void* out, int K, int N, int gated,
                                   float limit, float alpha, float shift, hipStream_t stream) {
  BH_REQUIRE(n_tiles > 0 && bh_experts_products_takes(K, N), "experts_products: K must be a multiple of %d, got %d", EM_K, K);
  const int outs = gated ? EM_TILE / 2 : EM_TILE;
  dim3 grid(n_tiles, (N + outs - 1) / outs);
  BH_REQUIRE(grid.y <= 65535, "experts_products: too many outputs");
  if (gated)
    experts_products_kernel<true><<<grid, 256, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, tiles, out, K, N, limit, alpha, shift);
  else
    experts_products_kernel<false><<<grid, 256, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, tiles, out, K, N, limit, alpha, shift);
  return bh_check_launch("experts_products");
}
