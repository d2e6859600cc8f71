// The per-head products of latent attention on the matrix cores, bf16: out[t, h, :] = W[h] in[t, h, :] for all heads in
// one launch (W[h] is [N, K] row-major; see latent_generic.hip for the two forms). MFMA 16x16x32 with the weight rows
// as the first operand and 16 activation rows as the second, both read k-contiguous straight from memory (the
// weights of a head are small and stay in the caches; nothing is staged): a lane ends up with four consecutive
// outputs of one row, stores them at once, and in the gated form multiplies them by sigmoid of the four gate
// entries first (fp32). The tail of the query side (rotation and copy) is done by one more column of workgroups.
#include <math.h>

#include "common.h"
#include "mfma.h"

#define LHM_WAVES 4

// RB = 1 (up to 16 rows: a decode step): the four waves of a workgroup take four blocks of 64 outputs of the same 16
// rows. RB = 4: a wave takes 64 rows by 64 outputs (a weight fragment meets four activation fragments), the four waves
// four such row blocks.
template <int RB>
__global__ __launch_bounds__(LHM_WAVES * 64) void latent_heads_mfma_kernel(
    const bf16_t* __restrict__ in, int ld_in, int in_hstride, const bf16_t* __restrict__ W, bf16_t* __restrict__ out,
    int ld_out, int out_hstride, int M, int N, int K, int mode, int tail, int rot_dims,
    const int* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const bf16_t* __restrict__ gate, int ld_gate, int n_blocks) {
  const int h = blockIdx.z;
  constexpr int ROWS = RB == 1 ? 16 : LHM_WAVES * 64;  // rows of a workgroup
  const int m0 = blockIdx.x * ROWS;
  const bf16_t* a = in + (size_t)h * in_hstride;
  bf16_t* o = out + (size_t)h * out_hstride;
  if ((int)blockIdx.y == n_blocks) {  // the rotated tail of this head for these rows
    const int half = rot_dims >> 1;
    for (int e = threadIdx.x; e < ROWS * tail; e += LHM_WAVES * 64) {
      const int m = m0 + e / tail, i = e % tail;
      if (m >= M) break;
      const bf16_t* src = a + (size_t)m * ld_in + K;
      const size_t at = (size_t)positions[m] * half;
      float v = ldf(src, i);
      if (i < half)
        v = v * cos_t[at + i] - ldf(src, i + half) * sin_t[at + i];
      else if (i < rot_dims)
        v = v * cos_t[at + i - half] + ldf(src, i - half) * sin_t[at + i - half];
      stf(o + (size_t)m * ld_out, N + i, v);
    }
    return;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane & 15, q4 = lane >> 4;
  const int t0 = RB == 1 ? m0 : m0 + wave * 64;
  const int n0 = RB == 1 ? (blockIdx.y * LHM_WAVES + wave) * 64 : blockIdx.y * 64;
  if (t0 >= M || n0 >= N) return;
  const bf16_t* xrow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) xrow[rb] = a + (size_t)min(t0 + 16 * rb + sub, M - 1) * ld_in + 8 * q4;
  const bf16_t* w = W + (size_t)h * N * K + 8 * q4;
  floatx4 acc[RB][4];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[rb][b] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool in_k = k0 + 8 * q4 < K;
    u32x4 xf[RB], wf[4];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) xf[rb] = in_k ? *(const u32x4*)(xrow[rb] + k0) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int n = n0 + 16 * b + sub;
      wf[b] = (in_k && n < N) ? *(const u32x4*)(w + (size_t)n * K + k0) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int b = 0; b < 4; ++b) acc[rb][b] = mfma16(wf[b], xf[rb], acc[rb][b]);
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int t = t0 + 16 * rb + sub;
    if (t >= M) continue;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int n = n0 + 16 * b + 4 * q4;  // this lane's four outputs n .. n + 3 of row t
      if (n >= N) continue;
      float v[4] = {acc[rb][b][0], acc[rb][b][1], acc[rb][b][2], acc[rb][b][3]};
      if (mode == 1) {
        const u32x2 g = *(const u32x2*)(gate + (size_t)t * ld_gate + (size_t)h * N + n);
        const float gv[4] = {__uint_as_float(g[0] << 16), __uint_as_float(g[0] & 0xffff0000u), __uint_as_float(g[1] << 16),
                             __uint_as_float(g[1] & 0xffff0000u)};
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = v[i] / (1.0f + __expf(-gv[i]));
      }
      *(u32x2*)(o + (size_t)t * ld_out + n) = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
    }
  }
}

// returns 0 when it ran, 1 when the shape is not one it takes, -1 on errors
extern "C" int jllm_latent_heads_bf16(const void* in, int ld_in, int in_hstride, const void* W, void* out, int ld_out,
                                      int out_hstride, int M, int H, int N, int K, int mode, int tail, int rot_dims,
                                      const int* positions, const float* cos_t, const float* sin_t, const void* gate,
                                      int ld_gate, hipStream_t stream) {
  if (M <= 0) return 0;
  if (H <= 0 || N <= 0 || K <= 0 || H > 65535 || (mode != 0 && mode != 1)) JLLM_FAIL("latent_heads: %d heads of %d x %d, mode %d", H, N, K, mode);
  // 16-byte operand loads and 8-byte stores: every head's inputs, weights, outputs and gate entries must start on them
  if ((K & 7) || (N & 3) || (ld_in & 7) || (in_hstride & 7) || (ld_out & 3) || (out_hstride & 3) || ((uintptr_t)in & 15) ||
      ((uintptr_t)W & 15) || ((uintptr_t)out & 7))
    return 1;
  if (mode == 1 && ((ld_gate & 3) || ((uintptr_t)gate & 7) || !gate)) return 1;
  if (mode == 0 && tail > 0 && (!positions || (rot_dims && (!cos_t || !sin_t)))) JLLM_FAIL("latent_heads: the rotated tail needs positions and tables");
  const bool few = M <= 16;
  const int n_blocks = few ? (N + LHM_WAVES * 64 - 1) / (LHM_WAVES * 64) : (N + 63) / 64;
  const int rows = few ? 16 : LHM_WAVES * 64;
  dim3 grid((M + rows - 1) / rows, n_blocks + ((mode == 0 && tail > 0) ? 1 : 0), H);
  if (grid.y > 65535) return 1;
  if (few)
    latent_heads_mfma_kernel<1><<<grid, LHM_WAVES * 64, 0, stream>>>((const bf16_t*)in, ld_in, in_hstride, (const bf16_t*)W,
                                                                    (bf16_t*)out, ld_out, out_hstride, M, N, K, mode,
                                                                    mode == 0 ? tail : 0, rot_dims, positions, cos_t, sin_t,
                                                                    (const bf16_t*)gate, ld_gate, n_blocks);
  else
    latent_heads_mfma_kernel<4><<<grid, LHM_WAVES * 64, 0, stream>>>((const bf16_t*)in, ld_in, in_hstride, (const bf16_t*)W,
                                                                    (bf16_t*)out, ld_out, out_hstride, M, N, K, mode,
                                                                    mode == 0 ? tail : 0, rot_dims, positions, cos_t, sin_t,
                                                                    (const bf16_t*)gate, ld_gate, n_blocks);
  JLLM_CHECK_LAUNCH("latent_heads_bf16");
  return 0;
}
