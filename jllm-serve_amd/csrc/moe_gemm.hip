// The grouped products of a table-routed mixture of experts on the matrix cores, bf16 (the tiles, maps and epilogues
// of moe_generic.hip). A tile is up to 16 rows of one expert; a wave multiplies them with 64 rows of the expert's weight
// (MFMA 16x16x32, weight rows as the first operand, the tile's activation rows, gathered by the tile's row list, as
// the second, both k-contiguous straight from memory): a lane ends up with four consecutive outputs of one row. With
// few rows per expert (decode steps) this streams every needed expert's weights once; a workgroup of four waves owns
// 256 outputs (128 of the gated product, whose waves hold the gate and the up sums of the same outputs).
#include "common.h"
#include "mfma.h"

#define MM_WAVES 4

// RB: 16-row blocks of a tile. Built with RB = 1: steps that give the experts many rows each go through the grouped form
// of the tiled product (gemm_mfma.hip) instead, which shares its operands through LDS.
template <bool GATED, int RB>
__global__ __launch_bounds__(MM_WAVES * 64) void moe_gemm_mfma_kernel(
    const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const bf16_t* __restrict__ W2,
    void* __restrict__ out, int out_dtype, int ldo, int N, int K, const int* __restrict__ sorted,
    const int* __restrict__ tiles, int top, int in_map, int out_map, float weight, GateSpec gs) {
  const int tile = blockIdx.y;
  const int rows = tiles[3 * tile + 2];
  if (rows == 0) return;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane & 15, q4 = lane >> 4;
  constexpr int NB = GATED ? 2 : 4;  // 16-output blocks per wave
  const int n0 = (blockIdx.x * MM_WAVES + wave) * (16 * NB);
  if (n0 >= N) return;
  int place[RB], asg[RB];
  const bf16_t* xrow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    place[rb] = first + min(16 * rb + sub, rows - 1);
    asg[rb] = sorted[place[rb]];
    xrow[rb] = A + (size_t)(in_map ? asg[rb] / top : place[rb]) * lda + 8 * q4;
  }
  const bf16_t* w = W + (size_t)e * N * K + 8 * q4;
  const bf16_t* w2 = GATED ? W2 + (size_t)e * N * K + 8 * q4 : nullptr;
  floatx4 acc[RB][NB], acc2[RB][NB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[rb][b] = acc2[rb][b] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool in_k = k0 + 8 * q4 < K;
    u32x4 xf[RB], wf[NB], uf[NB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) xf[rb] = in_k ? *(const u32x4*)(xrow[rb] + k0) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int n = n0 + 16 * b + sub;
      const bool ok = in_k && n < N;
      wf[b] = ok ? *(const u32x4*)(w + (size_t)n * K + k0) : u32x4{0u, 0u, 0u, 0u};
      if (GATED) uf[b] = ok ? *(const u32x4*)(w2 + (size_t)n * K + k0) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        acc[rb][b] = mfma16(wf[b], xf[rb], acc[rb][b]);
        if (GATED) acc2[rb][b] = mfma16(uf[b], xf[rb], acc2[rb][b]);
      }
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    if (16 * rb + sub >= rows) continue;
    const size_t orow = out_map == 0 ? (size_t)place[rb] : out_map == 1 ? (size_t)asg[rb] : (size_t)(asg[rb] / top);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int n = n0 + 16 * b + 4 * q4;
      if (n >= N) continue;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = GATED ? gated<true>(acc[rb][b][i], acc2[rb][b][i], gs) : acc[rb][b][i];
      const size_t o = orow * ldo + n;
      if (out_map == 2) {
        floatx4* dst = (floatx4*)((float*)out + o);
        const floatx4 cur = *dst;
        *dst = floatx4{cur[0] + weight * v[0], cur[1] + weight * v[1], cur[2] + weight * v[2], cur[3] + weight * v[3]};
      } else if (out_dtype == JLLM_BF16) {
        *(u32x2*)((bf16_t*)out + o) = u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
      } else {
        *(floatx4*)((float*)out + o) = floatx4{v[0], v[1], v[2], v[3]};
      }
    }
  }
}

// returns 0 when it ran, 1 when the shape is not one it takes, -1 on errors
extern "C" int jllm_moe_gemm_bf16(const void* A, int a_dtype, int lda, const void* W, const void* W2, int w_dtype, void* out,
                                  int out_dtype, int ldo, int N, int K, const int* sorted, const int* tiles, int max_tiles,
                                  int tile_rows, int top, int in_map, int out_map, float weight, int epilogue,
                                  float gate_limit, hipStream_t stream) {
  if (max_tiles <= 0) return 0;
  if (a_dtype != JLLM_BF16 || w_dtype != JLLM_BF16) return 1;
  if (N <= 0 || K <= 0 || lda < K || ldo < N) JLLM_FAIL("moe_gemm: N %d K %d lda %d ldo %d", N, K, lda, ldo);
  if (tile_rows != 16) JLLM_FAIL("moe_gemm: this kernel takes tiles of 16 rows, the route made %d", tile_rows);
  JLLM_TAKE_GATE("moe_gemm", epilogue, gate_limit, gs);
  if ((epilogue != 0 && epilogue != 2) || (epilogue == 2) != (W2 != nullptr)) JLLM_FAIL("moe_gemm: epilogue %d", epilogue);
  if (in_map < 0 || in_map > 1 || out_map < 0 || out_map > 2) JLLM_FAIL("moe_gemm: maps %d / %d", in_map, out_map);
  if (out_map == 2 && (top != 1 || out_dtype != JLLM_F32)) JLLM_FAIL("moe_gemm: adding into the token's row needs top = 1 and fp32 rows");
  if (max_tiles > 65535) return 1;
  // 16-byte operand loads, 8- or 16-byte stores
  if ((K & 7) || (N & 3) || (lda & 7) || ((uintptr_t)A & 15) || ((uintptr_t)W & 15) || (W2 && ((uintptr_t)W2 & 15))) return 1;
  const int need = out_dtype == JLLM_BF16 ? 7 : 15;
  if (((uintptr_t)out & need) || (ldo & 3)) return 1;
  const int per_group = MM_WAVES * 16 * (W2 ? 2 : 4);
  dim3 grid((N + per_group - 1) / per_group, max_tiles);
#define MM_LAUNCH(GATED, RB)                                                                                                    \
  moe_gemm_mfma_kernel<GATED, RB><<<grid, MM_WAVES * 64, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)W2, out, \
                                                                      out_dtype, ldo, N, K, sorted, tiles, top, in_map, out_map, weight, gs)
  if (W2)
    MM_LAUNCH(true, 1);
  else
    MM_LAUNCH(false, 1);
#undef MM_LAUNCH
  JLLM_CHECK_LAUNCH("moe_gemm_bf16");
  return 0;
}
