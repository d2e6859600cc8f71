// Layer norm with weight and bias over fp32 rows of the residual stream, alone or as the seam between two sublayers.
//
//   y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w + b          all sums and the result in fp32
//
// One workgroup per row, the row in registers, two block sums in a fixed order (mean, then the squared deviations), so
// a row's result depends on nothing but the row. One kernel does up to three things to a row, in this order:
//   1. with `a`: the row t = s1 * a (+ s2 * a2) is normed with (w_post, b_post) and added into the residual row
//      (a sublayer whose output passes a norm of its own before it joins the stream; two branches with fixed weights)
//   2. with `add_vec`: a vector is added to the residual row (a learned offset for every row of the step)
//   3. with `out`: the (new) residual row is normed with (w_next, b_next) into `out` for the next sublayer's products
// With a row list, only 3 runs and row i of `out` is the norm of residual row rows[i] (the rows whose logits are wanted).
#include <math.h>

#include "common.h"

#define LN_THREADS 256

template <int VPT>
__device__ __forceinline__ void ln_stats(const float (&v)[VPT], int d, float* red, float& mean, float& rstd, float eps) {
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    if (i < d) s += v[k];
  }
  mean = block_sum<LN_THREADS / 64>(s, red) / (float)d;
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    if (i < d) {
      const float c = v[k] - mean;
      q = fmaf(c, c, q);
    }
  }
  const float var = block_sum<LN_THREADS / 64>(q, red) / (float)d;
  rstd = (float)(1.0 / sqrt((double)(var + eps)));
}

template <typename TA, typename TW, typename TO, int VPT>
__global__ __launch_bounds__(LN_THREADS) void layernorm_seam_kernel(
    float* __restrict__ residual, const int* __restrict__ rows, int d, const TA* __restrict__ a, int lda,
    const TA* __restrict__ a2, int lda2, float s1, float s2, const TW* __restrict__ w_post, const TW* __restrict__ b_post,
    const TW* __restrict__ add_vec, const TW* __restrict__ w_next, const TW* __restrict__ b_next, float eps,
    TO* __restrict__ out, int ldo) {
  __shared__ float red[LN_THREADS / 64];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = residual + src * d;
  // everything the row needs is requested before the first sum: with a few rows a launch is a chain of memory
  // latencies, and each phase that asked for its own operands added one
  float x[VPT], t[VPT], wp[VPT], bp[VPT], wn[VPT], bn[VPT], av[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    const bool on = i < d;
    x[k] = on ? xr[i] : 0.f;
    t[k] = (on && a) ? ldf(a + (size_t)r * lda, i) : 0.f;
    av[k] = (on && a2) ? ldf(a2 + (size_t)r * lda2, i) : 0.f;
    wp[k] = (on && a) ? ldf(w_post, i) : 0.f;
    bp[k] = (on && a) ? ldf(b_post, i) : 0.f;
    wn[k] = (on && out) ? ldf(w_next, i) : 0.f;
    bn[k] = (on && out) ? ldf(b_next, i) : 0.f;
  }
  if (a) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) t[k] = a2 ? fmaf(s2, av[k], s1 * t[k]) : s1 * t[k];
    float mean, rstd;
    ln_stats<VPT>(t, d, red, mean, rstd, eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) x[k] += (t[k] - mean) * rstd * wp[k] + bp[k];
  }
  if (add_vec) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int i = threadIdx.x + k * LN_THREADS;
      if (i < d) x[k] += ldf(add_vec, i);
    }
  }
  if (a || add_vec) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int i = threadIdx.x + k * LN_THREADS;
      if (i < d) xr[i] = x[k];
    }
  }
  if (out) {
    float mean, rstd;
    ln_stats<VPT>(x, d, red, mean, rstd, eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int i = threadIdx.x + k * LN_THREADS;
      if (i < d) stf(out + (size_t)r * ldo, i, (x[k] - mean) * rstd * wn[k] + bn[k]);
    }
  }
}

// The same with four consecutive elements per thread and load (16 bytes of fp32, 8 of bf16) and one barrier per sum:
// every sum has its own place in LDS, so nothing has to be waited for before it is written. For rows whose length and
// strides are multiples of four; the sums run over the same elements in another order than in the kernel above.
__device__ __forceinline__ void ld4(const float* p, float (&v)[4]) {
  const float4 t = *(const float4*)p;
  v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
}
__device__ __forceinline__ void ld4(const bf16_t* p, float (&v)[4]) {
  const uint2 t = *(const uint2*)p;
  v[0] = __uint_as_float(t.x << 16), v[1] = __uint_as_float(t.x & 0xffff0000u);
  v[2] = __uint_as_float(t.y << 16), v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void st4(float* p, const float (&v)[4]) { *(float4*)p = float4{v[0], v[1], v[2], v[3]}; }
__device__ __forceinline__ void st4(bf16_t* p, const float (&v)[4]) {
  uint2 t;
  t.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
  t.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
  *(uint2*)p = t;
}

__device__ __forceinline__ float block_sum_once(float v, float* red) {  // red: LN_THREADS / 64 floats of this sum's own
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < LN_THREADS / 64; ++i) s += red[i];
  return s;
}

template <int G>
__device__ __forceinline__ void ln_stats4(const float (&v)[G][4], int d, float* red, float& mean, float& rstd, float eps) {
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < G; ++k)
    if ((threadIdx.x + k * LN_THREADS) * 4 < d) s += (v[k][0] + v[k][1]) + (v[k][2] + v[k][3]);
  mean = block_sum_once(s, red) / (float)d;
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < G; ++k)
    if ((threadIdx.x + k * LN_THREADS) * 4 < d) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float c = v[k][e] - mean;
        q = fmaf(c, c, q);
      }
    }
  const float var = block_sum_once(q, red + LN_THREADS / 64) / (float)d;
  rstd = (float)(1.0 / sqrt((double)(var + eps)));
}

template <typename TA, typename TW, typename TO, int G>
__global__ __launch_bounds__(LN_THREADS) void layernorm_seam4_kernel(
    float* __restrict__ residual, const int* __restrict__ rows, int d, const TA* __restrict__ a, int lda,
    const TA* __restrict__ a2, int lda2, float s1, float s2, const TW* __restrict__ w_post, const TW* __restrict__ b_post,
    const TW* __restrict__ add_vec, const TW* __restrict__ w_next, const TW* __restrict__ b_next, float eps,
    TO* __restrict__ out, int ldo) {
  __shared__ float red[4 * (LN_THREADS / 64)];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* xr = residual + src * d;
  float x[G][4], t[G][4], av[G][4], wp[G][4], bp[G][4], wn[G][4], bn[G][4], vc[G][4];
#pragma unroll
  for (int k = 0; k < G; ++k) {
    const int i = (threadIdx.x + k * LN_THREADS) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) x[k][e] = t[k][e] = av[k][e] = wp[k][e] = bp[k][e] = wn[k][e] = bn[k][e] = vc[k][e] = 0.f;
    if (i >= d) continue;
    ld4(xr + i, x[k]);
    if (a) {
      ld4(a + (size_t)r * lda + i, t[k]);
      ld4(w_post + i, wp[k]);
      ld4(b_post + i, bp[k]);
    }
    if (a2) ld4(a2 + (size_t)r * lda2 + i, av[k]);
    if (add_vec) ld4(add_vec + i, vc[k]);
    if (out) {
      ld4(w_next + i, wn[k]);
      ld4(b_next + i, bn[k]);
    }
  }
  if (a) {
#pragma unroll
    for (int k = 0; k < G; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) t[k][e] = a2 ? fmaf(s2, av[k][e], s1 * t[k][e]) : s1 * t[k][e];
    float mean, rstd;
    ln_stats4<G>(t, d, red, mean, rstd, eps);
#pragma unroll
    for (int k = 0; k < G; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) x[k][e] += (t[k][e] - mean) * rstd * wp[k][e] + bp[k][e];
  }
  if (add_vec) {
#pragma unroll
    for (int k = 0; k < G; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) x[k][e] += vc[k][e];
  }
  if (a || add_vec) {
#pragma unroll
    for (int k = 0; k < G; ++k) {
      const int i = (threadIdx.x + k * LN_THREADS) * 4;
      if (i < d) st4(xr + i, x[k]);
    }
  }
  if (out) {
    float mean, rstd;
    ln_stats4<G>(x, d, red + 2 * (LN_THREADS / 64), mean, rstd, eps);
#pragma unroll
    for (int k = 0; k < G; ++k) {
      const int i = (threadIdx.x + k * LN_THREADS) * 4;
      if (i >= d) continue;
      float y[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = (x[k][e] - mean) * rstd * wn[k][e] + bn[k][e];
      st4(out + (size_t)r * ldo + i, y);
    }
  }
}

// residual fp32 [*, d] contiguous; a, a2: [n, >= d] in a_dtype or null; weights, biases and the vector in w_dtype;
// out [n, ldo] in out_dtype or null
extern "C" int jllm_layernorm_seam(float* residual, const int* rows, int n, int d, const void* a, int lda, const void* a2,
                                   int lda2, int a_dtype, float s1, float s2, const void* w_post, const void* b_post,
                                   const void* add_vec, const void* w_next, const void* b_next, int w_dtype, float eps,
                                   void* out, int out_dtype, int ldo, hipStream_t stream) {
  if (n <= 0) return 0;
  if (d <= 0 || d > LN_THREADS * 32) JLLM_FAIL("layernorm: rows of %d entries (this kernel takes 1..%d)", d, LN_THREADS * 32);
  if (a && (!w_post || !b_post || lda < d || (a2 && lda2 < d))) JLLM_FAIL("layernorm: a branch without its norm or with short rows");
  if (a2 && !a) JLLM_FAIL("layernorm: a second branch without a first");
  if (out && (!w_next || !b_next || ldo < d)) JLLM_FAIL("layernorm: an output without its norm or with short rows");
  if (rows && (a || add_vec)) JLLM_FAIL("layernorm: a row list goes with the output norm alone");
  if (!a && !add_vec && !out) return 0;
  // four elements per thread and load where the rows allow it
  auto mult = [](const void* p, size_t bytes) { return ((uintptr_t)p % bytes) == 0; };
  const size_t ea = a_dtype == JLLM_F32 ? 4 : 2, ew = w_dtype == JLLM_F32 ? 4 : 2, eo = out_dtype == JLLM_F32 ? 4 : 2;
  const bool wide = d % 4 == 0 && d <= LN_THREADS * 32 && mult(residual, 16) && (!a || (lda % 4 == 0 && mult(a, 4 * ea))) &&
                    (!a2 || (lda2 % 4 == 0 && mult(a2, 4 * ea))) && mult(w_post, 4 * ew) && mult(b_post, 4 * ew) &&
                    mult(add_vec, 4 * ew) && mult(w_next, 4 * ew) && mult(b_next, 4 * ew) && (!out || (ldo % 4 == 0 && mult(out, 4 * eo)));
#define LN_LAUNCH4(G)                                                                                                 \
  layernorm_seam4_kernel<TA, TW, TO, G><<<n, LN_THREADS, 0, stream>>>(                                                \
      residual, rows, d, (const TA*)a, lda, (const TA*)a2, lda2, s1, s2, (const TW*)w_post, (const TW*)b_post,        \
      (const TW*)add_vec, (const TW*)w_next, (const TW*)b_next, eps, (TO*)out, ldo)
#define LN_LAUNCH(VPT)                                                                                                \
  layernorm_seam_kernel<TA, TW, TO, VPT><<<n, LN_THREADS, 0, stream>>>(                                               \
      residual, rows, d, (const TA*)a, lda, (const TA*)a2, lda2, s1, s2, (const TW*)w_post, (const TW*)b_post,        \
      (const TW*)add_vec, (const TW*)w_next, (const TW*)b_next, eps, (TO*)out, ldo)
  JLLM_DISPATCH_1(a_dtype, TA, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      JLLM_DISPATCH_1(out_dtype, TO, {
        if (wide && d <= LN_THREADS * 4)
          LN_LAUNCH4(1);
        else if (wide && d <= LN_THREADS * 8)
          LN_LAUNCH4(2);
        else if (wide && d <= LN_THREADS * 16)
          LN_LAUNCH4(4);
        else if (wide)
          LN_LAUNCH4(8);
        else if (d <= LN_THREADS * 4)
          LN_LAUNCH(4);
        else if (d <= LN_THREADS * 8)
          LN_LAUNCH(8);
        else if (d <= LN_THREADS * 16)
          LN_LAUNCH(16);
        else
          LN_LAUNCH(32);
      })
    })
  })
#undef LN_LAUNCH
#undef LN_LAUNCH4
  JLLM_CHECK_LAUNCH("layernorm_seam");
  return 0;
}
