// A gated delta rule with short causal convolutions in front: a recurrent mixer whose per-request state is one matrix
// per head (fp32) and the last taps - 1 inputs of every convolved channel. fp32 or bf16 activations, all arithmetic in
// fp32. A request's rows of a step are consecutive and in order (row_req ascends), so every kernel finds a request's
// rows in the step by itself and the same launches serve portions of prompts, single rows and steps of fixed size.
//
//   short_conv_silu      y[t, c] = silu(sum_j taps[c, K - 1 - j] x[t - j, c]); inputs before the step's first row of a
//                        request come from that request's state, inputs before position 0 are the state's zeros
//   short_conv_advance   the state's K - 1 inputs per channel move on by the request's rows of this step
//   gated_delta          per (request, head), token by token, with S [dk, dv] in registers:
//                          q <- q / sqrt(sum q^2 + 1e-6) / sqrt(dk), k <- k / sqrt(sum k^2 + 1e-6)
//                          beta = sigmoid(b), g = exp(-exp(A_log) * softplus(a + dt_bias))
//                          S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//                        computed as  S^T k and S^T q of the old S in one pass, o = g S^T q + (k . q) u
//                          out = o / sqrt(mean(o^2) + eps) * gain * silu(gate)
#include <math.h>

#include "common.h"

#define CONV_MAX_TAPS 16
#define GDR_MAX_PARTS 32

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

template <typename T, typename TW>
__global__ __launch_bounds__(256) void short_conv_silu_kernel(const T* __restrict__ x, int ldx, T* __restrict__ y, int ldy,
                                                              int channels, int taps, const TW* __restrict__ w,
                                                              const float* __restrict__ state,
                                                              const int* __restrict__ row_req,
                                                              const int* __restrict__ state_slots) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int req = row_req[t];
  int m = 0;  // rows of the same request in front of this one, as far as the taps reach
  while (m < taps - 1 && t - m - 1 >= 0 && row_req[t - m - 1] == req) ++m;
  const float* st = state + (size_t)state_slots[req] * (taps - 1) * channels;
  float acc = 0.f;
  for (int j = taps - 1; j >= 0; --j) {  // oldest input first
    float v;
    if (j <= m)
      v = ldf(x + (size_t)(t - j) * ldx, c);
    else
      v = st[(size_t)(taps - 1 - (j - m)) * channels + c];
    acc = fmaf(ldf(w, (size_t)c * taps + (taps - 1 - j)), v, acc);
  }
  stf(y + (size_t)t * ldy, c, silu_f(acc));
}

// first row and number of rows of request `req` in the ascending list row_req[0 .. n)
__device__ __forceinline__ void rows_of_request(const int* __restrict__ row_req, int n, int req, int& lo, int& cnt) {
  int a = 0, b = n;
  while (a < b) {
    const int mid = (a + b) >> 1;
    if (row_req[mid] < req) a = mid + 1; else b = mid;
  }
  lo = a;
  b = n;
  while (a < b) {
    const int mid = (a + b) >> 1;
    if (row_req[mid] <= req) a = mid + 1; else b = mid;
  }
  cnt = a - lo;
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_advance_kernel(const T* __restrict__ x, int ldx, int channels, int taps,
                                                                 float* __restrict__ state, const int* __restrict__ row_req,
                                                                 int n_rows, const int* __restrict__ state_slots) {
  const int req = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  int lo, n;
  rows_of_request(row_req, n_rows, req, lo, n);
  if (n == 0) return;
  float* st = state + (size_t)state_slots[req] * (taps - 1) * channels;
  float keep[CONV_MAX_TAPS];
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS; ++i) {
    if (i >= taps - 1) break;
    const int at = n - (taps - 1) + i;  // which input of this step, counted from the request's first row
    keep[i] = at >= 0 ? ldf(x + (size_t)(lo + at) * ldx, c) : st[(size_t)(taps - 1 + at) * channels + c];
  }
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS; ++i) {
    if (i >= taps - 1) break;
    st[(size_t)i * channels + c] = keep[i];
  }
}

extern "C" int jllm_short_conv(const void* x, int ldx, void* y, int ldy, int dtype, int n_rows, int n_requests, int channels,
                               int taps, const void* w, int w_dtype, float* state, const int* row_req,
                               const int* state_slots, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (channels <= 0 || taps < 1 || taps > CONV_MAX_TAPS) JLLM_FAIL("short_conv: %d channels, %d taps (1..%d taps are taken)", channels, taps, CONV_MAX_TAPS);
  if (ldx < channels || ldy < channels || n_requests <= 0 || n_requests > n_rows) JLLM_FAIL("short_conv: rows %d/%d of %d channels, %d requests in %d rows", ldx, ldy, channels, n_requests, n_rows);
  const int cb = (channels + 255) / 256;
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      short_conv_silu_kernel<T, TW><<<dim3(n_rows, cb), 256, 0, stream>>>((const T*)x, ldx, (T*)y, ldy, channels, taps, (const TW*)w,
                                                                          state, row_req, state_slots);
    })
    if (taps > 1)
      short_conv_advance_kernel<T><<<dim3(n_requests, cb), 256, 0, stream>>>((const T*)x, ldx, channels, taps, state, row_req,
                                                                             n_rows, state_slots);
  })
  JLLM_CHECK_LAUNCH("short_conv");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------

struct GdrArgs {
  const void* qkv;   // [rows, ldc]: q (kv_heads x dk) | k (kv_heads x dk) | v (heads x dv), convolved
  int ldc;
  const void* proj;  // [rows, ldp]: the projection's row, which holds the gate (heads x dv), a and b (heads each)
  int ldp, gate_off, a_off, b_off;
  const void* a_log;    // [heads]
  const void* dt_bias;  // [heads]
  const void* gain;     // [dv]
  float* state;         // [slots, heads, dk, dv]
  void* out;            // [rows, ldo]: heads x dv
  int ldo;
  const int* row_req;
  const int* state_slots;
  int n_rows, heads, kv_heads, dk, dv, parts;
  float eps;
};

// Threads (j, part): j = tid % dv is a value column, part = tid / dv owns rows part, part + P, ... of S (E at most).
// The workgroup is filled up to whole waves; the threads beyond dv * P only take part in the waves' sums.
template <typename T, typename TW, int E>
__global__ void gated_delta_kernel(GdrArgs A) {
  extern __shared__ float sm[];
  const int dk = A.dk, dv = A.dv, P = A.parts;
  const int nthreads = blockDim.x;
  const int tid = threadIdx.x;
  const int j = tid % dv, part = tid / dv;
  const bool act = part < P;
  const int lane = tid & 63;
  // per parity: q[dk], k[dk], partial sums [2][P][dv], o[dv]
  const int per = 2 * dk + 2 * P * dv + dv;
  const int req = blockIdx.x, h = blockIdx.y;
  int lo, n;
  rows_of_request(A.row_req, A.n_rows, req, lo, n);
  if (n == 0) return;
  const int kvh = h / (A.heads / A.kv_heads);
  float* S_at = A.state + ((size_t)A.state_slots[req] * A.heads + h) * dk * dv;
  float S[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = part + e * P;
    S[e] = (act && i < dk) ? S_at[(size_t)i * dv + j] : 0.f;
  }
  const float decay_rate = expf(ldf((const TW*)A.a_log, h));
  const float dtb = ldf((const TW*)A.dt_bias, h);
  const float gain = ldf((const TW*)A.gain, j);
  const float q_scale = 1.0f / sqrtf((float)dk);
  const T* conv = (const T*)A.qkv;
  const T* proj = (const T*)A.proj;
  T* out = (T*)A.out;
  for (int r = 0; r < n; ++r) {
    const size_t row = (size_t)(lo + r);
    float* buf = sm + (size_t)(r & 1) * per;
    float* qs = buf;
    float* ks = buf + dk;
    float* pk = buf + 2 * dk;
    float* pq = pk + P * dv;
    float* os = pq + P * dv;
    const T* cr = conv + row * A.ldc;
    for (int i = tid; i < 2 * dk; i += nthreads)
      buf[i] = ldf(cr, (size_t)(i < dk ? 0 : A.kv_heads * dk) + (size_t)kvh * dk + (i < dk ? i : i - dk));
    const float v = ldf(cr, (size_t)2 * A.kv_heads * dk + (size_t)h * dv + j);
    const T* pr = proj + row * A.ldp;
    const float a = ldf(pr, A.a_off + h), b = ldf(pr, A.b_off + h);
    const float gate = ldf(pr, (size_t)A.gate_off + (size_t)h * dv + j);
    __syncthreads();
    // every wave sums the squares and q . k for itself, in the same order
    float sq = 0.f, sk = 0.f, qk = 0.f;
    for (int i = lane; i < dk; i += 64) {
      sq = fmaf(qs[i], qs[i], sq);
      sk = fmaf(ks[i], ks[i], sk);
      qk = fmaf(qs[i], ks[i], qk);
    }
    sq = wave_sum(sq), sk = wave_sum(sk), qk = wave_sum(qk);
    const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
    qk *= rq * rk;
    float dk_ = 0.f, dq_ = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = part + e * P;
      if (i < dk) {
        dk_ = fmaf(S[e], ks[i], dk_);
        dq_ = fmaf(S[e], qs[i], dq_);
      }
    }
    if (act) {
      pk[part * dv + j] = dk_;
      pq[part * dv + j] = dq_;
    }
    __syncthreads();
    float Sk = 0.f, Sq = 0.f;
    for (int p = 0; p < P; ++p) {
      Sk += pk[p * dv + j];
      Sq += pq[p * dv + j];
    }
    Sk *= rk, Sq *= rq;
    const float z = a + dtb;
    const float sp = z > 20.f ? z : log1pf(expf(z));
    const float g = expf(-decay_rate * sp);
    const float beta = 1.0f / (1.0f + expf(-b));
    const float u = beta * (v - g * Sk);
    const float o = fmaf(g, Sq, qk * u);
    const float ku = u * rk;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = part + e * P;
      if (i < dk) S[e] = fmaf(ks[i], ku, g * S[e]);
    }
    if (part == 0) os[j] = o;
    __syncthreads();
    float ss = 0.f;
    for (int i = lane; i < dv; i += 64) ss = fmaf(os[i], os[i], ss);
    ss = wave_sum(ss);
    if (part == 0) {
      stf(out + row * A.ldo, (size_t)h * dv + j, o * norm_scale(ss, dv, A.eps) * gain * silu_f(gate));
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = part + e * P;
    if (act && i < dk) S_at[(size_t)i * dv + j] = S[e];
  }
}

extern "C" int jllm_gated_delta(const void* qkv, int ldc, const void* proj, int ldp, int gate_off, int a_off, int b_off,
                                int dtype, const void* a_log, const void* dt_bias, const void* gain, int w_dtype, float* state,
                                void* out, int ldo, const int* row_req, const int* state_slots, int n_rows, int n_requests,
                                int heads, int kv_heads, int dk, int dv, float eps, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || heads > 65535) JLLM_FAIL("gated_delta: %d heads over %d key heads", heads, kv_heads);
  if (dk <= 0 || dv <= 0 || dv > 1024) JLLM_FAIL("gated_delta: key size %d, value size %d (values up to 1024 are taken)", dk, dv);
  if (n_requests <= 0 || n_requests > n_rows) JLLM_FAIL("gated_delta: %d requests in %d rows", n_requests, n_rows);
  if (ldc < 2 * kv_heads * dk + heads * dv || ldo < heads * dv || ldp < gate_off + heads * dv || ldp < a_off + heads || ldp < b_off + heads)
    JLLM_FAIL("gated_delta: short rows");
  // as many parts of the key rows as keep a workgroup near 256 threads; more where a thread would hold too many
  int parts = 1;
  while (parts * 2 * dv <= 256 && parts * 2 <= dk && parts < GDR_MAX_PARTS) parts *= 2;
  while ((dk + parts - 1) / parts > 64 && parts * 2 * dv <= 1024 && parts < GDR_MAX_PARTS) parts *= 2;
  const int per_thread = (dk + parts - 1) / parts;
  if (per_thread > 64) JLLM_FAIL("gated_delta: a state of %d x %d per head does not fit a workgroup's registers", dk, dv);
  GdrArgs A{qkv, ldc, proj, ldp, gate_off, a_off, b_off, a_log, dt_bias, gain, state, out, ldo, row_req, state_slots,
            n_rows, heads, kv_heads, dk, dv, parts, eps};
  const size_t smem = (size_t)2 * (2 * dk + 2 * parts * dv + dv) * sizeof(float);
  if (smem > 64 * 1024) JLLM_FAIL("gated_delta: %zu bytes of LDS for key size %d, value size %d", smem, dk, dv);
  dim3 grid(n_requests, heads);
  const int threads = (dv * parts + 63) / 64 * 64;
#define GDR_LAUNCH(E) gated_delta_kernel<T, TW, E><<<grid, threads, smem, stream>>>(A)
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      if (per_thread <= 8)
        GDR_LAUNCH(8);
      else if (per_thread <= 16)
        GDR_LAUNCH(16);
      else if (per_thread <= 32)
        GDR_LAUNCH(32);
      else
        GDR_LAUNCH(64);
    })
  })
#undef GDR_LAUNCH
  JLLM_CHECK_LAUNCH("gated_delta");
  return 0;
}
