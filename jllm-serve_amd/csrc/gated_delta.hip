// A gated delta rule with short causal convolutions in front: a recurrent mixer whose per-request state is one matrix
// per head (fp32) and the last taps - 1 inputs of every convolved channel. fp32 or bf16 activations, all arithmetic in
// fp32. A request's rows of a step are consecutive and in order (row_req ascends), so every kernel finds a request's
// rows in the step by itself and the same launches serve portions of prompts, single rows and steps of fixed size.
//
//   short_conv_silu      y[t, c] = silu(sum_j taps[c, K - 1 - j] x[t - j, c]); inputs before the step's first row of a
//                        request come from that request's state, inputs before position 0 are the state's zeros
//   short_conv_advance   the state's K - 1 inputs per channel move on by the request's rows of this step
//   gated_delta          token by token, with S [dk, dv] in registers:
//                          q <- q / sqrt(sum q^2 + 1e-6) / sqrt(dk), k <- k / sqrt(sum k^2 + 1e-6)
//                          beta = sigmoid(b), g = exp(-exp(A_log) * softplus(a + dt_bias))
//                          S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//                        computed as  S^T k and S^T q of the old S in one pass, o = g S^T q + (k . q) u.
//                        The columns of S never meet: column j only needs v[j], so a workgroup is ONE wave that owns 16
//                        value columns of one head of one request (4 lanes per column, a quarter of the key rows
//                        each) and walks the request's rows without a barrier; a step of one request and 16 heads of
//                        128 x 128 is 128 such waves. The read-out o goes out raw in fp32; the heads' norm, gain and
//                        gate need all columns of a head and are the finishing kernel's (attention_dv.hip).
#include <math.h>

#include "common.h"

#define CONV_MAX_TAPS 16
#define GDR_COLS 16   // value columns of a wave
#define GDR_PARTS 4   // lanes per column: each owns a quarter of the key rows

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
  const void* proj;  // [rows, ldp]: the projection's row, which holds a and b (heads each) at their offsets
  int ldp, a_off, b_off;
  const void* a_log;    // [heads]
  const void* dt_bias;  // [heads]
  float* state;         // [slots, heads, dk, dv]
  float* out;           // [rows, ldo]: heads x dv, the raw read-out
  int ldo;
  const int* row_req;
  const int* state_slots;
  int n_rows, heads, kv_heads, dk, dv;
};

// what a lane needs of one row: its quarter of q and k, its column's v, the head's a and b
template <typename T, int E>
struct GdrRow {
  float q[E], k[E], v, a, b;
  __device__ __forceinline__ void load(const GdrArgs& A, size_t row, int kvh, int h, int i0, int col, bool col_on) {
    const T* cr = (const T*)A.qkv + row * A.ldc;
    const T* qr = cr + (size_t)kvh * A.dk;
    const T* kr = cr + (size_t)(A.kv_heads + kvh) * A.dk;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const bool on = i0 + e < A.dk;
      q[e] = on ? ldf(qr, i0 + e) : 0.f;
      k[e] = on ? ldf(kr, i0 + e) : 0.f;
    }
    v = col_on ? ldf(cr, (size_t)2 * A.kv_heads * A.dk + (size_t)h * A.dv + col) : 0.f;
    const T* pr = (const T*)A.proj + row * A.ldp;
    a = ldf(pr, A.a_off + h);
    b = ldf(pr, A.b_off + h);
  }
};

__device__ __forceinline__ float parts_sum(float v) {  // over the four lanes of a column, the same in all of them
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// lane = part * 16 + c: column blockIdx.z * 16 + c, key rows part * E .. + E
template <typename T, typename TW, int E, bool AHEAD>
__global__ __launch_bounds__(64) void gated_delta_kernel(GdrArgs A) {
  const int lane = threadIdx.x;
  const int c = lane & (GDR_COLS - 1), part = lane / GDR_COLS;
  const int req = blockIdx.x, h = blockIdx.y;
  const int col = blockIdx.z * GDR_COLS + c;
  const bool col_on = col < A.dv;
  int lo, n;
  rows_of_request(A.row_req, A.n_rows, req, lo, n);
  if (n == 0) return;
  const int kvh = h / (A.heads / A.kv_heads);
  const int i0 = part * E;
  float* S_at = A.state + ((size_t)A.state_slots[req] * A.heads + h) * A.dk * A.dv;
  float S[E];
#pragma unroll
  for (int e = 0; e < E; ++e) S[e] = (col_on && i0 + e < A.dk) ? S_at[(size_t)(i0 + e) * A.dv + col] : 0.f;
  const float decay_rate = expf(ldf((const TW*)A.a_log, h));
  const float dtb = ldf((const TW*)A.dt_bias, h);
  const float q_scale = 1.0f / sqrtf((float)A.dk);
  GdrRow<T, E> cur, nxt;
  cur.load(A, (size_t)lo, kvh, h, i0, col, col_on);
  for (int r = 0; r < n; ++r) {
    if (AHEAD && r + 1 < n) nxt.load(A, (size_t)(lo + r + 1), kvh, h, i0, col, col_on);  // in flight under this row's sums
    float sq = 0.f, sk = 0.f, qk = 0.f, dk_ = 0.f, dq_ = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      sq = fmaf(cur.q[e], cur.q[e], sq);
      sk = fmaf(cur.k[e], cur.k[e], sk);
      qk = fmaf(cur.q[e], cur.k[e], qk);
      dk_ = fmaf(S[e], cur.k[e], dk_);
      dq_ = fmaf(S[e], cur.q[e], dq_);
    }
    sq = parts_sum(sq), sk = parts_sum(sk), qk = parts_sum(qk), dk_ = parts_sum(dk_), dq_ = parts_sum(dq_);
    const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
    const float z = cur.a + dtb;
    const float sp = z > 20.f ? z : log1pf(expf(z));
    const float g = expf(-decay_rate * sp);
    const float beta = 1.0f / (1.0f + expf(-cur.b));
    const float u = beta * (cur.v - g * (dk_ * rk));
    const float o = fmaf(g, dq_ * rq, qk * rq * rk * u);
    const float ku = u * rk;
#pragma unroll
    for (int e = 0; e < E; ++e) S[e] = fmaf(cur.k[e], ku, g * S[e]);
    if (part == 0 && col_on) A.out[(size_t)(lo + r) * A.ldo + (size_t)h * A.dv + col] = o;
    if (AHEAD)
      cur = nxt;
    else if (r + 1 < n)
      cur.load(A, (size_t)(lo + r + 1), kvh, h, i0, col, col_on);
  }
#pragma unroll
  for (int e = 0; e < E; ++e)
    if (col_on && i0 + e < A.dk) S_at[(size_t)(i0 + e) * A.dv + col] = S[e];
}

extern "C" int jllm_gated_delta(const void* qkv, int ldc, const void* proj, int ldp, int a_off, int b_off, int dtype,
                                const void* a_log, const void* dt_bias, int w_dtype, float* state, float* out, int ldo,
                                const int* row_req, const int* state_slots, int n_rows, int n_requests, int heads,
                                int kv_heads, int dk, int dv, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || heads > 65535) JLLM_FAIL("gated_delta: %d heads over %d key heads", heads, kv_heads);
  if (dk <= 0 || dk > GDR_PARTS * 64 || dv <= 0 || dv > GDR_COLS * 65535) JLLM_FAIL("gated_delta: key size %d (1..%d are taken), value size %d", dk, GDR_PARTS * 64, dv);
  if (n_requests <= 0 || n_requests > n_rows) JLLM_FAIL("gated_delta: %d requests in %d rows", n_requests, n_rows);
  if (ldc < 2 * kv_heads * dk + heads * dv || ldo < heads * dv || ldp < a_off + heads || ldp < b_off + heads || a_off < 0 || b_off < 0)
    JLLM_FAIL("gated_delta: short rows");
  GdrArgs A{qkv, ldc, proj, ldp, a_off, b_off, a_log, dt_bias, state, out, ldo, row_req, state_slots, n_rows, heads, kv_heads, dk, dv};
  dim3 grid(n_requests, heads, (dv + GDR_COLS - 1) / GDR_COLS);
  const int per_lane = (dk + GDR_PARTS - 1) / GDR_PARTS;
#define GDR_LAUNCH(E, AHEAD) gated_delta_kernel<T, TW, E, AHEAD><<<grid, 64, 0, stream>>>(A)
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      if (per_lane <= 8)
        GDR_LAUNCH(8, true);
      else if (per_lane <= 16)
        GDR_LAUNCH(16, true);
      else if (per_lane <= 32)
        GDR_LAUNCH(32, true);
      else
        GDR_LAUNCH(64, false);
    })
  })
#undef GDR_LAUNCH
  JLLM_CHECK_LAUNCH("gated_delta");
  return 0;
}
