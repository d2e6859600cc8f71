// Latent attention on the matrix cores, bf16: portions of prompts and single decoded rows through one kernel.
//
// All heads of a row attend over the same cached rows (Dk = R + Dr numbers per position, the first R of which are also
// the values), so the query vectors of many heads and rows share every key they read. A workgroup takes 64 query
// vectors of one run of rows of one request (HB heads x 64 / HB consecutive rows). It has eight waves: waves w and w + 4
// own the same 16 query vectors and both compute their scores and softmax, but each keeps only one half of the latent's
// accumulators (a 512-wide latent is 128 registers per lane; one wave holding all of it and its queries left no
// registers to have LDS reads in flight, and timestamps showed every fragment read's latency standing in front of its
// product: 2,900 cycles for the 18 score products of 16 keys). The workgroup
// walks the keys its rows can see in blocks of 64 aligned to absolute positions, and stages each block once in LDS as
// it lies in the cache (two buffers take turns: the next block travels while this one is multiplied). Per 16 keys a wave computes
//   S^T = K . Q^T   (MFMA 16x16x32; K fragments from LDS, Q^T in registers): a lane then holds four keys' scores of
//                   ONE query vector, so masks (causal and window, per query vector), maximum and sum need only two
//                   shuffles over the lane groups;
//   O^T += V^T . P^T (MFMA 16x16x16): those probabilities, packed to bf16, already are the B operand, and V^T is read
//                   from the staged block with the transposing LDS load.
// The running maximum moves only when it grows by more than 8 (probabilities stay below e^8, exact in fp32 sums).
// exp(sink) of the query vector's head joins the denominator at the end. Scores, softmax and sums are fp32.
//
// The runs come from the step's plan: (request, first row, rows <= 16, -) per tile; positions are read per row.
//
// Steps of single rows (decoding) with few workgroups cut every row's keys into absolute ranges of `split` keys over
// gridDim.z: a workgroup then leaves maximum, sum and unnormalised sums per query vector, and a second kernel merges
// the ranges in ascending order, adds the sink and normalises.
#include <math.h>

#include "common.h"
#include "mfma.h"

#define LM_WAVES 8
#define LM_QW 4  // waves with query vectors of their own; waves 4..7 repeat them for the other half of the latent
#define LM_KEYS 64
#define LM_TILE_ROWS 16

__device__ __forceinline__ float lm_exp_diff(float a, float b) { return a == -INFINITY ? 0.f : __expf(a - b); }

// RT: 16-dim blocks of the latent the accumulators hold at most; DKS: 32-dim steps of a key row at most
template <int RT, int DKS>
__global__ __launch_bounds__(LM_WAVES * 64) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ qa, int ldq, bf16_t* __restrict__ out, int ldo, const bf16_t* __restrict__ cache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tiles,
    const int* __restrict__ positions, int H, int R, int Dk, int page_size, int window, float scale,
    const float* __restrict__ sink, int HB, int n_hb, int LD, int split, float* __restrict__ part) {
  extern __shared__ __align__(16) unsigned char lm_smem[];
  bf16_t* Ks = (bf16_t*)lm_smem;  // [2][LM_KEYS][LD]
  const int tile = blockIdx.x;
  const int req = tiles[4 * tile], row0 = tiles[4 * tile + 1], rows = tiles[4 * tile + 2];
  const int RW = 64 / HB;
  const int rg = blockIdx.y / n_hb, hb = blockIdx.y % n_hb;
  const int r_lo = rg * RW;
  if (r_lo >= rows) return;
  const int r_hi = min(rows, r_lo + RW) - 1;
  const int p_lo = positions[row0 + r_lo];
  const int p_hi = p_lo + (r_hi - r_lo);
  int kb = window > 0 ? max(0, p_lo + 1 - window) : 0;
  int ke = p_hi;
  if (split > 0) {  // single rows: this workgroup's range of the row's keys
    const int s0 = kb / split + (int)blockIdx.z;
    kb = max(kb, s0 * split);
    ke = min(ke, s0 * split + split - 1);
    if (kb > ke) return;
  }
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int sub = lane & 15, q4 = lane >> 4;
  // A single row of at most 16 heads is 16 query vectors, one wave's worth: then all four waves take the same query
  // vectors and every fourth group of 16 keys each, and merge at the end in the order of the waves.
  const bool kpar = r_hi == r_lo && HB <= 16;
  const int qwave = wave & (LM_QW - 1), rhalf = wave / LM_QW;
  const int v = kpar ? sub : qwave * 16 + sub;
  const int my_r = r_lo + v / HB, my_h = hb * HB + v % HB;
  const bool live = my_r <= r_hi && my_h < H;
  const int my_pos = p_lo + v / HB;
  const int my_first = window > 0 ? max(0, my_pos + 1 - window) : 0;
  // the keys this wave's rows can see (a wave without a live query vector only helps to load)
  const int wr_lo = kpar ? r_lo : r_lo + (qwave * 16) / HB, wr_hi = kpar ? r_lo : min(r_hi, r_lo + (qwave * 16 + 15) / HB);
  const bool wave_live = wr_lo <= r_hi;
  const int w_lo = window > 0 ? max(0, p_lo + (wr_lo - r_lo) + 1 - window) : 0;
  const int w_hi = p_lo + (wr_hi - r_lo);  // (with a split the loop's own bounds narrow these further)
  const int dks = (Dk + 31) >> 5, r16 = R >> 4;
  constexpr int RTH = (RT + 1) / 2;  // accumulators of one wave: its half of the latent's 16-dim blocks
  const int j_lo = rhalf ? (r16 + 1) / 2 : 0, nj = rhalf ? r16 - (r16 + 1) / 2 : (r16 + 1) / 2;
  const int psh = __builtin_ctz(page_size);
  const int* tbl = block_table + (size_t)req * max_blocks;

  u32x4 qf[DKS];
  {
    const bf16_t* qrow = qa + (size_t)(row0 + min(my_r, r_hi)) * ldq + (size_t)min(my_h, H - 1) * Dk;
#pragma unroll
    for (int j = 0; j < DKS; ++j) {
      const int d = 32 * j + 8 * q4;
      qf[j] = (live && j < dks && d < Dk) ? *(const u32x4*)(qrow + d) : u32x4{0u, 0u, 0u, 0u};
    }
  }
  floatx4 acc[RTH];
#pragma unroll
  for (int j = 0; j < RTH; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m1 = -INFINITY, l1 = 0.f;
  // A block of 64 keys goes global -> registers -> LDS. All of a thread's pieces are requested together (first their
  // table entries, then the rows: two latencies a block, not two per piece), and the next block's are requested before
  // this block is multiplied, into the other of two LDS buffers: one barrier per block.
  // eight threads to a key row (512 threads, 64 rows): a thread's pieces are 16 bytes at (tid % 8) * 16 + 128 i of its
  // row: one table entry and one address per block
  constexpr int CPT = (DKS + 1) / 2;
  static_assert(LM_WAVES * 64 == 8 * LM_KEYS, "eight threads stage a key row");
  uint4 staged[CPT];
  const int srow = threadIdx.x >> 3, scol = (threadIdx.x & 7) * 8;
  auto fetch = [&](int blk) {
    const int key = min(max(blk * LM_KEYS + srow, kb), ke);  // a key outside the range is masked below and reads one inside it
    const bf16_t* src = cache + ((((size_t)tbl[key >> psh]) << psh) + (key & (page_size - 1))) * Dk + scol;
#pragma unroll
    for (int i = 0; i < CPT; ++i) staged[i] = (scol + 64 * i < Dk) ? *(const uint4*)(src + 64 * i) : uint4{0u, 0u, 0u, 0u};
  };
  auto put = [&](bf16_t* buf) {
    bf16_t* dst = buf + srow * LD + scol;
#pragma unroll
    for (int i = 0; i < CPT; ++i)
      if (scol + 64 * i < dks * 32) *(uint4*)(dst + 64 * i) = staged[i];
  };
  const int blk_last = ke >> 6;
  int cur = 0;
  fetch(kb >> 6);
  put(Ks);
  __syncthreads();
  for (int blk = kb >> 6; blk <= blk_last; ++blk) {
    const int c0 = blk * LM_KEYS;
    const bf16_t* Kb = Ks + (size_t)cur * LM_KEYS * LD;
    if (blk < blk_last) fetch(blk + 1);
    if (wave_live) {
#pragma unroll 1
      for (int st = 0; st < LM_KEYS / 16; ++st) {
        const int k0 = c0 + st * 16;
        if (k0 + 15 < w_lo || k0 > w_hi) continue;  // none of these keys is seen by a row of this wave
        if (kpar && st != qwave) continue;           // another wave's keys
        floatx4 sc = floatx4{0.f, 0.f, 0.f, 0.f}, sc2 = floatx4{0.f, 0.f, 0.f, 0.f};  // two chains of dependent MFMAs
        const bf16_t* krow = Kb + (st * 16 + sub) * LD + 8 * q4;
#pragma unroll
        for (int j = 0; j < DKS; j += 2) {
          if (j < dks) sc = mfma16(*(const u32x4*)(krow + 32 * j), qf[j], sc);
          if (j + 1 < DKS && j + 1 < dks) sc2 = mfma16(*(const u32x4*)(krow + 32 * (j + 1)), qf[j + 1 < DKS ? j + 1 : j], sc2);
        }
        sc += sc2;
        float z[4];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = k0 + 4 * q4 + i;
          z[i] = (live && key >= my_first && key <= my_pos && key >= kb && key <= ke) ? sc[i] * scale : -INFINITY;
          mx = fmaxf(mx, z[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        if (mx > m1 + 8.0f) {  // also the first visible key (m1 = -inf)
          const float alpha = lm_exp_diff(m1, mx);
          l1 *= alpha;
#pragma unroll
          for (int j = 0; j < RTH; ++j) acc[j] *= alpha;
          m1 = mx;
        }
        float p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[i] = lm_exp_diff(z[i], m1);
          l1 += p[i];
        }
        const u32x2 pb = u32x2{pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3])};
        const bf16_t* v_tr = Kb + (st * 16 + 4 * q4 + (sub >> 2)) * LD + 4 * (sub & 3);
#pragma unroll
        for (int j = 0; j < RTH; ++j)
          if (j < nj) acc[j] = mfma16k16(lds_read_tr16(v_tr + 16 * (j_lo + j)), pb, acc[j]);
      }
    }
    if (blk < blk_last) put(Ks + (size_t)(cur ^ 1) * LM_KEYS * LD);
    __syncthreads();  // the other buffer is whole, and everyone is done with this one
    cur ^= 1;
  }
  l1 += __shfl_xor(l1, 16, 64);
  l1 += __shfl_xor(l1, 32, 64);
  if (kpar) {  // the loop's last barrier has passed: the key buffers now carry the merge
    constexpr int MS = 2 + 4 * RTH;
    float* mrg = (float*)lm_smem + (size_t)rhalf * (LM_QW - 1) * 64 * MS;  // [2][LM_QW - 1][64][MS]
    if (qwave > 0) {
      float* d = mrg + (size_t)((qwave - 1) * 64 + lane) * MS;
      d[0] = m1, d[1] = l1;
#pragma unroll
      for (int j = 0; j < RTH; ++j)
        if (j < nj) {
#pragma unroll
          for (int i = 0; i < 4; ++i) d[2 + 4 * j + i] = acc[j][i];
        }
    }
    __syncthreads();
    if (qwave > 0) return;
#pragma unroll 1
    for (int w = 0; w < LM_QW - 1; ++w) {
      const float* src = mrg + (size_t)(w * 64 + lane) * MS;
      const float om = src[0], ol = src[1];
      const float mn = fmaxf(m1, om);
      const float a = lm_exp_diff(m1, mn), b = lm_exp_diff(om, mn);
      l1 = l1 * a + ol * b;
#pragma unroll
      for (int j = 0; j < RTH; ++j)
        if (j < nj) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[j][i] = acc[j][i] * a + src[2 + 4 * j + i] * b;
        }
      m1 = mn;
    }
  }
  if (!live) return;
  if (split > 0) {
    float* dst = part + (((size_t)(row0 + my_r) * H + my_h) * gridDim.z + blockIdx.z) * (R + 4);  // R sums, maximum, sum
    if (q4 == 0 && rhalf == 0) dst[R] = m1, dst[R + 1] = l1;
#pragma unroll
    for (int j = 0; j < RTH; ++j)
      if (j < nj) *(floatx4*)(dst + 16 * (j_lo + j) + 4 * q4) = acc[j];
    return;
  }
  float ca = 1.0f;
  if (sink) {
    const float sk = sink[my_h];
    const float mn = fmaxf(m1, sk);
    ca = lm_exp_diff(m1, mn);
    l1 = l1 * ca + __expf(sk - mn);
  }
  const float inv = ca / l1;
  bf16_t* o = out + (size_t)(row0 + my_r) * ldo + (size_t)my_h * R + 4 * q4;
#pragma unroll
  for (int j = 0; j < RTH; ++j)
    if (j < nj)
      *(u32x2*)(o + 16 * (j_lo + j)) = u32x2{pack_bf16(acc[j][0] * inv, acc[j][1] * inv), pack_bf16(acc[j][2] * inv, acc[j][3] * inv)};
}

// merges the key ranges of one (row, head); four waves per (row, head), a thread owns dims tid and tid + 256. Lane z of
// every wave first takes range z's maximum and sum (all ranges at once: n_z <= 64), the wave agrees on the overall
// maximum and every range's weight, and then the weighted sums are added in ascending order of the ranges with eight
// ranges' loads in flight.
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(const float* __restrict__ part, const int* __restrict__ positions,
                                                                   int H, int R, int window, int split, int n_z,
                                                                   const float* __restrict__ sink, bf16_t* __restrict__ out,
                                                                   int ldo) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63;
  const int pos = positions[t];
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  const int s0 = first / split;
  const int n_valid = min(n_z, pos / split - s0 + 1);  // the ranges that hold keys of this row
  const float* base = part + ((size_t)t * H + h) * n_z * (R + 4);
  float pm = -INFINITY, pl = 0.f;
  if (lane < n_valid) pm = base[(size_t)lane * (R + 4) + R], pl = base[(size_t)lane * (R + 4) + R + 1];
  float m = wave_max(pm);
  const float sk = sink ? sink[h] : -INFINITY;
  m = fmaxf(m, sk);
  const float wz = lm_exp_diff(pm, m);
  float l = wave_sum(pl * wz) + (sink ? __expf(sk - m) : 0.f);
  float acc[2] = {0.f, 0.f};  // R <= 512
#pragma unroll 8
  for (int z = 0; z < n_valid; ++z) {
    const float w = __shfl(wz, z, 64);
    const float* src = base + (size_t)z * (R + 4);
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int d = threadIdx.x + 256 * a;
      if (d < R) acc[a] = fmaf(src[d], w, acc[a]);
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int d = threadIdx.x + 256 * a;
    if (d < R) stf(out + (size_t)t * ldo + (size_t)h * R, d, acc[a] * inv);
  }
}

template <int RT, int DKS>
static int lm_launch(dim3 grid, size_t smem, hipStream_t stream, const void* qa, int ldq, void* out, int ldo, const void* cache,
                     const int* block_table, int max_blocks, const int* tiles, const int* positions, int H, int R, int Dk,
                     int page_size, int window, float scale, const float* sink, int HB, int n_hb, int LD, int split, float* part) {
  static size_t reserved = 0;
  if (smem > 48 * 1024 && smem > reserved) {
    if (hipFuncSetAttribute((const void*)latent_attention_mfma_kernel<RT, DKS>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
      JLLM_FAIL("latent_attention: cannot reserve %zu bytes of LDS", smem);
    reserved = smem;
  }
  latent_attention_mfma_kernel<RT, DKS><<<grid, LM_WAVES * 64, smem, stream>>>(
      (const bf16_t*)qa, ldq, (bf16_t*)out, ldo, (const bf16_t*)cache, block_table, max_blocks, tiles, positions, H, R, Dk,
      page_size, window, scale, sink, HB, n_hb, LD, split, part);
  return 0;
}

// returns 0 when it ran, 1 when the shape is not one it takes (the caller uses the general kernel), -1 on errors
extern "C" int jllm_latent_attention_bf16(const void* qa, int ldq, void* out, int ldo, const void* cache,
                                          const int* block_table, int max_blocks, const int* tiles, const int* positions,
                                          int n_tiles, int tile_rows, int H, int R, int Dk, int page_size, int window,
                                          float scale, const float* sink, int split, int n_z, float* part,
                                          hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (tile_rows != LM_TILE_ROWS) JLLM_FAIL("latent_attention: runs of %d rows, this kernel takes %d", tile_rows, LM_TILE_ROWS);
  if (H <= 0 || R <= 0 || Dk < R || window < 0 || page_size <= 0 || max_blocks <= 0) JLLM_FAIL("latent_attention: H %d R %d Dk %d window %d", H, R, Dk, window);
  if ((R & 15) || (Dk & 7) || R > 512 || Dk > 640 || (page_size & (page_size - 1))) return 1;
  if (((uintptr_t)qa & 15) || ((uintptr_t)cache & 15) || ((uintptr_t)out & 7) || (ldq & 7) || (ldo & 3)) return 1;
  if (ldq < H * Dk || ldo < H * R) JLLM_FAIL("latent_attention: row strides %d/%d", ldq, ldo);
  int HB = 1;
  while (HB < H && HB < 64) HB <<= 1;
  const int RW = 64 / HB;
  const int n_hb = (H + HB - 1) / HB, n_rg = (LM_TILE_ROWS + RW - 1) / RW;
  if ((long)n_hb * n_rg > 65535) return 1;
  // staged rows lie (Dk rounded up to 32) + pad elements apart, with the stride = 16 mod 64 elements (8 mod 32 words):
  // four consecutive rows of a transposing load then cover all banks
  const int dkp = (Dk + 31) & ~31;
  int LD = dkp + 16;
  while ((LD & 63) != 16) LD += 8;
  const size_t smem = (size_t)2 * LM_KEYS * LD * sizeof(bf16_t);  // two buffers that take turns
  // `split` > 0: every tile is a single row (the caller's promise), whose keys are cut into absolute ranges of `split`
  // keys over n_z workgroups; `part` holds rows x H x n_z x (R + 4) floats
  if (split > 0 && ((split & 63) || n_z < 1 || n_z > 64 || !part)) JLLM_FAIL("latent_attention: ranges of %d keys over %d workgroups", split, n_z);
  dim3 grid(n_tiles, n_hb * (split > 0 ? 1 : n_rg), split > 0 ? n_z : 1);
  int rc;
  if (R <= 64 && dkp <= 128)
    rc = lm_launch<4, 4>(grid, smem, stream, qa, ldq, out, ldo, cache, block_table, max_blocks, tiles, positions, H, R, Dk, page_size, window, scale, sink, HB, n_hb, LD, split, part);
  else if (R <= 128 && dkp <= 256)
    rc = lm_launch<8, 8>(grid, smem, stream, qa, ldq, out, ldo, cache, block_table, max_blocks, tiles, positions, H, R, Dk, page_size, window, scale, sink, HB, n_hb, LD, split, part);
  else
    rc = lm_launch<32, 20>(grid, smem, stream, qa, ldq, out, ldo, cache, block_table, max_blocks, tiles, positions, H, R, Dk, page_size, window, scale, sink, HB, n_hb, LD, split, part);
  if (rc != 0) return rc;
  JLLM_CHECK_LAUNCH("latent_attention");
  if (split > 0) {
    latent_attention_merge_kernel<<<dim3(n_tiles, H), 256, 0, stream>>>(part, positions, H, R, window, split, n_z, sink, (bf16_t*)out, ldo);
    JLLM_CHECK_LAUNCH("latent_attention_merge");
  }
  return 0;
}
