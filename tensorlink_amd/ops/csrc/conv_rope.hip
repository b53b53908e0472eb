// Short causal convolution over time + rotate-half positions + page
// scatter in one kernel (gfx950).
//
// Columns [col, col + n_heads*D) of the fused projection (bf16 or fp32)
// pass a per-channel convolution with K taps,
//     y_t[c] = sum_j taps[c][j] u_(t-K+1+j)[c]  (+ bias[c], silu),
// whose inputs before the step's first token come from the sequence's
// history [slots, K-1, N] (fp32; zeros when the sequence has no cached
// tokens). The first rot_dims dimensions of every head are then rotated by
// the token's position: pair (i, i + rot_dims/2), angle pos * freqs[i]
// formed in double, cos and sin times `mult`. The first n_heads -
// pool_heads heads are written densely in fp32 (queries, or the inputs of a
// recurrence); the last pool_heads heads go to the tokens' page rows of
// `pool` (rotated) and, when given, of `raw_pool` (the unrotated
// convolution output: a value pool that shares the key projection).
//
// One block per tile of <= TILE tokens of one sequence (with few tiles the
// work items of a tile are spread over several blocks). A work item is a
// rotated pair or a single unrotated channel, so rotation needs no
// exchange between threads; the tile's cos/sin table is built once in LDS
// and shared by all heads. TILE >= K-1, so only the block of a portion's
// first tile reads the old history; the same block writes the new one
// after a barrier.

#include "common.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int TILE = 8;
constexpr int PAGE = 128;
constexpr int MAXK = 9;

template <typename T> DEVINLINE float ldf(const T* p, int64_t i);
template <> DEVINLINE float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <> DEVINLINE float ldf<bf16>(const bf16* p, int64_t i) { return bf2f(p[i]); }
template <typename T> DEVINLINE void stf(T* p, int64_t i, float v);
template <> DEVINLINE void stf<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> DEVINLINE void stf<bf16>(bf16* p, int64_t i, float v) { p[i] = f2bf(v); }

DEVINLINE float silu_f(float z) { return z / (1.f + expf(-z)); }

template <typename T>
__global__ __launch_bounds__(BLOCK) void conv_rope_rows_kernel(
    const T* __restrict__ src, int ld, int col, int n_heads, int D,
    const float* __restrict__ taps, const float* __restrict__ bias,
    int act_silu, float* __restrict__ hist, int K, int rot_dims,
    const double* __restrict__ freqs, float mult,
    const int* __restrict__ tiles, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ pos0,
    const int* __restrict__ table, int P, float* __restrict__ out,
    T* __restrict__ pool, T* __restrict__ raw_pool, int pool_heads) {
  extern __shared__ float cs[];     // [TILE][half][2]
  const int seq = tiles[blockIdx.x * 4 + 0];
  const int tok0 = tiles[blockIdx.x * 4 + 1];
  const int n = tiles[blockIdx.x * 4 + 2];
  const int p0 = tiles[blockIdx.x * 4 + 3];
  const int c0 = cu[seq], ntot = cu[seq + 1] - c0;
  const bool first = tok0 == c0;
  const bool fresh = pos0[seq] == 0;
  const int half = rot_dims / 2;
  const int N = n_heads * D;
  const int dense = n_heads - pool_heads;
  for (int i = threadIdx.x; i < n * half; i += BLOCK) {
    const int t = i / half, p = i - t * half;
    const double ang = (double)(p0 + t) * freqs[p];
    cs[i * 2 + 0] = (float)(cos(ang) * (double)mult);
    cs[i * 2 + 1] = (float)(sin(ang) * (double)mult);
  }
  __syncthreads();
  float* hs = hist + (int64_t)slots[seq] * (K - 1) * N;
  const int iph = D - half;         // work items per head
  const int* tab = table + (int64_t)seq * P;
  // few tiles (decoding): the work items are spread over gridDim.y blocks
  const int e_first = blockIdx.y * BLOCK + threadIdx.x;
  const int e_step = gridDim.y * BLOCK;
  for (int e = e_first; e < n_heads * iph; e += e_step) {
    const int hd = e / iph, r = e - hd * iph;
    const bool pair = r < half;
    const int d0 = pair ? r : r + half;
    const int ch0 = hd * D + d0, ch1 = ch0 + half;
    // taps and the sliding window are aligned at the END of fixed-size
    // arrays (leading entries zero), so every index is static
    float w0[MAXK], w1[MAXK], u0[MAXK - 1], u1[MAXK - 1];
#pragma unroll
    for (int m = 0; m < MAXK; ++m) {
      const int j = m - (MAXK - K);
      w0[m] = j >= 0 ? taps[(int64_t)ch0 * K + j] : 0.f;
      w1[m] = (pair && j >= 0) ? taps[(int64_t)ch1 * K + j] : 0.f;
    }
#pragma unroll
    for (int m = 0; m < MAXK - 1; ++m) {
      const int j = m - (MAXK - K);
      float a = 0.f, b = 0.f;
      if (j >= 0) {
        const int row = tok0 - (K - 1) + j;
        if (row >= c0) {
          a = ldf<T>(src, (int64_t)row * ld + col + ch0);
          if (pair) b = ldf<T>(src, (int64_t)row * ld + col + ch1);
        } else if (!fresh) {
          const int64_t hr = (int64_t)(K - 1 + row - c0) * N;
          a = hs[hr + ch0];
          if (pair) b = hs[hr + ch1];
        }
      }
      u0[m] = a;
      u1[m] = b;
    }
    const float b0 = bias ? bias[ch0] : 0.f;
    const float b1 = (bias && pair) ? bias[ch1] : 0.f;
    for (int i = 0; i < n; ++i) {
      const int64_t ro = (int64_t)(tok0 + i) * ld + col;
      const float c0v = ldf<T>(src, ro + ch0);
      const float c1v = pair ? ldf<T>(src, ro + ch1) : 0.f;
      float a0 = b0 + w0[MAXK - 1] * c0v, a1 = b1 + w1[MAXK - 1] * c1v;
#pragma unroll
      for (int m = 0; m < MAXK - 1; ++m) {
        a0 += w0[m] * u0[m];
        a1 += w1[m] * u1[m];
      }
#pragma unroll
      for (int m = 0; m < MAXK - 2; ++m) {
        u0[m] = u0[m + 1];
        u1[m] = u1[m + 1];
      }
      u0[MAXK - 2] = c0v;
      u1[MAXK - 2] = c1v;
      if (act_silu) {
        a0 = silu_f(a0);
        a1 = silu_f(a1);
      }
      float x0 = a0, x1 = a1;
      if (pair) {
        const float c = cs[(i * half + r) * 2], s = cs[(i * half + r) * 2 + 1];
        x0 = a0 * c - a1 * s;
        x1 = a1 * c + a0 * s;
      }
      const int tok = tok0 + i;
      if (hd < dense) {
        float* o = out + (int64_t)tok * dense * D + hd * D;
        o[d0] = x0;
        if (pair) o[d0 + half] = x1;
      } else {
        const int pos = p0 + i;
        const int64_t prow =
            (((int64_t)tab[pos / PAGE] * pool_heads + (hd - dense)) * PAGE +
             (pos % PAGE)) * D;
        stf<T>(pool, prow + d0, x0);
        if (pair) stf<T>(pool, prow + d0 + half, x1);
        if (raw_pool) {
          stf<T>(raw_pool, prow + d0, a0);
          if (pair) stf<T>(raw_pool, prow + d0 + half, a1);
        }
      }
    }
  }
  if (!first || K <= 1) return;
  __syncthreads();       // every read of the old history is done
  // a block updates the channels of its own work items
  for (int e = e_first; e < n_heads * iph; e += e_step) {
    const int hd = e / iph, r = e - hd * iph;
    const bool pair = r < half;
    const int ch0 = hd * D + (pair ? r : r + half);
    for (int k = 0; k < (pair ? 2 : 1); ++k) {
      const int c = ch0 + k * half;
      for (int r2 = 0; r2 < K - 1; ++r2) {
        const int rr = ntot - (K - 1) + r2;
        float v;
        if (rr >= 0)
          v = ldf<T>(src, (int64_t)(c0 + rr) * ld + col + c);
        else    // ascending: source index r2 + ntot is not yet overwritten
          v = fresh ? 0.f : hs[(int64_t)(r2 + ntot) * N + c];
        hs[(int64_t)r2 * N + c] = v;
      }
    }
  }
}

}  // namespace

extern "C" {

int tl_conv_rope_tile() { return TILE; }

// returns 0 on success, 1 if the shape is outside what the kernel serves
int tl_conv_rope_rows(const void* src, int ld, int col, int n_heads, int D,
                      const void* taps, const void* bias, int act_silu,
                      void* hist, int K, int rot_dims, const void* freqs,
                      float mult, const void* tiles, int n_tiles,
                      const void* cu, const void* slots, const void* pos0,
                      const void* table, int P, void* out, void* pool,
                      void* raw_pool, int pool_heads, int is_f32,
                      hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (K < 1 || K > MAXK || K - 1 > TILE || (rot_dims & 1) || rot_dims > D)
    return 1;
  const size_t smem = sizeof(float) * 2 * TILE * (size_t)(rot_dims / 2);
  if (smem > 64 * 1024) return 1;
  const int items = n_heads * (D - rot_dims / 2);
  const int gy = n_tiles >= 512 ? 1 : min(16, max(1, (items + BLOCK - 1) / BLOCK));
  const dim3 grid(n_tiles, gy);
  if (is_f32)
    hipLaunchKernelGGL(conv_rope_rows_kernel<float>, grid,
                       dim3(BLOCK), smem, stream, (const float*)src, ld, col,
                       n_heads, D, (const float*)taps, (const float*)bias,
                       act_silu, (float*)hist, K, rot_dims,
                       (const double*)freqs, mult, (const int*)tiles,
                       (const int*)cu, (const int*)slots, (const int*)pos0,
                       (const int*)table, P, (float*)out, (float*)pool,
                       (float*)raw_pool, pool_heads);
  else
    hipLaunchKernelGGL(conv_rope_rows_kernel<bf16>, grid,
                       dim3(BLOCK), smem, stream, (const bf16*)src, ld, col,
                       n_heads, D, (const float*)taps, (const float*)bias,
                       act_silu, (float*)hist, K, rot_dims,
                       (const double*)freqs, mult, (const int*)tiles,
                       (const int*)cu, (const int*)slots, (const int*)pos0,
                       (const int*)table, P, (float*)out, (bf16*)pool,
                       (bf16*)raw_pool, pool_heads);
  return 0;
}

}  // extern "C"
