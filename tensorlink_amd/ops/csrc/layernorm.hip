// Row-wise kernels of the layer-norm layered family (gfx950).
//
// The residual X is fp32. A sublayer reads h = layer_norm(X) * w (weight,
// no bias; variance = mean of squared deviations) plus a causal
// per-channel convolution of h over time, and its output is added back
// through a second layer norm.
//
//   tl_layer_norm_rows   plain layer norm of rows (final norm).
//   tl_ln_canon          statistics, norm and the input convolution in one
//                        kernel: one block per tile of <= TILE tokens of one
//                        sequence. The waves first compute mean and 1/std of
//                        the tile's rows and of the K-1 rows before it; every
//                        thread then owns channels and forms
//                        h_t + sum_j taps[c][j] h_(t-K+1+j) from X (cache
//                        hits) and the row statistics. Rows before the
//                        step's first token come from the sequence's history
//                        [slots, K-1, W] (zeros when it has no cached
//                        tokens). TILE >= K-1, so only the block of a
//                        portion's first tile reads the old history; the same
//                        block, after a barrier, writes the new one (the
//                        portion's last K-1 normed rows), so no other block
//                        can see a half-updated history.
//   tl_postln_add        X += layer_norm(u) * w with u = y, or
//                        u = (y/rms(y) * wy + y2/rms(y2) * wy2) / 2 (two
//                        branch outputs); u is staged in LDS.
//   tl_polynorm          c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, N = division
//                        by the row's root mean square.
//   tl_gated_group_rms   u = y * silu(gate); each of `groups` equal parts of
//                        a row divided by its own root mean square; times w.
// Statistics and activations are fp32 whatever the serving dtype.

#include "common.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int NW = BLOCK / WAVE_SIZE;
constexpr int TILE = 8;           // tokens per block of tl_ln_canon
constexpr int MAXROWS = 3 * TILE; // halo + tile + the portion's last rows
constexpr int MAXK = TILE + 1;    // most taps (history of at most TILE rows)

template <typename T> DEVINLINE float ldf(const T* p, int64_t i);
template <> DEVINLINE float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <> DEVINLINE float ldf<bf16>(const bf16* p, int64_t i) { return bf2f(p[i]); }
template <typename T> DEVINLINE void stf(T* p, int64_t i, float v);
template <> DEVINLINE void stf<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> DEVINLINE void stf<bf16>(bf16* p, int64_t i, float v) { p[i] = f2bf(v); }

DEVINLINE float silu_f(float z) { return z / (1.f + expf(-z)); }

// mean and 1/sqrt(var + eps) of one fp32 row, by one wave
DEVINLINE void wave_row_stats(const float* __restrict__ xr, int W, float eps,
                              int lane, float* mean, float* rstd) {
  float s = 0.f;
  for (int c = lane; c < W; c += WAVE_SIZE) s += xr[c];
  const float mu = wave_reduce_sum(s) / (float)W;
  float v = 0.f;
  for (int c = lane; c < W; c += WAVE_SIZE) {
    const float d = xr[c] - mu;
    v += d * d;
  }
  *mean = mu;
  *rstd = 1.0f / sqrtf(wave_reduce_sum(v) / (float)W + eps);
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void layer_norm_rows_kernel(
    const float* __restrict__ x, const float* __restrict__ w,
    T* __restrict__ out, int W, float eps) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  const float* xr = x + row * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += BLOCK) s += xr[c];
  const float mu = block_reduce_sum<NW>(s, red) / (float)W;
  __syncthreads();
  float v = 0.f;
  for (int c = threadIdx.x; c < W; c += BLOCK) {
    const float d = xr[c] - mu;
    v += d * d;
  }
  const float rs = 1.0f / sqrtf(block_reduce_sum<NW>(v, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += BLOCK)
    stf<T>(out, row * W + c, (xr[c] - mu) * rs * w[c]);
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void ln_canon_kernel(
    const float* __restrict__ X, const float* __restrict__ w,
    const float* __restrict__ taps, float* __restrict__ hist,
    const int* __restrict__ tiles, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ pos0,
    T* __restrict__ out, int W, int K, float eps) {
  __shared__ float s_mean[MAXROWS], s_rstd[MAXROWS];
  const int seq = tiles[blockIdx.x * 4 + 0];
  const int tok0 = tiles[blockIdx.x * 4 + 1];
  const int n = tiles[blockIdx.x * 4 + 2];
  const int c0 = cu[seq], ntot = cu[seq + 1] - c0;
  const bool first = tok0 == c0;
  const bool fresh = pos0[seq] == 0;
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int r_lo = max(c0, tok0 - (K - 1));     // first row with statistics
  const int n_main = tok0 + n - r_lo;
  // the portion's last K-1 rows, for the new history (first tile only)
  const int e_lo = max(max(c0, c0 + ntot - (K - 1)), tok0 + n);
  const int n_extra = first ? max(0, c0 + ntot - e_lo) : 0;
  for (int i = wave; i < n_main + n_extra; i += NW) {
    const int row = i < n_main ? r_lo + i : e_lo + (i - n_main);
    float mu, rs;
    wave_row_stats(X + (int64_t)row * W, W, eps, lane, &mu, &rs);
    if (lane == 0) {
      s_mean[i] = mu;
      s_rstd[i] = rs;
    }
  }
  __syncthreads();
  float* hs = hist + (int64_t)slots[seq] * (K - 1) * W;
  // few tiles (decoding): the channels are spread over gridDim.y blocks,
  // each with its own copy of the row statistics
  const int c_first = blockIdx.y * BLOCK + threadIdx.x;
  const int c_step = gridDim.y * BLOCK;
  for (int c = c_first; c < W; c += c_step) {
    const float wc = w[c];
    // taps and the sliding window of normed values are aligned at the END
    // of fixed-size arrays (leading entries zero): every index is static
    float tw[MAXK], hv[MAXK - 1];
#pragma unroll
    for (int m = 0; m < MAXK; ++m) {
      const int j = m - (MAXK - K);
      tw[m] = j >= 0 ? taps[(int64_t)c * K + j] : 0.f;
    }
#pragma unroll
    for (int m = 0; m < MAXK - 1; ++m) {
      const int j = m - (MAXK - K);
      float v = 0.f;
      if (j >= 0) {
        const int row = tok0 - (K - 1) + j;
        if (row >= c0) {
          const int si = row - r_lo;
          v = (X[(int64_t)row * W + c] - s_mean[si]) * s_rstd[si] * wc;
        } else if (!fresh) {
          v = hs[(int64_t)(K - 1 + row - c0) * W + c];
        }
      }
      hv[m] = v;
    }
    for (int i = 0; i < n; ++i) {
      const int row = tok0 + i, si = row - r_lo;
      const float self =
          (X[(int64_t)row * W + c] - s_mean[si]) * s_rstd[si] * wc;
      float acc = tw[MAXK - 1] * self;
#pragma unroll
      for (int m = 0; m < MAXK - 1; ++m) acc += tw[m] * hv[m];
#pragma unroll
      for (int m = 0; m < MAXK - 2; ++m) hv[m] = hv[m + 1];
      hv[MAXK - 2] = self;
      stf<T>(out, (int64_t)row * W + c, self + acc);
    }
  }
  if (!first || K <= 1) return;
  __syncthreads();       // every read of the old history is done
  for (int c = c_first; c < W; c += c_step) {
    const float wc = w[c];
    for (int r = 0; r < K - 1; ++r) {
      const int rr = ntot - (K - 1) + r;        // row within the portion
      float hv;
      if (rr >= 0) {
        const int row = c0 + rr;
        const int si = row < tok0 + n ? row - r_lo : n_main + (row - e_lo);
        hv = (X[(int64_t)row * W + c] - s_mean[si]) * s_rstd[si] * wc;
      } else {
        // ascending r: the source index r + ntot is not yet overwritten
        hv = fresh ? 0.f : hs[(int64_t)(r + ntot) * W + c];
      }
      hs[(int64_t)r * W + c] = hv;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void postln_add_kernel(
    float* __restrict__ X, const T* __restrict__ y, const T* __restrict__ y2,
    const float* __restrict__ w, const float* __restrict__ wy,
    const float* __restrict__ wy2, int W, float eps) {
  extern __shared__ float u[];      // [W]
  __shared__ float red[NW], red2[NW];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * W;
  if (y2) {
    const T* y2r = y2 + row * W;
    float a = 0.f, b = 0.f;
    for (int c = threadIdx.x; c < W; c += BLOCK) {
      const float p = ldf<T>(yr, c), q = ldf<T>(y2r, c);
      a += p * p;
      b += q * q;
    }
    const float ra = 1.0f / sqrtf(block_reduce_sum<NW>(a, red) / (float)W + eps);
    const float rb = 1.0f / sqrtf(block_reduce_sum<NW>(b, red2) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += BLOCK)
      u[c] = 0.5f * (ldf<T>(yr, c) * ra * wy[c] + ldf<T>(y2r, c) * rb * wy2[c]);
  } else {
    for (int c = threadIdx.x; c < W; c += BLOCK) u[c] = ldf<T>(yr, c);
  }
  __syncthreads();
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += BLOCK) s += u[c];
  const float mu = block_reduce_sum<NW>(s, red) / (float)W;
  float v = 0.f;
  for (int c = threadIdx.x; c < W; c += BLOCK) {
    const float d = u[c] - mu;
    v += d * d;
  }
  const float rs = 1.0f / sqrtf(block_reduce_sum<NW>(v, red2) / (float)W + eps);
  float* xr = X + row * W;
  for (int c = threadIdx.x; c < W; c += BLOCK)
    xr[c] += (u[c] - mu) * rs * w[c];
}

// bf16 rows whose length is a multiple of 8: 16-byte loads and stores
__global__ __launch_bounds__(BLOCK) void polynorm_vec8_kernel(
    const bf16* __restrict__ z, const float* __restrict__ coef,
    bf16* __restrict__ out, int N, float eps) {
  __shared__ float r1[NW], r2[NW], r3[NW];
  const int64_t row = blockIdx.x;
  const bf16x8* zr = reinterpret_cast<const bf16x8*>(z + row * N);
  bf16x8* orow = reinterpret_cast<bf16x8*>(out + row * N);
  float a = 0.f, b = 0.f, c3 = 0.f;
  for (int c = threadIdx.x; c < N / 8; c += BLOCK) {
    const bf16x8 v8 = zr[c];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = bf2f(v8.v[e]), v2 = v * v;
      a += v2;
      b += v2 * v2;
      c3 += v2 * v2 * v2;
    }
  }
  const float n1 = 1.0f / sqrtf(block_reduce_sum<NW>(a, r1) / (float)N + eps);
  const float n2 = 1.0f / sqrtf(block_reduce_sum<NW>(b, r2) / (float)N + eps);
  const float n3 = 1.0f / sqrtf(block_reduce_sum<NW>(c3, r3) / (float)N + eps);
  const float k1 = coef[0] * n1, k2 = coef[1] * n2, k3 = coef[2] * n3,
              k0 = coef[3];
  for (int c = threadIdx.x; c < N / 8; c += BLOCK) {
    const bf16x8 v8 = zr[c];
    bf16x8 o8;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = bf2f(v8.v[e]), v2 = v * v;
      o8.v[e] = f2bf(k1 * v + k2 * v2 + k3 * v2 * v + k0);
    }
    orow[c] = o8;
  }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void polynorm_kernel(
    const T* __restrict__ z, const float* __restrict__ coef,
    T* __restrict__ out, int N, float eps) {
  __shared__ float r1[NW], r2[NW], r3[NW];
  const int64_t row = blockIdx.x;
  const T* zr = z + row * N;
  float a = 0.f, b = 0.f, c3 = 0.f;
  for (int c = threadIdx.x; c < N; c += BLOCK) {
    const float v = ldf<T>(zr, c), v2 = v * v;
    a += v2;
    b += v2 * v2;
    c3 += v2 * v2 * v2;
  }
  const float n1 = 1.0f / sqrtf(block_reduce_sum<NW>(a, r1) / (float)N + eps);
  const float n2 = 1.0f / sqrtf(block_reduce_sum<NW>(b, r2) / (float)N + eps);
  const float n3 = 1.0f / sqrtf(block_reduce_sum<NW>(c3, r3) / (float)N + eps);
  const float k1 = coef[0] * n1, k2 = coef[1] * n2, k3 = coef[2] * n3,
              k0 = coef[3];
  for (int c = threadIdx.x; c < N; c += BLOCK) {
    const float v = ldf<T>(zr, c), v2 = v * v;
    stf<T>(out, row * N + c, k1 * v + k2 * v2 + k3 * v2 * v + k0);
  }
}

// grid (rows, groups)
template <typename T>
__global__ __launch_bounds__(BLOCK) void gated_group_rms_kernel(
    const float* __restrict__ y, const T* __restrict__ gate, int ldg,
    int gate_col, const float* __restrict__ w, T* __restrict__ out, int N,
    int NG, float eps) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  const int c_lo = blockIdx.y * NG;
  const float* yr = y + row * N + c_lo;
  const T* gr = gate + row * ldg + gate_col + c_lo;
  float ss = 0.f;
  for (int c = threadIdx.x; c < NG; c += BLOCK) {
    const float v = yr[c] * silu_f(ldf<T>(gr, c));
    ss += v * v;
  }
  const float rn = 1.0f / sqrtf(block_reduce_sum<NW>(ss, red) / (float)NG + eps);
  for (int c = threadIdx.x; c < NG; c += BLOCK) {
    const float v = yr[c] * silu_f(ldf<T>(gr, c));
    stf<T>(out, row * N + c_lo + c, v * rn * w[c_lo + c]);
  }
}

}  // namespace

extern "C" {

int tl_ln_canon_tile() { return TILE; }

void tl_layer_norm_rows(const void* x, const void* w, void* out, int64_t rows,
                        int W, float eps, int out_f32, hipStream_t stream) {
  if (rows <= 0) return;
  if (out_f32)
    hipLaunchKernelGGL(layer_norm_rows_kernel<float>, dim3(rows), dim3(BLOCK),
                       0, stream, (const float*)x, (const float*)w,
                       (float*)out, W, eps);
  else
    hipLaunchKernelGGL(layer_norm_rows_kernel<bf16>, dim3(rows), dim3(BLOCK),
                       0, stream, (const float*)x, (const float*)w,
                       (bf16*)out, W, eps);
}

void tl_ln_canon(const void* X, const void* w, const void* taps, void* hist,
                 const void* tiles, int n_tiles, const void* cu,
                 const void* slots, const void* pos0, void* out, int W, int K,
                 float eps, int out_f32, hipStream_t stream) {
  if (n_tiles <= 0) return;
  const int gy = n_tiles >= 512 ? 1 : min(8, max(1, (W + BLOCK - 1) / BLOCK));
  const dim3 grid(n_tiles, gy);
  if (out_f32)
    hipLaunchKernelGGL(ln_canon_kernel<float>, grid, dim3(BLOCK), 0,
                       stream, (const float*)X, (const float*)w,
                       (const float*)taps, (float*)hist, (const int*)tiles,
                       (const int*)cu, (const int*)slots, (const int*)pos0,
                       (float*)out, W, K, eps);
  else
    hipLaunchKernelGGL(ln_canon_kernel<bf16>, grid, dim3(BLOCK), 0,
                       stream, (const float*)X, (const float*)w,
                       (const float*)taps, (float*)hist, (const int*)tiles,
                       (const int*)cu, (const int*)slots, (const int*)pos0,
                       (bf16*)out, W, K, eps);
}

void tl_postln_add(void* X, const void* y, const void* y2, const void* w,
                   const void* wy, const void* wy2, int64_t rows, int W,
                   float eps, int is_f32, hipStream_t stream) {
  if (rows <= 0) return;
  const size_t smem = sizeof(float) * (size_t)W;
  if (is_f32)
    hipLaunchKernelGGL(postln_add_kernel<float>, dim3(rows), dim3(BLOCK), smem,
                       stream, (float*)X, (const float*)y, (const float*)y2,
                       (const float*)w, (const float*)wy, (const float*)wy2,
                       W, eps);
  else
    hipLaunchKernelGGL(postln_add_kernel<bf16>, dim3(rows), dim3(BLOCK), smem,
                       stream, (float*)X, (const bf16*)y, (const bf16*)y2,
                       (const float*)w, (const float*)wy, (const float*)wy2,
                       W, eps);
}

void tl_polynorm(const void* z, const void* coef, void* out, int64_t rows,
                 int N, float eps, int is_f32, hipStream_t stream) {
  if (rows <= 0) return;
  if (is_f32)
    hipLaunchKernelGGL(polynorm_kernel<float>, dim3(rows), dim3(BLOCK), 0,
                       stream, (const float*)z, (const float*)coef,
                       (float*)out, N, eps);
  else if (N % 8 == 0)
    hipLaunchKernelGGL(polynorm_vec8_kernel, dim3(rows), dim3(BLOCK), 0,
                       stream, (const bf16*)z, (const float*)coef, (bf16*)out,
                       N, eps);
  else
    hipLaunchKernelGGL(polynorm_kernel<bf16>, dim3(rows), dim3(BLOCK), 0,
                       stream, (const bf16*)z, (const float*)coef, (bf16*)out,
                       N, eps);
}

void tl_gated_group_rms(const void* y, const void* gate, int ldg, int gate_col,
                        const void* w, void* out, int64_t rows, int N,
                        int groups, float eps, int is_f32,
                        hipStream_t stream) {
  if (rows <= 0) return;
  dim3 grid(rows, groups);
  if (is_f32)
    hipLaunchKernelGGL(gated_group_rms_kernel<float>, grid, dim3(BLOCK), 0,
                       stream, (const float*)y, (const float*)gate, ldg,
                       gate_col, (const float*)w, (float*)out, N, N / groups,
                       eps);
  else
    hipLaunchKernelGGL(gated_group_rms_kernel<bf16>, grid, dim3(BLOCK), 0,
                       stream, (const float*)y, (const bf16*)gate, ldg,
                       gate_col, (const float*)w, (bf16*)out, N, N / groups,
                       eps);
}

}  // extern "C"
