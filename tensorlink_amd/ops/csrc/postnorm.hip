// Row-wise kernels of the post-norm layered family (gfx950).
//
// The residual X is fp32 and every sublayer's output y is normalised
// BEFORE it is added:  X <- X + y / rms(y) * g,  g = w or 1 + w.
// tl_postnorm_add does the row statistic, the scaled add and the cast of
// the new residual to the serving dtype (the next sublayer's GEMM input)
// in one kernel: y is read twice (the second time from cache), X makes one
// round trip. tl_rms_scale is the plain / gated RMS scaling (final norm;
// read-out norm of a linear-attention mixer with its sigmoid gate), tl_gelu
// the exact or tanh-form GELU with an optional gathered per-token factor,
// tl_soft_cap the logit cap. Statistics and activations are fp32.
//
// Pre-norm layers use tl_add_rms: the previous sublayer's output is added
// to the fp32 residual and the NEXT sublayer's input, rms(X) * w, is written
// in the serving dtype by the same kernel (X <- X + y;  h = X / rms(X) * w).
// tl_gelu_gate is the gated feed-forward's activation on a fused [gate | up]
// projection: gelu(gate) * up.

#include "common.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int NW = BLOCK / WAVE_SIZE;

template <typename T> DEVINLINE float ldf(const T* p, int64_t i);
template <> DEVINLINE float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <> DEVINLINE float ldf<bf16>(const bf16* p, int64_t i) { return bf2f(p[i]); }
template <typename T> DEVINLINE void stf(T* p, int64_t i, float v);
template <> DEVINLINE void stf<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> DEVINLINE void stf<bf16>(bf16* p, int64_t i, float v) { p[i] = f2bf(v); }

DEVINLINE float gelu_f(float z, int tanh_form) {
  if (tanh_form)
    return 0.5f * z *
           (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return 0.5f * z * (1.f + erff(z * 0.7071067811865476f));
}

// one block per row
template <typename T>
__global__ __launch_bounds__(BLOCK) void postnorm_add_kernel(
    float* __restrict__ X, const T* __restrict__ y,
    const float* __restrict__ w, T* __restrict__ h, int W, float eps,
    int one_plus) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += BLOCK) {
    const float v = ldf<T>(yr, c);
    ss += v * v;
  }
  const float tot = block_reduce_sum<NW>(ss, red);
  const float rn = 1.0f / sqrtf(tot / (float)W + eps);
  float* xr = X + row * W;
  for (int c = threadIdx.x; c < W; c += BLOCK) {
    const float g = one_plus ? 1.f + w[c] : w[c];
    const float v = xr[c] + ldf<T>(yr, c) * rn * g;
    xr[c] = v;
    if (h) stf<T>(h, row * W + c, v);
  }
}

// X += y (if given); h = X / rms(X) * w in the serving dtype (no w: no h)
template <typename T>
__global__ __launch_bounds__(BLOCK) void add_rms_kernel(
    float* __restrict__ X, const T* __restrict__ y,
    const float* __restrict__ w, T* __restrict__ h, int W, float eps,
    float x_scale) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  float* xr = X + row * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += BLOCK) {
    float v = xr[c] * x_scale;
    if (y) v += ldf<T>(y, row * W + c);
    if (y || x_scale != 1.f) xr[c] = v;
    ss += v * v;
  }
  if (!w) return;                 // the residual add alone
  const float tot = block_reduce_sum<NW>(ss, red);
  const float rn = 1.0f / sqrtf(tot / (float)W + eps);
  // a thread reads back only what it wrote itself
  for (int c = threadIdx.x; c < W; c += BLOCK)
    stf<T>(h, row * W + c, xr[c] * rn * w[c]);
}

// out[r][c] = gelu(p[r][c]) * p[r][N + c] on rows of 2N columns
template <typename T>
__global__ __launch_bounds__(BLOCK) void gelu_gate_kernel(
    const T* __restrict__ p, T* __restrict__ out, int64_t n, int N,
    int tanh_form) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * BLOCK) {
    const int64_t r = i / N;
    const int c = (int)(i - r * N);
    const T* row = p + r * 2 * N;
    stf<T>(out, i, gelu_f(ldf<T>(row, c), tanh_form) * ldf<T>(row, N + c));
  }
}

// bf16 rows whose half width is a multiple of 8: 16-byte loads and stores
__global__ __launch_bounds__(BLOCK) void gelu_gate_vec8_kernel(
    const bf16x8* __restrict__ p, bf16x8* __restrict__ out, int64_t n8,
    int N8, int tanh_form) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n8;
       i += (int64_t)gridDim.x * BLOCK) {
    const int64_t r = i / N8;
    const int c = (int)(i - r * N8);
    const bf16x8 a = p[r * 2 * N8 + c], b = p[r * 2 * N8 + N8 + c];
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      o.v[e] = f2bf(gelu_f(bf2f(a.v[e]), tanh_form) * bf2f(b.v[e]));
    out[i] = o;
  }
}

// out = x / rms(x) * g [* sigmoid(gate)], x fp32 [rows, N]
template <typename T>
__global__ __launch_bounds__(BLOCK) void rms_scale_kernel(
    const float* __restrict__ x, const float* __restrict__ w,
    const T* __restrict__ gate, int ldg, int gate_col, T* __restrict__ out,
    int N, float eps, int one_plus) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  const float* xr = x + row * N;
  float ss = 0.f;
  for (int c = threadIdx.x; c < N; c += BLOCK) ss += xr[c] * xr[c];
  const float tot = block_reduce_sum<NW>(ss, red);
  const float rn = 1.0f / sqrtf(tot / (float)N + eps);
  for (int c = threadIdx.x; c < N; c += BLOCK) {
    float v = xr[c] * rn * (one_plus ? 1.f + w[c] : w[c]);
    if (gate) {
      const float z = ldf<T>(gate, row * ldg + gate_col + c);
      v *= 1.f / (1.f + expf(-z));
    }
    stf<T>(out, row * N + c, v);
  }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void gelu_kernel(
    const T* __restrict__ x, T* __restrict__ out, int64_t n, int N,
    int tanh_form, const T* __restrict__ table, int ldt, int table_col,
    const int* __restrict__ tokens) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * BLOCK) {
    float v = gelu_f(ldf<T>(x, i), tanh_form);
    if (table) {
      const int64_t r = i / N;
      const int c = (int)(i - r * N);
      v *= ldf<T>(table, (int64_t)tokens[r] * ldt + table_col + c);
    }
    stf<T>(out, i, v);
  }
}

// bf16, no gathered factor, n a multiple of 8: 16-byte loads and stores
__global__ __launch_bounds__(BLOCK) void gelu_vec8_kernel(
    const bf16x8* __restrict__ x, bf16x8* __restrict__ out, int64_t n8,
    int tanh_form) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n8;
       i += (int64_t)gridDim.x * BLOCK) {
    const bf16x8 a = x[i];
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r.v[e] = f2bf(gelu_f(bf2f(a.v[e]), tanh_form));
    out[i] = r;
  }
}

__global__ __launch_bounds__(BLOCK) void soft_cap_kernel(float* z, int64_t n,
                                                         float cap) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * BLOCK)
    z[i] = cap * tanhf(z[i] / cap);
}

int ew_grid(int64_t n) {
  const int64_t b = (n + BLOCK - 1) / BLOCK;
  return (int)(b < 1 ? 1 : (b > 8192 ? 8192 : b));
}

}  // namespace

extern "C" {

void tl_postnorm_add(void* X, const void* y, const void* w, void* h,
                     int64_t rows, int W, float eps, int one_plus, int is_f32,
                     hipStream_t stream) {
  if (rows <= 0) return;
  dim3 grid((unsigned)rows), block(BLOCK);
  if (is_f32)
    hipLaunchKernelGGL(postnorm_add_kernel<float>, grid, block, 0, stream,
                       (float*)X, (const float*)y, (const float*)w,
                       (float*)h, W, eps, one_plus);
  else
    hipLaunchKernelGGL(postnorm_add_kernel<bf16>, grid, block, 0, stream,
                       (float*)X, (const bf16*)y, (const float*)w, (bf16*)h,
                       W, eps, one_plus);
}

void tl_add_rms(void* X, const void* y, const void* w, void* h, int64_t rows,
                int W, float eps, float x_scale, int is_f32,
                hipStream_t stream) {
  if (rows <= 0) return;
  dim3 grid((unsigned)rows), block(BLOCK);
  if (is_f32)
    hipLaunchKernelGGL(add_rms_kernel<float>, grid, block, 0, stream,
                       (float*)X, (const float*)y, (const float*)w, (float*)h,
                       W, eps, x_scale);
  else
    hipLaunchKernelGGL(add_rms_kernel<bf16>, grid, block, 0, stream,
                       (float*)X, (const bf16*)y, (const float*)w, (bf16*)h,
                       W, eps, x_scale);
}

void tl_gelu_gate(const void* p, void* out, int64_t rows, int N,
                  int tanh_form, int is_f32, hipStream_t stream) {
  const int64_t n = rows * N;
  if (n <= 0) return;
  if (!is_f32 && N % 8 == 0) {
    hipLaunchKernelGGL(gelu_gate_vec8_kernel, dim3(ew_grid(n / 8)),
                       dim3(BLOCK), 0, stream, (const bf16x8*)p, (bf16x8*)out,
                       n / 8, N / 8, tanh_form);
    return;
  }
  dim3 grid(ew_grid(n)), block(BLOCK);
  if (is_f32)
    hipLaunchKernelGGL(gelu_gate_kernel<float>, grid, block, 0, stream,
                       (const float*)p, (float*)out, n, N, tanh_form);
  else
    hipLaunchKernelGGL(gelu_gate_kernel<bf16>, grid, block, 0, stream,
                       (const bf16*)p, (bf16*)out, n, N, tanh_form);
}

void tl_rms_scale(const void* x, const void* w, const void* gate, int ldg,
                  int gate_col, void* out, int64_t rows, int N, float eps,
                  int one_plus, int is_f32, hipStream_t stream) {
  if (rows <= 0) return;
  dim3 grid((unsigned)rows), block(BLOCK);
  if (is_f32)
    hipLaunchKernelGGL(rms_scale_kernel<float>, grid, block, 0, stream,
                       (const float*)x, (const float*)w, (const float*)gate,
                       ldg, gate_col, (float*)out, N, eps, one_plus);
  else
    hipLaunchKernelGGL(rms_scale_kernel<bf16>, grid, block, 0, stream,
                       (const float*)x, (const float*)w, (const bf16*)gate,
                       ldg, gate_col, (bf16*)out, N, eps, one_plus);
}

void tl_gelu(const void* x, void* out, int64_t n, int N, int tanh_form,
             const void* table, int ldt, int table_col, const void* tokens,
             int is_f32, hipStream_t stream) {
  if (n <= 0) return;
  if (!is_f32 && !table && n % 8 == 0) {
    hipLaunchKernelGGL(gelu_vec8_kernel, dim3(ew_grid(n / 8)), dim3(BLOCK), 0,
                       stream, (const bf16x8*)x, (bf16x8*)out, n / 8,
                       tanh_form);
    return;
  }
  dim3 grid(ew_grid(n)), block(BLOCK);
  if (is_f32)
    hipLaunchKernelGGL(gelu_kernel<float>, grid, block, 0, stream,
                       (const float*)x, (float*)out, n, N, tanh_form,
                       (const float*)table, ldt, table_col,
                       (const int*)tokens);
  else
    hipLaunchKernelGGL(gelu_kernel<bf16>, grid, block, 0, stream,
                       (const bf16*)x, (bf16*)out, n, N, tanh_form,
                       (const bf16*)table, ldt, table_col,
                       (const int*)tokens);
}

void tl_soft_cap(void* z, int64_t n, float cap, hipStream_t stream) {
  if (n <= 0) return;
  hipLaunchKernelGGL(soft_cap_kernel, dim3(ew_grid(n)), dim3(BLOCK), 0,
                     stream, (float*)z, n, cap);
}

}  // extern "C"
