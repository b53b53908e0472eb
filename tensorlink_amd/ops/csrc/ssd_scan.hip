// Selective state-space recurrence with one scalar decay per head and token
// over ragged sequences (gfx950).
//
// Per head h of group g = h / (H/G), with raw step size r_t from the fused
// projection:
//     dt_t = softplus(r_t + dt_bias_h)
//     S_t  = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T   (S: [N, P])
//     y_t  = S_t^T C_t + skip_h x_t
// x [H*P], B [G*N], C [G*N] arrive in fp32 (the convolution kernel writes
// them so); softplus, exponentials, the state and the read-out are fp32.
// One block per (sequence, head) walks the sequence's new tokens in order;
// the state comes from the sequence's slot (zeros when it has no cached
// tokens) and goes back there, so prompt portions of any size and single
// decoded tokens run the same arithmetic in the same order.
//
// Register form: thread (c, q) owns column c of S for the rows
// n = q, q + NG, ... (NR of them, PR columns c + u*PT per thread); the NG
// partial read-outs of a column meet in LDS. Tokens are staged in rounds of
// RT so a round needs three barriers. Shapes beyond the register budget
// take the generic kernel, which keeps S in the slot's memory.
//
// Long prompt portions take the chunk form around batched fp32 GEMMs of the
// vendor library. With chunks of C tokens, S0 the state before a chunk,
// i, j indices inside it, a_m = -exp(A_log) dt_m and L_i = sum_{m<=i} a_m:
//     y_i = exp(L_i) S0^T C_i + sum_{j<=i} exp(L_i - L_j) (C_i . B_j) dt_j x_j
//     S1  = exp(L_n) S0 + sum_j exp(L_n - L_j) dt_j B_j x_j^T
// Only exponentials of non-positive numbers occur. tl_ssd_chunk_prep lays
// out C, B, dt x per (chunk, head), zero-padded, with the weighted copies
// exp(L_i) C_i and exp(L_n - L_j) B_j, the running sums L and exp(L_n);
// tl_ssd_decay_mask applies M[i][j] = exp(L_i - L_j) (j <= i, else 0);
// tl_ssd_chain turns the chunk summaries into the state before each chunk
// and leaves the final state in the slot. Everything is fp32.

#include "common.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int RT = 8;  // tokens per round

template <typename T> DEVINLINE float ldf(const T* p) ;
template <> DEVINLINE float ldf<float>(const float* p) { return *p; }
template <> DEVINLINE float ldf<bf16>(const bf16* p) { return bf2f(*p); }

DEVINLINE float softplus_f(float v) {
  return v > 20.f ? v : log1pf(expf(v));
}

template <typename T, int NR, int PR>
__global__ __launch_bounds__(BLOCK) void ssd_scan_kernel(
    const float* __restrict__ xbc, int ldx, int x_off, int b_off, int c_off,
    const T* __restrict__ dt_src, int ldd, int dt_col,
    const float* __restrict__ dt_bias, const float* __restrict__ A_log,
    const float* __restrict__ skip, float* __restrict__ S,
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ pos0, float* __restrict__ out, int H, int G,
    int N, int P, int PT, int NG) {
  extern __shared__ float lds[];
  // lds: xs[RT][P] | bs[RT][N] | cs[RT][N] | dec[RT] | part[RT][NG][P]
  float* xs = lds;
  float* bs = xs + RT * P;
  float* cs = bs + RT * N;
  float* dec = cs + RT * N;
  float* part = dec + RT;
  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 <= t0) return;
  const int g = h / (H / G);
  const int c0 = threadIdx.x % PT, q = threadIdx.x / PT;
  const float nA = -expf(A_log[h]);
  const float dtb = dt_bias[h], sk = skip[h];
  float* Sh = S + ((int64_t)slots[b] * H + h) * N * P;
  float st[NR][PR];
  const bool fresh = pos0[b] == 0;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int n = q + r * NG;
#pragma unroll
    for (int u = 0; u < PR; ++u) {
      const int c = c0 + u * PT;
      st[r][u] = (!fresh && n < N && c < P) ? Sh[(int64_t)n * P + c] : 0.f;
    }
  }
  for (int tb = t0; tb < t1; tb += RT) {
    const int nt = min(RT, t1 - tb);
    __syncthreads();
    if (threadIdx.x < nt) {
      const float dt = softplus_f(
          ldf<T>(dt_src + (int64_t)(tb + threadIdx.x) * ldd + dt_col + h) + dtb);
      dec[threadIdx.x] = expf(nA * dt);
      part[threadIdx.x] = dt;        // staged for the B rows below
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * N; i += BLOCK) {
      const int tt = i / N, n = i - tt * N;
      const float* row = xbc + (int64_t)(tb + tt) * ldx;
      bs[i] = row[b_off + g * N + n] * part[tt];
      cs[i] = row[c_off + g * N + n];
    }
    for (int i = threadIdx.x; i < nt * P; i += BLOCK) {
      const int tt = i / P, c = i - tt * P;
      xs[i] = xbc[(int64_t)(tb + tt) * ldx + x_off + h * P + c];
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      float xv[PR], acc[PR];
      const float a = dec[tt];
#pragma unroll
      for (int u = 0; u < PR; ++u) {
        const int c = c0 + u * PT;
        xv[u] = c < P ? xs[tt * P + c] : 0.f;
        acc[u] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        const int n = q + r * NG;
        const float bn = n < N ? bs[tt * N + n] : 0.f;
        const float cn = n < N ? cs[tt * N + n] : 0.f;
#pragma unroll
        for (int u = 0; u < PR; ++u) {
          st[r][u] = a * st[r][u] + bn * xv[u];
          acc[u] += st[r][u] * cn;
        }
      }
#pragma unroll
      for (int u = 0; u < PR; ++u) {
        const int c = c0 + u * PT;
        if (c < P) part[RT + (tt * NG + q) * P + c] = acc[u];
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * P; i += BLOCK) {
      const int tt = i / P, c = i - tt * P;
      float o = sk * xs[i];
      for (int qq = 0; qq < NG; ++qq) o += part[RT + (tt * NG + qq) * P + c];
      out[((int64_t)(tb + tt) * H + h) * P + c] = o;
    }
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int n = q + r * NG;
#pragma unroll
    for (int u = 0; u < PR; ++u) {
      const int c = c0 + u * PT;
      if (n < N && c < P) Sh[(int64_t)n * P + c] = st[r][u];
    }
  }
}

// Any head size: the state stays in the slot's memory; thread c owns the
// columns c, c + BLOCK, ... and walks all rows for every token.
template <typename T>
__global__ __launch_bounds__(BLOCK) void ssd_scan_generic_kernel(
    const float* __restrict__ xbc, int ldx, int x_off, int b_off, int c_off,
    const T* __restrict__ dt_src, int ldd, int dt_col,
    const float* __restrict__ dt_bias, const float* __restrict__ A_log,
    const float* __restrict__ skip, float* __restrict__ S,
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ pos0, float* __restrict__ out, int H, int G,
    int N, int P) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 <= t0) return;
  const int g = h / (H / G);
  const float nA = -expf(A_log[h]);
  const float dtb = dt_bias[h], sk = skip[h];
  float* Sh = S + ((int64_t)slots[b] * H + h) * N * P;
  if (pos0[b] == 0)
    for (int i = threadIdx.x; i < N * P; i += BLOCK) Sh[i] = 0.f;
  __syncthreads();
  // from here a thread only touches its own columns of Sh
  for (int t = t0; t < t1; ++t) {
    const float* row = xbc + (int64_t)t * ldx;
    const float dt =
        softplus_f(ldf<T>(dt_src + (int64_t)t * ldd + dt_col + h) + dtb);
    const float a = expf(nA * dt);
    for (int c = threadIdx.x; c < P; c += BLOCK) {
      const float xv = row[x_off + h * P + c];
      float acc = sk * xv;
      for (int n = 0; n < N; ++n) {
        const float s = a * Sh[(int64_t)n * P + c] +
                        dt * row[b_off + g * N + n] * xv;
        Sh[(int64_t)n * P + c] = s;
        acc += s * row[c_off + g * N + n];
      }
      out[((int64_t)t * H + h) * P + c] = acc;
    }
  }
}

// grid (chunks, H); outputs [chunk][h][C][N|P] fp32, rows >= n are zero
template <typename T>
__global__ __launch_bounds__(BLOCK) void ssd_chunk_prep_kernel(
    const float* __restrict__ xbc, int ldx, int x_off, int b_off, int c_off,
    const T* __restrict__ dt_src, int ldd, int dt_col,
    const float* __restrict__ dt_bias, const float* __restrict__ A_log,
    const int* __restrict__ cu_c, float* __restrict__ Cs,
    float* __restrict__ Cd, float* __restrict__ Bs, float* __restrict__ Bw,
    float* __restrict__ Xd, float* __restrict__ Lc, float* __restrict__ tot,
    int H, int G, int N, int P, int C) {
  extern __shared__ float sh[];            // dts[C] | Ls[C]
  float* dts = sh;
  float* Ls = sh + C;
  const int c = blockIdx.x, h = blockIdx.y;
  const int g = h / (H / G);
  const int t0 = cu_c[c], n = cu_c[c + 1] - t0;
  const float nA = -expf(A_log[h]);
  for (int r = threadIdx.x; r < C; r += BLOCK) {
    float dt = 0.f;
    if (r < n)
      dt = softplus_f(ldf<T>(dt_src + (int64_t)(t0 + r) * ldd + dt_col + h) +
                      dt_bias[h]);
    dts[r] = dt;
    Ls[r] = nA * dt;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = 0.f;
    for (int r = 0; r < C; ++r) {
      run += Ls[r];
      Ls[r] = run;
    }
  }
  __syncthreads();
  const float Ln = Ls[C - 1];              // padded rows add nothing
  const int64_t base = ((int64_t)c * H + h) * C;
  for (int r = threadIdx.x; r < C; r += BLOCK) Lc[base + r] = Ls[r];
  if (threadIdx.x == 0) tot[(int64_t)c * H + h] = expf(Ln);
  for (int i = threadIdx.x; i < C * N; i += BLOCK) {
    const int r = i / N, e = i - r * N;
    float cv = 0.f, bv = 0.f;
    if (r < n) {
      const float* row = xbc + (int64_t)(t0 + r) * ldx;
      cv = row[c_off + g * N + e];
      bv = row[b_off + g * N + e];
    }
    const int64_t o = (base + r) * N + e;
    Cs[o] = cv;
    Cd[o] = cv * expf(Ls[r]);
    Bs[o] = bv;
    Bw[o] = bv * expf(Ln - Ls[r]);
  }
  for (int i = threadIdx.x; i < C * P; i += BLOCK) {
    const int r = i / P, e = i - r * P;
    float xv = 0.f;
    if (r < n)
      xv = dts[r] * xbc[(int64_t)(t0 + r) * ldx + x_off + h * P + e];
    Xd[(base + r) * P + e] = xv;
  }
}

// A [chunks*H][C][C] in place: A[i][j] *= exp(L_i - L_j) for j <= i, else 0
__global__ __launch_bounds__(BLOCK) void ssd_decay_mask_kernel(
    float* __restrict__ A, const float* __restrict__ Lc, int C) {
  extern __shared__ float Ls[];
  for (int i = threadIdx.x; i < C; i += BLOCK)
    Ls[i] = Lc[(int64_t)blockIdx.x * C + i];
  __syncthreads();
  float* Ab = A + (int64_t)blockIdx.x * C * C;
  for (int i = threadIdx.x; i < C * C; i += BLOCK) {
    const int r = i / C, j = i - r * C;
    Ab[i] = j <= r ? Ab[i] * expf(Ls[r] - Ls[j]) : 0.f;
  }
}

// grid (B, H, ceil(N*P / BLOCK)): U [chunks][H][N*P] holds the chunk
// summaries on entry and the state BEFORE each chunk on exit; the slot
// receives the state after the sequence's last chunk.
__global__ __launch_bounds__(BLOCK) void ssd_chain_kernel(
    float* __restrict__ U, float* __restrict__ S,
    const float* __restrict__ tot, const int* __restrict__ chunk_base,
    const int* __restrict__ n_chunks, const int* __restrict__ slots,
    const int* __restrict__ pos0, int H, int NP) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * BLOCK + threadIdx.x;
  const int nc = n_chunks[b];
  if (e >= NP || nc <= 0) return;
  float* Sp = S + ((int64_t)slots[b] * H + h) * NP + e;
  float s = pos0[b] == 0 ? 0.f : *Sp;
  const int c0 = chunk_base[b];
  for (int c = c0; c < c0 + nc; ++c) {
    float* up = U + ((int64_t)c * H + h) * NP + e;
    const float u = *up;
    *up = s;
    s = tot[(int64_t)c * H + h] * s + u;
  }
  *Sp = s;
}

}  // namespace

extern "C" {

void tl_ssd_chunk_prep(const void* xbc, int ldx, int x_off, int b_off,
                       int c_off, const void* dt_src, int ldd, int dt_col,
                       const void* dt_bias, const void* A_log,
                       const void* cu_c, void* Cs, void* Cd, void* Bs,
                       void* Bw, void* Xd, void* Lc, void* tot, int NC, int H,
                       int G, int N, int P, int C, int dt_f32,
                       hipStream_t stream) {
  if (NC <= 0) return;
  dim3 grid(NC, H), block(BLOCK);
  const size_t smem = sizeof(float) * 2 * C;
  if (dt_f32)
    hipLaunchKernelGGL(ssd_chunk_prep_kernel<float>, grid, block, smem, stream,
                       (const float*)xbc, ldx, x_off, b_off, c_off,
                       (const float*)dt_src, ldd, dt_col,
                       (const float*)dt_bias, (const float*)A_log,
                       (const int*)cu_c, (float*)Cs, (float*)Cd, (float*)Bs,
                       (float*)Bw, (float*)Xd, (float*)Lc, (float*)tot, H, G,
                       N, P, C);
  else
    hipLaunchKernelGGL(ssd_chunk_prep_kernel<bf16>, grid, block, smem, stream,
                       (const float*)xbc, ldx, x_off, b_off, c_off,
                       (const bf16*)dt_src, ldd, dt_col,
                       (const float*)dt_bias, (const float*)A_log,
                       (const int*)cu_c, (float*)Cs, (float*)Cd, (float*)Bs,
                       (float*)Bw, (float*)Xd, (float*)Lc, (float*)tot, H, G,
                       N, P, C);
}

void tl_ssd_decay_mask(void* A, const void* Lc, int NCH, int C,
                       hipStream_t stream) {
  if (NCH <= 0) return;
  hipLaunchKernelGGL(ssd_decay_mask_kernel, dim3(NCH), dim3(BLOCK),
                     sizeof(float) * C, stream, (float*)A, (const float*)Lc,
                     C);
}

void tl_ssd_chain(void* U, void* S, const void* tot, const void* chunk_base,
                  const void* n_chunks, const void* slots, const void* pos0,
                  int B, int H, int NP, hipStream_t stream) {
  if (B <= 0) return;
  dim3 grid(B, H, (NP + BLOCK - 1) / BLOCK);
  hipLaunchKernelGGL(ssd_chain_kernel, grid, dim3(BLOCK), 0, stream,
                     (float*)U, (float*)S, (const float*)tot,
                     (const int*)chunk_base, (const int*)n_chunks,
                     (const int*)slots, (const int*)pos0, H, NP);
}

// returns 0 on success, 1 if the launch cannot be made
int tl_ssd_scan(const void* xbc, int ldx, int x_off, int b_off, int c_off,
                const void* dt_src, int ldd, int dt_col, const void* dt_bias,
                const void* A_log, const void* skip, void* S, const void* cu,
                const void* slots, const void* pos0, void* out, int B, int H,
                int G, int N, int P, int dt_f32, hipStream_t stream) {
  if (B <= 0 || H <= 0 || G <= 0 || H % G || N <= 0 || P <= 0) return 1;
  dim3 grid(B, H), block(BLOCK);
  int PT = 1;
  while (PT < P && PT < BLOCK) PT <<= 1;
  const int NG = BLOCK / PT;
  const int pr = (P + PT - 1) / PT;
  const int nr = (N + NG - 1) / NG;
  const size_t smem = sizeof(float) * ((size_t)RT * (P + 2 * N + 1) + RT +
                                       (size_t)RT * NG * P);
#define TL_SS(TT, NRR, PRR)                                                  \
  hipLaunchKernelGGL((ssd_scan_kernel<TT, NRR, PRR>), grid, block, smem,     \
                     stream, (const float*)xbc, ldx, x_off, b_off, c_off,    \
                     (const TT*)dt_src, ldd, dt_col, (const float*)dt_bias,  \
                     (const float*)A_log, (const float*)skip, (float*)S,     \
                     (const int*)cu, (const int*)slots, (const int*)pos0,    \
                     (float*)out, H, G, N, P, PT, NG)
#define TL_SS_T(NRR, PRR)     \
  do {                        \
    if (dt_f32)               \
      TL_SS(float, NRR, PRR); \
    else                      \
      TL_SS(bf16, NRR, PRR);  \
    return 0;                 \
  } while (0)
  if (smem <= 64 * 1024) {
    if (pr == 1) {
      if (nr <= 8) TL_SS_T(8, 1);
      if (nr <= 16) TL_SS_T(16, 1);
      if (nr <= 32) TL_SS_T(32, 1);
      if (nr <= 64) TL_SS_T(64, 1);
      if (nr <= 128) TL_SS_T(128, 1);
    }
  }
#undef TL_SS_T
#undef TL_SS
  if (dt_f32)
    hipLaunchKernelGGL(ssd_scan_generic_kernel<float>, grid, block, 0, stream,
                       (const float*)xbc, ldx, x_off, b_off, c_off,
                       (const float*)dt_src, ldd, dt_col,
                       (const float*)dt_bias, (const float*)A_log,
                       (const float*)skip, (float*)S, (const int*)cu,
                       (const int*)slots, (const int*)pos0, (float*)out, H, G,
                       N, P);
  else
    hipLaunchKernelGGL(ssd_scan_generic_kernel<bf16>, grid, block, 0, stream,
                       (const float*)xbc, ldx, x_off, b_off, c_off,
                       (const bf16*)dt_src, ldd, dt_col,
                       (const float*)dt_bias, (const float*)A_log,
                       (const float*)skip, (float*)S, (const int*)cu,
                       (const int*)slots, (const int*)pos0, (float*)out, H, G,
                       N, P);
  return 0;
}

}  // extern "C"
