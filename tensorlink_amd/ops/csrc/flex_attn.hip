// Softmax attention over a paged pool with the options that layered
// models combine (gfx950): grouped / single key heads, sliding window,
// a sink in the denominator, mixing of the heads' scores before the
// softmax, and values that are a prefix of the key row (latent attention,
// where every head attends the same cached rows [latent | rotated key]).
//
// tl_norm_rope_rows prepares rows of a fused projection: one RMS norm over
// a leading range of the columns (the WHOLE query or key projection, or
// the latent part of a latent row), rotate-half positions on a sub-range of
// every head, then either a dense fp32 copy (queries) or a scatter into the
// tokens' page rows (keys, values, latents). Angles are pos * f_i in double.
// Options: the norm per head over the head's columns with one shared weight,
// rotation pairs (2i, 2i+1) instead of halves, a multiplier on cos and sin
// (scaled rotations), and a blend (1 - lam) x + lam m with the same token's
// columns of another projection (value mixing across layers) before the
// row is written.
//
// tl_flex_attn_rows serves one query token and HB query heads of one key
// group per block. Each of the four waves strides over 64-key tiles of the
// visible range (one key per lane for the score dot products, one value
// column per lane for P.V), keeps online-softmax statistics per head, and
// the waves merge through LDS. Score mixing is linear and heads of one key
// group share their key, so the mixed score of head h is one dot product
// between the mixed query [sum_{g in c} T[h,g] q_g]_c and the G key heads'
// rows side by side: the block stages mixed queries and then works as if
// the key were G times as wide.
// Further options (TlFlexExtra): keys of the query's own chunk only, a kept
// prefix (the first positions stay visible beyond the window: the block
// walks the prefix tiles, then the window's), a learned distance bias from
// a per-head table indexed by i - j, and a sigmoid output gate per column
// or per head applied where the row is written.
// With few rows over long ranges the keys are also split over blockIdx.z
// and a merge kernel finishes the rows. It is exact for any query position,
// so it serves prompt portions and decoding alike; scores, weights and
// sums are fp32.

#include "common.hpp"
#include "flex_attn.hpp"

#include <cstdlib>

namespace {

constexpr int PAGE = 128;
static_assert(PAGE % WAVE_SIZE == 0, "a key tile must not straddle pages");
constexpr int NWAVE = 4;
constexpr int BLOCK = NWAVE * WAVE_SIZE;
constexpr int MAX_NORM_HEADS = 512;   // heads of a per-head normed row

template <typename T> DEVINLINE float ldv(const T* p);
template <> DEVINLINE float ldv<float>(const float* p) { return *p; }
template <> DEVINLINE float ldv<bf16>(const bf16* p) { return bf2f(*p); }
template <typename T> DEVINLINE void stv(T* p, float v);
template <> DEVINLINE void stv<float>(float* p, float v) { *p = v; }
template <> DEVINLINE void stv<bf16>(bf16* p, float v) { *p = f2bf(v); }

// ---------------------------------------------------------------- prepare
template <typename T>
__global__ __launch_bounds__(BLOCK) void norm_rope_rows_kernel(
    const T* __restrict__ src, int ld, int col, int n_heads, int head_dim,
    const float* __restrict__ norm_w, int norm_cols, float eps, int rot_off,
    int rot_dims, const double* __restrict__ freqs,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ table, int P, float* __restrict__ out,
    T* __restrict__ pool, int head_norm, int interleaved, float rot_mult,
    const T* __restrict__ mix_src, int mix_ld, int mix_col,
    const float* __restrict__ mix_lam) {
  __shared__ float red[NWAVE];
  __shared__ float head_rn[MAX_NORM_HEADS];
  const int t = blockIdx.x;
  const int N = n_heads * head_dim;
  const T* row = src + (int64_t)t * ld + col;
  float rn = 1.f;
  if (norm_w && head_norm) {
    // one statistic per head, the weight [head_dim] shared by the heads
    const int lane = threadIdx.x & (WAVE_SIZE - 1);
    for (int hd = threadIdx.x / WAVE_SIZE; hd < n_heads; hd += NWAVE) {
      float ss = 0.f;
      for (int e = lane; e < head_dim; e += WAVE_SIZE) {
        const float v = ldv<T>(row + hd * head_dim + e);
        ss += v * v;
      }
      ss = wave_reduce_sum(ss);
      if (lane == 0) head_rn[hd] = 1.0f / sqrtf(ss / (float)head_dim + eps);
    }
    __syncthreads();
  } else if (norm_w) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < norm_cols; c += BLOCK) {
      const float v = ldv<T>(row + c);
      ss += v * v;
    }
    const float tot = block_reduce_sum<NWAVE>(ss, red);
    rn = 1.0f / sqrtf(tot / (float)norm_cols + eps);
  }
  const int pos = tok_pos[t];
  const int half = rot_dims / 2;
  int64_t prow = 0;
  if (pool) {
    const int page = table[(int64_t)tok_seq[t] * P + pos / PAGE];
    prow = (int64_t)page * n_heads * PAGE + (pos % PAGE);
  }
  const float lam = mix_src ? mix_lam[0] : 0.f;
  for (int c = threadIdx.x; c < N; c += BLOCK) {
    const int hd = c / head_dim, e = c - hd * head_dim;
    float x = ldv<T>(row + c);
    if (norm_w) {
      if (head_norm) x = x * head_rn[hd] * norm_w[e];
      else if (c < norm_cols) x = x * rn * norm_w[c];
    }
    const int r = e - rot_off;
    if (r >= 0 && r < rot_dims) {
      // the pair's first member: r < half (halves) or r even (interleaved)
      const bool is_u = interleaved ? (r & 1) == 0 : r < half;
      const int i = interleaved ? r >> 1 : (r < half ? r : r - half);
      const int step = interleaved ? 1 : half;
      const int cp = is_u ? c + step : c - step;       // the pair's other
      float y = ldv<T>(row + cp);
      if (norm_w) {
        if (head_norm) y = y * head_rn[hd] * norm_w[cp - hd * head_dim];
        else if (cp < norm_cols) y = y * rn * norm_w[cp];
      }
      const double ang = (double)pos * freqs[i];
      const float cs = (float)cos(ang) * rot_mult;
      const float sn = (float)sin(ang) * rot_mult;
      // (u, v) -> (u cos - v sin, v cos + u sin); x is u or v
      x = is_u ? x * cs - y * sn : x * cs + y * sn;
    }
    // blend with the same token's row of another projection
    if (mix_src)
      x = (1.f - lam) * x +
          lam * ldv<T>(mix_src + (int64_t)t * mix_ld + mix_col + c);
    if (pool)
      stv<T>(pool + (prow + (int64_t)hd * PAGE) * head_dim + e, x);
    else
      out[(int64_t)t * N + c] = x;
  }
}

// -------------------------------------------------------------- attention
// lanes that cover one value row of V columns with 16-byte loads: the
// power of two at or above V / 8
__host__ __device__ inline int vec_lanes(int V) {
  int n = 1;
  while (n * 8 < V) n <<= 1;
  return n;
}

// sigmoid of the output gate of column c of head h of token t; 1 without
DEVINLINE float out_gate(const TlFlexExtra& ex, int64_t t, int h, int V,
                         int c) {
  if (!ex.gate) return 1.f;
  const int64_t i =
      t * ex.gate_ld + ex.gate_col + (ex.gate_heads ? h : h * V + c);
  const float g = ex.gate_f32 ? ((const float*)ex.gate)[i]
                              : bf2f(((const bf16*)ex.gate)[i]);
  return 1.f / (1.f + expf(-g));
}

// part row (key split z of token t, head h): m, l, acc[V]
template <typename TK, int HB, int VR, bool TALK>
__global__ __launch_bounds__(BLOCK) void flex_attn_row_kernel(
    const float* __restrict__ q, const TK* __restrict__ kpool,
    const TK* __restrict__ vpool, int vld, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const int* __restrict__ table, int P,
    const float* __restrict__ talk, void* __restrict__ out, int out_f32,
    float* __restrict__ part, int H, int G, int DK, int V, float scale,
    int window, int sink, float softcap, const float* __restrict__ sinks,
    TlFlexExtra ex) {
  extern __shared__ float lds[];
  const int t = blockIdx.x, h0 = blockIdx.y * HB;
  const int ns = gridDim.z, z = blockIdx.z;
  const int rep = H / G;
  const int g0 = h0 / rep;           // key group of this block's heads
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int KG = TALK ? G : 1;       // key heads a query row meets
  const int QD = KG * DK;
  // lds: qs[HB][KG*DK] | stat[NWAVE][HB][2] | acc[NWAVE][HB][V]
  float* qs = lds;
  float* stat = qs + HB * QD;
  float* accs = stat + NWAVE * HB * 2;

  const int seq = tok_seq[t], pos = tok_pos[t];
  const int* tab = table + (int64_t)seq * P;
  const float* qt = q + (int64_t)t * H * DK;
  for (int i = threadIdx.x; i < HB * QD; i += BLOCK) {
    const int b = i / QD, r = i - b * QD;
    if (!TALK) {
      qs[i] = qt[(h0 + b) * DK + r] * scale;
    } else {
      const int c = r / DK, d = r - c * DK;
      float acc = 0.f;
      for (int g = c * rep; g < (c + 1) * rep; ++g)
        acc += talk[(h0 + b) * H + g] * qt[g * DK + d];
      qs[i] = acc * scale;
    }
  }
  __syncthreads();

  // VR == 0: value rows are fetched with 16-byte loads (bf16 pools, value
  // size a multiple of 8): CPR lanes (the power of two at or above V / 8;
  // those beyond the row stay idle) cover one row, so one load instruction
  // brings 64 / CPR rows; a lane accumulates 8 columns for the keys of its
  // row group and the row groups meet through shuffles at the end
  constexpr int AC = VR == 0 ? 8 : VR;
  float m[HB], l[HB], a[HB][AC];
#pragma unroll
  for (int b = 0; b < HB; ++b) {
    m[b] = -INFINITY;
    l[b] = 0.f;
#pragma unroll
    for (int r = 0; r < AC; ++r) a[b][r] = 0.f;
  }
  const int lo = tl_flex_lo(pos, window, ex.chunk);
  const int first = (lo / WAVE_SIZE) * WAVE_SIZE;
  // kept prefix [0, kp) below the main range [lo, pos]: its tiles come first
  const int kp = min(ex.keep, lo);
  const int n_pre = (kp + WAVE_SIZE - 1) / WAVE_SIZE;
  const bool vec8 = sizeof(TK) == 2 && (DK % 8) == 0;
  for (int it = z * NWAVE + wave;; it += ns * NWAVE) {
    const bool pre = it < n_pre;
    const int j0 = pre ? it * WAVE_SIZE : first + (it - n_pre) * WAVE_SIZE;
    if (j0 > pos) break;
    const int rlo = pre ? 0 : lo, rhi = pre ? kp - 1 : pos;
    const int j = j0 + lane;
    const bool valid = j >= rlo && j <= rhi;
    // a 64-key tile lies inside ONE 128-position page
    const int64_t page_row = (int64_t)tab[j0 / PAGE] * G * PAGE + (j0 % PAGE);
    float s[HB];
#pragma unroll
    for (int b = 0; b < HB; ++b) s[b] = 0.f;
    if (valid) {
      for (int c = 0; c < KG; ++c) {
        const int g = TALK ? c : g0;
        const TK* kr = kpool + (page_row + (int64_t)g * PAGE + lane) * DK;
        const float* qc = qs + c * DK;
        if (vec8) {
          const bf16x8* k8 = reinterpret_cast<const bf16x8*>(kr);
          for (int d8 = 0; d8 < DK / 8; ++d8) {
            const bf16x8 kk = k8[d8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float kd = bf2f(kk.v[e]);
#pragma unroll
              for (int b = 0; b < HB; ++b)
                s[b] += qc[b * QD + d8 * 8 + e] * kd;
            }
          }
        } else {
          for (int d = 0; d < DK; ++d) {
            const float kd = ldv<TK>(kr + d);
#pragma unroll
            for (int b = 0; b < HB; ++b) s[b] += qc[b * QD + d] * kd;
          }
        }
      }
    }
    float p[HB];
    const float* brow =
        ex.bias ? ex.bias + (int64_t)h0 * ex.nb + min(max(pos - j, 0), ex.nb - 1)
                : nullptr;
#pragma unroll
    for (int b = 0; b < HB; ++b) {
      float sc = softcap > 0.f ? softcap * tanhf(s[b] / softcap) : s[b];
      if (brow && valid) sc += brow[(int64_t)b * ex.nb];
      const float sv = valid ? sc : -INFINITY;
      const float nm = fmaxf(m[b], wave_reduce_max(sv));
      // nm is finite: every tile of the loop holds at least one valid key
      const float c = expf(m[b] - nm);
      p[b] = valid ? expf(sv - nm) : 0.f;
      l[b] = l[b] * c + wave_reduce_sum(p[b]);
      m[b] = nm;
#pragma unroll
      for (int r = 0; r < AC; ++r) a[b][r] *= c;
    }
    const int jb = max(0, rlo - j0), je = min(WAVE_SIZE, rhi + 1 - j0);
    const TK* vtile = vpool + (page_row + (int64_t)g0 * PAGE) * vld;
    if constexpr (VR == 0) {
      const int CPR = vec_lanes(V), KGR = WAVE_SIZE / CPR;
      const int cc = lane & (CPR - 1), kg = lane / CPR;
      const bool col_on = cc * 8 < V;
      for (int jj0 = jb; jj0 < je; jj0 += 4 * KGR) {
        bf16x8 vv[4];
        int jk[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          jk[u] = jj0 + u * KGR + kg;
          if (jk[u] < je && col_on)
            vv[u] = *reinterpret_cast<const bf16x8*>(
                vtile + (int64_t)jk[u] * vld + cc * 8);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bool on = jk[u] < je && col_on;
          const int src = min(jk[u], WAVE_SIZE - 1);
#pragma unroll
          for (int b = 0; b < HB; ++b) {
            const float ws = __shfl(p[b], src, WAVE_SIZE);
            if (on) {
#pragma unroll
              for (int e = 0; e < 8; ++e) a[b][e] += ws * bf2f(vv[u].v[e]);
            }
          }
        }
      }
      continue;
    }
    // eight keys' value rows are loaded before they are used, so their
    // latencies overlap instead of adding up
    for (int jj0 = jb; jj0 < je; jj0 += 8) {
      float vv[8][AC];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const TK* vr = vtile + (int64_t)(jj0 + u) * vld;
#pragma unroll
        for (int r = 0; r < AC; ++r) {
          const int c = lane + r * WAVE_SIZE;
          vv[u][r] = (jj0 + u < je && c < V) ? ldv<TK>(vr + c) : 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        // lanes past the range hold weight 0
        const int jj = min(jj0 + u, WAVE_SIZE - 1);
#pragma unroll
        for (int b = 0; b < HB; ++b) {
          const float w = jj0 + u < je ? __shfl(p[b], jj, WAVE_SIZE) : 0.f;
#pragma unroll
          for (int r = 0; r < AC; ++r) a[b][r] += w * vv[u][r];
        }
      }
    }
  }
  // a wave whose tiles were all beyond the range keeps m = -inf, l = 0
#pragma unroll
  for (int b = 0; b < HB; ++b) {
    if (lane == 0) {
      stat[(wave * HB + b) * 2 + 0] = m[b];
      stat[(wave * HB + b) * 2 + 1] = l[b];
    }
    if constexpr (VR == 0) {
      const int CPR = vec_lanes(V);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float s = a[b][e];
        for (int off = CPR; off < WAVE_SIZE; off <<= 1)
          s += __shfl_xor(s, off, WAVE_SIZE);
        if (lane < CPR && lane * 8 < V)
          accs[(wave * HB + b) * V + lane * 8 + e] = s;
      }
    } else {
#pragma unroll
      for (int r = 0; r < AC; ++r) {
        const int c = lane + r * WAVE_SIZE;
        if (c < V) accs[(wave * HB + b) * V + c] = a[b][r];
      }
    }
  }
  __syncthreads();
  for (int b = 0; b < HB; ++b) {
    float M = -INFINITY;
    for (int w = 0; w < NWAVE; ++w) M = fmaxf(M, stat[(w * HB + b) * 2]);
    float f[NWAVE], L = 0.f;
    if (ns > 1) {
      // partial of this key split; an empty split stores m = -inf, l = 0
      for (int w = 0; w < NWAVE; ++w) {
        const float mw = stat[(w * HB + b) * 2];
        f[w] = (mw == -INFINITY) ? 0.f : expf(mw - M);
        L += f[w] * stat[(w * HB + b) * 2 + 1];
      }
      float* pr = part + (((int64_t)t * H + h0 + b) * ns + z) * (2 + V);
      if (threadIdx.x == 0) {
        pr[0] = M;
        pr[1] = L;
      }
      for (int c = threadIdx.x; c < V; c += BLOCK) {
        float A = 0.f;
        for (int w = 0; w < NWAVE; ++w) A += f[w] * accs[(w * HB + b) * V + c];
        pr[2 + c] = A;
      }
      continue;
    }
    const float sl = sinks ? sinks[h0 + b] : 0.f;   // the sink's logit
    if (sink) M = fmaxf(M, sl);
    for (int w = 0; w < NWAVE; ++w) {
      const float mw = stat[(w * HB + b) * 2];
      f[w] = (mw == -INFINITY) ? 0.f : expf(mw - M);
      L += f[w] * stat[(w * HB + b) * 2 + 1];
    }
    if (sink) L += expf(sl - M);
    for (int c = threadIdx.x; c < V; c += BLOCK) {
      float A = 0.f;
      for (int w = 0; w < NWAVE; ++w) A += f[w] * accs[(w * HB + b) * V + c];
      const int64_t o = ((int64_t)t * H + h0 + b) * V + c;
      const float r = A / L * out_gate(ex, t, h0 + b, V, c);
      if (out_f32)
        ((float*)out)[o] = r;
      else
        ((bf16*)out)[o] = f2bf(r);
    }
  }
}

// one block per (token, head): merge the key splits
__global__ __launch_bounds__(BLOCK) void flex_attn_merge_kernel(
    const float* __restrict__ part, void* __restrict__ out, int out_f32,
    int ns, int V, int sink, int H, const float* __restrict__ sinks,
    TlFlexExtra ex) {
  const int64_t row = blockIdx.x;
  const float* pr = part + row * ns * (2 + V);
  float M = -INFINITY;
  for (int z = 0; z < ns; ++z) M = fmaxf(M, pr[z * (2 + V)]);
  const float sl = sinks ? sinks[row % H] : 0.f;
  if (sink) M = fmaxf(M, sl);
  float L = sink ? expf(sl - M) : 0.f;
  for (int z = 0; z < ns; ++z) {
    const float mz = pr[z * (2 + V)];
    L += (mz == -INFINITY ? 0.f : expf(mz - M)) * pr[z * (2 + V) + 1];
  }
  for (int c = threadIdx.x; c < V; c += BLOCK) {
    float A = 0.f;
    for (int z = 0; z < ns; ++z) {
      const float mz = pr[z * (2 + V)];
      A += (mz == -INFINITY ? 0.f : expf(mz - M)) * pr[z * (2 + V) + 2 + c];
    }
    const float r = A / L * out_gate(ex, row / H, (int)(row % H), V, c);
    if (out_f32)
      ((float*)out)[row * V + c] = r;
    else
      ((bf16*)out)[row * V + c] = f2bf(r);
  }
}

template <typename TK, int HB, int VR>
void launch_rows(bool has_talk, dim3 grid, size_t smem, hipStream_t stream,
                 const float* q, const TK* kpool, const TK* vpool, int vld,
                 const int* tok_seq, const int* tok_pos, const int* table,
                 int P, const float* talk, void* out, int out_f32,
                 float* part, int H, int G, int DK, int V, float scale,
                 int window, int sink, float softcap, const float* sinks,
                 const TlFlexExtra& ex) {
  if (has_talk)
    hipLaunchKernelGGL((flex_attn_row_kernel<TK, HB, VR, true>), grid,
                       dim3(BLOCK), smem, stream, q, kpool, vpool, vld,
                       tok_seq, tok_pos, table, P, talk, out, out_f32, part,
                       H, G, DK, V, scale, window, sink, softcap, sinks, ex);
  else
    hipLaunchKernelGGL((flex_attn_row_kernel<TK, HB, VR, false>), grid,
                       dim3(BLOCK), smem, stream, q, kpool, vpool, vld,
                       tok_seq, tok_pos, table, P, talk, out, out_f32, part,
                       H, G, DK, V, scale, window, sink, softcap, sinks, ex);
}

size_t rows_smem(bool has_talk, int hb, int G, int DK, int V) {
  return sizeof(float) * ((size_t)hb * (has_talk ? G : 1) * DK +
                          (size_t)NWAVE * hb * 2 + (size_t)NWAVE * hb * V);
}

}  // namespace

extern "C" {

void tl_norm_rope_rows(const void* src, int ld, int col, int n_heads,
                       int head_dim, const void* norm_w, int norm_cols,
                       float eps, int rot_off, int rot_dims,
                       const void* freqs, const void* tok_seq,
                       const void* tok_pos, const void* table, int P, int T,
                       void* out, void* pool, int is_f32, int head_norm,
                       int interleaved, float rot_mult, const void* mix_src,
                       int mix_ld, int mix_col, const void* mix_lam,
                       hipStream_t stream) {
  if (T <= 0) return;
  dim3 grid(T), block(BLOCK);
  if (is_f32)
    hipLaunchKernelGGL(norm_rope_rows_kernel<float>, grid, block, 0, stream,
                       (const float*)src, ld, col, n_heads, head_dim,
                       (const float*)norm_w, norm_cols, eps, rot_off,
                       rot_dims, (const double*)freqs, (const int*)tok_seq,
                       (const int*)tok_pos, (const int*)table, P,
                       (float*)out, (float*)pool, head_norm, interleaved,
                       rot_mult, (const float*)mix_src, mix_ld, mix_col,
                       (const float*)mix_lam);
  else
    hipLaunchKernelGGL(norm_rope_rows_kernel<bf16>, grid, block, 0, stream,
                       (const bf16*)src, ld, col, n_heads, head_dim,
                       (const float*)norm_w, norm_cols, eps, rot_off,
                       rot_dims, (const double*)freqs, (const int*)tok_seq,
                       (const int*)tok_pos, (const int*)table, P,
                       (float*)out, (bf16*)pool, head_norm, interleaved,
                       rot_mult, (const bf16*)mix_src, mix_ld, mix_col,
                       (const float*)mix_lam);
}

// heads per block for a shape: the largest of 8, 4, 2, 1 that divides the
// heads per key group and fits the register and LDS budgets; 0 if none
static int heads_per_block(int H, int G, int DK, int V, int has_talk,
                           int hb_max) {
  if (V > 512 || G <= 0 || H % G != 0) return 0;
  const int vr = (V + WAVE_SIZE - 1) / WAVE_SIZE;
  const int vrr = vr <= 1 ? 1 : vr <= 2 ? 2 : vr <= 4 ? 4 : 8;
  for (int hb = 8; hb >= 1; hb >>= 1) {
    if (hb > hb_max && hb > 1) continue;
    if ((H / G) % hb != 0 || hb * vrr > 32) continue;
    if (rows_smem(has_talk != 0, hb, G, DK, V) <= 64 * 1024) return hb;
  }
  return 0;
}

int tl_flex_attn_heads_per_block(int H, int G, int DK, int V, int has_talk) {
  return heads_per_block(H, G, DK, V, has_talk, 8);
}

// returns 0 on success, 1 if the shape is outside what the kernel serves.
// hb_max caps the heads per block: few rows (decoding) want many small
// blocks, many rows want the key and value loads shared by more heads.
int tl_flex_attn_rows(const void* q, const void* kpool, const void* vpool,
                      int vld, const void* tok_seq, const void* tok_pos,
                      const void* table, int P, const void* talk, void* out,
                      int out_f32, void* part, int ns, int T, int H, int G,
                      int DK, int V, float scale, int window, int sink,
                      int pool_f32, int hb_max, float softcap,
                      const void* sinks, TlFlexExtra ex, hipStream_t stream) {
  if (T <= 0) return 0;
  const bool has_talk = talk != nullptr;
  static const bool no_vec = getenv("TL_NO_VEC_VALUES") != nullptr;
  const int hb = heads_per_block(H, G, DK, V, has_talk ? 1 : 0, hb_max);
  if (hb == 0 || ns < 1 || (ns > 1 && !part)) return 1;
  const int vr = (V + WAVE_SIZE - 1) / WAVE_SIZE;
  const size_t smem = rows_smem(has_talk, hb, G, DK, V);
  dim3 grid(T, H / hb, ns);
#define TL_FA(TT, HBB, VRR)                                                  \
  launch_rows<TT, HBB, VRR>(has_talk, grid, smem, stream, (const float*)q,   \
                            (const TT*)kpool, (const TT*)vpool, vld,         \
                            (const int*)tok_seq, (const int*)tok_pos,        \
                            (const int*)table, P, (const float*)talk, out,   \
                            out_f32, (float*)part, H, G, DK, V, scale,       \
                            window, sink, softcap, (const float*)sinks, ex)
#define TL_FA_V(TT, HBB)                     \
  if (vr <= 1) TL_FA(TT, HBB, 1);            \
  else if (vr <= 2) TL_FA(TT, HBB, 2);       \
  else if (vr <= 4) TL_FA(TT, HBB, 4);       \
  else if (HBB <= 4) TL_FA(TT, (HBB <= 4 ? HBB : 4), 8);
#define TL_FA_H(TT)                    \
  if (hb == 8) { TL_FA_V(TT, 8) }      \
  else if (hb == 4) { TL_FA_V(TT, 4) } \
  else if (hb == 2) { TL_FA_V(TT, 2) } \
  else { TL_FA_V(TT, 1) }
  // 16-byte value loads: bf16 rows of a multiple of 8 columns, 16-byte
  // aligned
  const bool vec = !pool_f32 && V % 8 == 0 && V >= 8 &&
                   vec_lanes(V) <= WAVE_SIZE && vld % 8 == 0 && !no_vec;
  if (pool_f32) {
    TL_FA_H(float)
  } else if (vec) {
    if (hb == 8) TL_FA(bf16, 8, 0);
    else if (hb == 4) TL_FA(bf16, 4, 0);
    else if (hb == 2) TL_FA(bf16, 2, 0);
    else TL_FA(bf16, 1, 0);
  } else {
    TL_FA_H(bf16)
  }
#undef TL_FA_H
#undef TL_FA_V
#undef TL_FA
  if (ns > 1)
    hipLaunchKernelGGL(flex_attn_merge_kernel, dim3(T * H), dim3(BLOCK), 0,
                       stream, (const float*)part, out, out_f32, ns, V, sink, H,
                       (const float*)sinks, ex);
  return 0;
}

}  // extern "C"
