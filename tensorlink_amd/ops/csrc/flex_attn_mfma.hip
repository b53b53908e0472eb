// Flexible paged attention for prompt portions on MFMA (gfx950, bf16).
//
// One block = 64 consecutive query tokens of one sequence (16 per wave) and
// one query head. The products are arranged as in the framework's other
// tile kernels so that nothing is transposed through LDS:
//   S^T[key][q] = K Q^T      A = K rows (16 keys x 32 d), B = Q^T
//   O^T[v][q]  += V^T P^T    A = V^T (16 v x 32 keys),    B = P^T
// and the score fragment of two 16-key tiles is directly the B operand of
// the next product; the online-softmax rescale is lane-local.
//
// Options: a sliding window (key tiles wholly outside a wave's window are
// skipped), a sink (one more unit of weight in the denominator, folded in
// at the end), values that are the leading columns of the key row (latent
// attention, one shared key head), and mixing of the heads' scores before
// the softmax. The mixing is linear in the scores, and heads of one key
// group share their key, so
//     s'_h = sum_g T[h,g] q_g . k_grp(g) = sum_c (sum_{g in c} T[h,g] q_g) . k_c
// : the mixed score of head h is ONE dot product between a mixed query
// [q~_h,1 | ... | q~_h,G] and the G key heads' rows side by side.
// tl_stage_queries builds those mixed queries (or plain copies) in bf16
// from the fp32 normed/rotated queries; the tile kernel then only sees a
// query of KG*DK columns that meets KG key heads.
// Further options (TlFlexExtra): keys of the query's own chunk only, a kept
// prefix (its key tiles are walked before the window's), a learned distance
// bias from a per-head table indexed by i - j, a sigmoid output gate per
// column or per head applied to the normalised row.
// Scores, softmax statistics and accumulators are fp32; P is rounded to
// bf16 only as the MFMA operand.

#include "common.hpp"
#include "flex_attn.hpp"

namespace {

constexpr int PAGE = 128;
constexpr int QT = 64;           // queries per block
constexpr int KT = 64;           // keys per round
constexpr int VLD = KT + 8;      // LDS row stride of V^T (bf16 elements)

using f32x4 = __attribute__((ext_vector_type(4))) float;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));

DEVINLINE bf16x8_t zero8() {
  bf16x8_t z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// tanh through one fast exponential and one fast reciprocal:
// 1 - 2 / (exp(2x) + 1); exact at both ends (exp -> 0 or inf), absolute
// error of a few 1e-7 elsewhere, far below the bf16 rounding of P
DEVINLINE float fast_tanh(float x) {
  return 1.f - 2.f * __frcp_rn(__expf(2.f * x) + 1.f);
}

DEVINLINE float quad_max(float x) {
  x = fmaxf(x, __shfl_xor(x, 16, WAVE_SIZE));
  return fmaxf(x, __shfl_xor(x, 32, WAVE_SIZE));
}
DEVINLINE float quad_sum(float x) {
  x += __shfl_xor(x, 16, WAVE_SIZE);
  return x + __shfl_xor(x, 32, WAVE_SIZE);
}

// out[t][h][c][d] = sum_{g in key group c} talk[h][g] q[t][g][d]  (KG = G)
// or a plain copy of q[t][h][:]                                  (KG = 1)
__global__ __launch_bounds__(256) void stage_queries_kernel(
    const float* __restrict__ q, const float* __restrict__ talk,
    bf16* __restrict__ out, int H, int G, int DK) {
  const int t = blockIdx.x;
  const float* qr = q + (int64_t)t * H * DK;
  if (!talk) {
    for (int i = threadIdx.x; i < H * DK; i += 256)
      out[(int64_t)t * H * DK + i] = f2bf(qr[i]);
    return;
  }
  const int rep = H / G;
  const int QD = G * DK;
  for (int i = threadIdx.x; i < H * QD; i += 256) {
    const int h = i / QD, r = i - h * QD;
    const int c = r / DK, d = r - c * DK;
    float a = 0.f;
    for (int g = c * rep; g < (c + 1) * rep; ++g)
      a += talk[h * H + g] * qr[g * DK + d];
    out[(int64_t)t * H * QD + i] = f2bf(a);
  }
}

template <int QCMAX, int VTMAX>
__global__ __launch_bounds__(256) void flex_attn_tile_kernel(
    const bf16* __restrict__ q,      // [T][H][KG*DK]
    const bf16* __restrict__ kpool, const bf16* __restrict__ vpool, int vld,
    const int* __restrict__ tiles,   // [n][4]: seq, first token, count, pos
    const int* __restrict__ table, int P, void* __restrict__ out,
    int out_f32, int H, int G, int KG, int DK, int V, float scale,
    int window, int sink, float softcap, const float* __restrict__ sinks,
    TlFlexExtra ex) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16* vt_lds = reinterpret_cast<bf16*>(smem_raw);     // [V][VLD]

  const int h = blockIdx.y;
  const int gv = h / (H / G);
  const int seq = tiles[blockIdx.x * 4 + 0];
  const int tok0 = tiles[blockIdx.x * 4 + 1];
  const int n = tiles[blockIdx.x * 4 + 2];
  const int p0 = tiles[blockIdx.x * 4 + 3];
  const int* tab = table + (int64_t)seq * P;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, quad = lane >> 4;
  const int dch = (DK + 31) / 32;          // 32-wide chunks per key head
  const int qc = KG * dch;
  const int QD = KG * DK;
  const int nvt = V / 16;

  const int qi = wave * 16 + col;
  const bool q_valid = qi < n;
  const int qcl = min(qi, n - 1);
  const int tok = tok0 + qcl;
  const int qpos = p0 + qcl;
  const int k_end = p0 + n;                             // keys of the block
  const int wave_first = p0 + min(wave * 16, n - 1);
  const int wave_last = p0 + min(wave * 16 + 15, n - 1);
  const bool wave_on = wave * 16 < n;
  // lo() grows with the position: the block's oldest key is its first
  // query's, a wave's oldest its first query's
  const int k_begin = (tl_flex_lo(p0, window, ex.chunk) / KT) * KT;
  const int wave_old = tl_flex_lo(wave_first, window, ex.chunk);
  const int lo_q = tl_flex_lo(qpos, window, ex.chunk);
  const int keep = ex.keep;
  // kept prefix below the main range: rounds [0, n_pre) walk its tiles
  const int n_pre = (min(keep, k_begin) + KT - 1) / KT;
  const int n_round = n_pre + (k_end - k_begin + KT - 1) / KT;
  const float* brow = ex.bias ? ex.bias + (int64_t)h * ex.nb : nullptr;

  bf16x8_t qf[QCMAX];
#pragma unroll
  for (int i = 0; i < QCMAX; ++i) {
    qf[i] = zero8();
    if (i < qc) {
      const int kc = i / dch, c = i - kc * dch;
      const int d = c * 32 + quad * 8;
      if (d < DK)
        qf[i] = *reinterpret_cast<const bf16x8_t*>(
            q + ((int64_t)tok * H + h) * QD + kc * DK + d);
    }
  }

  f32x4 acc[VTMAX];
#pragma unroll
  for (int vt = 0; vt < VTMAX; ++vt) acc[vt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float mrun = -INFINITY, lrun = 0.f;
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;

  const int vchunks = V / 8;                // 16-byte chunks per value row
  for (int rd = 0; rd < n_round; ++rd) {
    const int k0 = rd < n_pre ? rd * KT : k_begin + (rd - n_pre) * KT;
    __syncthreads();                        // previous round's reads done
    // lane -> key fastest: the 2-byte transposed stores of a wave then
    // fall into consecutive LDS words instead of a few banks
    for (int i = threadIdx.x; i < KT * vchunks; i += 256) {
      const int c8 = i / KT, kk = i - c8 * KT;
      const int j = min(k0 + kk, k_end - 1);
      const int page = tab[j / PAGE];
      const bf16x8 v8 = *reinterpret_cast<const bf16x8*>(
          vpool + (((int64_t)page * G + gv) * PAGE + (j % PAGE)) * vld +
          c8 * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) vt_lds[(c8 * 8 + e) * VLD + kk] = v8.v[e];
    }
    __syncthreads();
    // wave-uniform skips: keys after the wave's last query, or older than
    // the range of its first and not of the kept prefix
    if (!wave_on || k0 > wave_last ||
        (k0 + KT - 1 < wave_old && k0 >= keep))
      continue;

#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int kb = k0 + sub * 32;
      if (kb > wave_last) break;
      if (kb + 31 < wave_old && kb >= keep) continue;
      // ---- S^T for two 16-key tiles
      f32x4 st[2];
#pragma unroll
      for (int t16 = 0; t16 < 2; ++t16) {
        const int j = min(kb + t16 * 16 + col, k_end - 1);
        const int64_t prow = (int64_t)tab[j / PAGE] * G * PAGE + (j % PAGE);
        f32x4 sacc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < QCMAX; ++i)
          if (i < qc) {
            const int kc = i / dch, c = i - kc * dch;
            const int d = c * 32 + quad * 8;
            const int g = KG == 1 ? gv : kc;
            const bf16x8_t kf =
                (d < DK) ? *reinterpret_cast<const bf16x8_t*>(
                               kpool + (prow + (int64_t)g * PAGE) * DK + d)
                         : zero8();
            sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[i], sacc,
                                                           0, 0, 0);
          }
        st[t16] = sacc;
      }
      // ---- online softmax (query = col; keys over r and quads)
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int t16 = 0; t16 < 2; ++t16)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = kb + t16 * 16 + quad * 4 + r;
          const bool ok = key <= qpos && (key >= lo_q || key < keep);
          float s = st[t16][r] * scale;
          if (softcap > 0.f) s = softcap * fast_tanh(s * inv_cap);
          if (brow) s += brow[min(max(qpos - key, 0), ex.nb - 1)];
          s = ok ? s : -INFINITY;
          sv[t16 * 4 + r] = s;
          mx = fmaxf(mx, s);
        }
      mx = quad_max(mx);
      const float m_new = fmaxf(mrun, mx);
      // a query may see none of this sub-tile's keys and none before
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float corr = __expf(mrun - m_safe);
      mrun = m_new;
      float ps = 0.f;
      bf16x8_t pf;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float p = __expf(sv[i] - m_safe);
        ps += p;
        pf[i] = (__bf16)p;
      }
      lrun = lrun * corr + ps;
#pragma unroll
      for (int vt = 0; vt < VTMAX; ++vt)
        if (vt < nvt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[vt][r] *= corr;
        }
      // ---- O^T += V^T P^T
#pragma unroll
      for (int vt = 0; vt < VTMAX; ++vt)
        if (vt < nvt) {
          const bf16* vr = vt_lds + (vt * 16 + col) * VLD + sub * 32 + quad * 4;
          const bf16x4_t lo = *reinterpret_cast<const bf16x4_t*>(vr);
          const bf16x4_t hi = *reinterpret_cast<const bf16x4_t*>(vr + 16);
          bf16x8_t vf;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            vf[i] = lo[i];
            vf[4 + i] = hi[i];
          }
          acc[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc[vt],
                                                            0, 0, 0);
        }
    }
  }

  if (!wave_on) return;
  float l = quad_sum(lrun);
  // every query sees itself, so mrun is finite here
  float f = 1.f;
  if (sink) {
    const float sl = sinks ? sinks[h] : 0.f;      // the sink's logit
    const float m_fin = fmaxf(mrun, sl);
    f = __expf(mrun - m_fin);
    l = l * f + __expf(sl - m_fin);
  }
  const float inv = f / l;
  if (q_valid) {
    const int64_t o0 = ((int64_t)tok * H + h) * V;
#pragma unroll
    for (int vt = 0; vt < VTMAX; ++vt)
      if (vt < nvt) {
        float g4[4] = {1.f, 1.f, 1.f, 1.f};
        if (ex.gate) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int64_t gi =
                (int64_t)tok * ex.gate_ld + ex.gate_col +
                (ex.gate_heads ? h : h * V + vt * 16 + quad * 4 + r);
            const float g = ex.gate_f32 ? ((const float*)ex.gate)[gi]
                                        : bf2f(((const bf16*)ex.gate)[gi]);
            g4[r] = 1.f / (1.f + __expf(-g));
          }
        }
        if (out_f32) {
          float* orow = (float*)out + o0 + vt * 16 + quad * 4;
#pragma unroll
          for (int r = 0; r < 4; ++r) orow[r] = acc[vt][r] * inv * g4[r];
        } else {
          bf16x4_t o4;
#pragma unroll
          for (int r = 0; r < 4; ++r)
            o4[r] = (__bf16)(acc[vt][r] * inv * g4[r]);
          *reinterpret_cast<bf16x4_t*>((bf16*)out + o0 + vt * 16 + quad * 4) =
              o4;
        }
      }
  }
}

}  // namespace

extern "C" {

// 1 if tl_flex_attn_tiles serves the shape
int tl_flex_attn_tiles_ok(int H, int G, int KG, int DK, int V) {
  if (G <= 0 || H % G != 0 || (KG != 1 && KG != G)) return 0;
  if (DK % 8 != 0 || V % 16 != 0 || V > 256) return 0;
  if (KG * ((DK + 31) / 32) > 20) return 0;
  return 1;
}

void tl_stage_queries(const void* q, const void* talk, void* out, int T,
                      int H, int G, int DK, hipStream_t stream) {
  if (T <= 0) return;
  hipLaunchKernelGGL(stage_queries_kernel, dim3(T), dim3(256), 0, stream,
                     (const float*)q, (const float*)talk, (bf16*)out, H, G,
                     DK);
}

// returns 0 on success, 1 if the shape is outside what this kernel serves
int tl_flex_attn_tiles(const void* q, const void* kpool, const void* vpool,
                       int vld, const void* tiles, int n_tiles,
                       const void* table, int P, void* out, int out_f32,
                       int H, int G, int KG, int DK, int V, float scale,
                       int window, int sink, float softcap, const void* sinks,
                       TlFlexExtra ex, hipStream_t stream) {
  if (!tl_flex_attn_tiles_ok(H, G, KG, DK, V) || vld % 8 != 0 ||
      n_tiles <= 0)
    return 1;
  const size_t smem = sizeof(bf16) * (size_t)V * VLD;
  dim3 grid(n_tiles, H), block(256);
  const int qc = KG * ((DK + 31) / 32), nvt = V / 16;
#define TL_FT_LAUNCH(QCC, VTM)                                               \
  hipLaunchKernelGGL((flex_attn_tile_kernel<QCC, VTM>), grid, block, smem,   \
                     stream, (const bf16*)q, (const bf16*)kpool,             \
                     (const bf16*)vpool, vld, (const int*)tiles,             \
                     (const int*)table, P, out, out_f32, H, G, KG, DK, V,    \
                     scale, window, sink, softcap, (const float*)sinks, ex)
#define TL_FT_V(QCC)                          \
  if (nvt <= 4) TL_FT_LAUNCH(QCC, 4);         \
  else if (nvt <= 8) TL_FT_LAUNCH(QCC, 8);    \
  else TL_FT_LAUNCH(QCC, 16);
  if (qc <= 2) { TL_FT_V(2) }
  else if (qc <= 4) { TL_FT_V(4) }
  else if (qc <= 8) { TL_FT_V(8) }
  else if (qc <= 12) { TL_FT_V(12) }
  else { TL_FT_V(20) }
#undef TL_FT_V
#undef TL_FT_LAUNCH
  return 0;
}

}  // extern "C"
