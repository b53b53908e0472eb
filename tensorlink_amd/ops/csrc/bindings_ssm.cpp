// Python bindings for the layer-norm layered family's kernels: layer norm,
// input convolution fused with the norm, post-layer-norm residual add,
// PolyNorm, grouped gated RMS, short convolution + rotation + page scatter,
// and the selective state-space scan. Host-side glue and shape checks only;
// registered into the main module by register_ssm_ops().

#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
int tl_ln_canon_tile();
int tl_conv_rope_tile();
void tl_layer_norm_rows(const void* x, const void* w, void* out, int64_t rows,
                        int W, float eps, int out_f32, hipStream_t stream);
void tl_ln_canon(const void* X, const void* w, const void* taps, void* hist,
                 const void* tiles, int n_tiles, const void* cu,
                 const void* slots, const void* pos0, void* out, int W, int K,
                 float eps, int out_f32, hipStream_t stream);
void tl_postln_add(void* X, const void* y, const void* y2, const void* w,
                   const void* wy, const void* wy2, int64_t rows, int W,
                   float eps, int is_f32, hipStream_t stream);
void tl_polynorm(const void* z, const void* coef, void* out, int64_t rows,
                 int N, float eps, int is_f32, hipStream_t stream);
void tl_gated_group_rms(const void* y, const void* gate, int ldg, int gate_col,
                        const void* w, void* out, int64_t rows, int N,
                        int groups, float eps, int is_f32, hipStream_t stream);
int tl_conv_rope_rows(const void* src, int ld, int col, int n_heads, int D,
                      const void* taps, const void* bias, int act_silu,
                      void* hist, int K, int rot_dims, const void* freqs,
                      float mult, const void* tiles, int n_tiles,
                      const void* cu, const void* slots, const void* pos0,
                      const void* table, int P, void* out, void* pool,
                      void* raw_pool, int pool_heads, int is_f32,
                      hipStream_t stream);
int tl_ssd_scan(const void* xbc, int ldx, int x_off, int b_off, int c_off,
                const void* dt_src, int ldd, int dt_col, const void* dt_bias,
                const void* A_log, const void* skip, void* S, const void* cu,
                const void* slots, const void* pos0, void* out, int B, int H,
                int G, int N, int P, int dt_f32, hipStream_t stream);
void tl_ssd_chunk_prep(const void* xbc, int ldx, int x_off, int b_off,
                       int c_off, const void* dt_src, int ldd, int dt_col,
                       const void* dt_bias, const void* A_log,
                       const void* cu_c, void* Cs, void* Cd, void* Bs,
                       void* Bw, void* Xd, void* Lc, void* tot, int NC, int H,
                       int G, int N, int P, int C, int dt_f32,
                       hipStream_t stream);
void tl_ssd_decay_mask(void* A, const void* Lc, int NCH, int C,
                       hipStream_t stream);
void tl_ssd_chain(void* U, void* S, const void* tot, const void* chunk_base,
                  const void* n_chunks, const void* slots, const void* pos0,
                  int B, int H, int NP, hipStream_t stream);
}

namespace {

using torch::Tensor;

hipStream_t ssm_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define SSM_IN(t)                                                    \
  TORCH_CHECK((t).is_cuda(), #t " must be on GPU");                  \
  TORCH_CHECK((t).is_contiguous(), #t " must be contiguous")
#define SSM_F32(t) \
  SSM_IN(t);       \
  TORCH_CHECK((t).scalar_type() == torch::kFloat, #t " must be fp32")
#define SSM_I32(t) \
  SSM_IN(t);       \
  TORCH_CHECK((t).scalar_type() == torch::kInt, #t " must be int32")

int ssm_is_f32(const Tensor& t) {
  TORCH_CHECK(t.scalar_type() == torch::kFloat ||
                  t.scalar_type() == torch::kBFloat16,
              "activations must be fp32 or bf16");
  return t.scalar_type() == torch::kFloat ? 1 : 0;
}

// the ragged step: tiles [n, 4], cu [B+1], slots [B], pos0 [B]
void check_step(const Tensor& tiles, const Tensor& cu, const Tensor& slots,
                const Tensor& pos0, int64_t n_slots) {
  SSM_I32(tiles);
  SSM_I32(cu);
  SSM_I32(slots);
  SSM_I32(pos0);
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 4, "tiles must be [n, 4]");
  TORCH_CHECK(cu.numel() == slots.numel() + 1 && pos0.numel() == slots.numel(),
              "ragged metadata");
  (void)n_slots;
}

Tensor layer_norm_rows(Tensor x, Tensor w, double eps, bool out_f32) {
  SSM_F32(x);
  SSM_F32(w);
  TORCH_CHECK(x.dim() == 2 && w.numel() == x.size(1), "x [T, W], w [W]");
  auto out = torch::empty_like(
      x, x.options().dtype(out_f32 ? torch::kFloat : torch::kBFloat16));
  tl_layer_norm_rows(x.data_ptr(), w.data_ptr(), out.data_ptr(), x.size(0),
                     (int)x.size(1), (float)eps, out_f32 ? 1 : 0,
                     ssm_stream());
  return out;
}

Tensor ln_canon(Tensor X, Tensor w, double eps, Tensor taps, Tensor hist,
                Tensor tiles, Tensor cu, Tensor slots, Tensor pos0,
                bool out_f32) {
  SSM_F32(X);
  SSM_F32(w);
  SSM_F32(taps);
  SSM_F32(hist);
  check_step(tiles, cu, slots, pos0, hist.size(0));
  TORCH_CHECK(X.dim() == 2, "X must be [T, W]");
  const int W = X.size(1);
  TORCH_CHECK(taps.dim() == 2 && taps.size(0) == W && w.numel() == W,
              "taps must be [W, K]");
  const int K = taps.size(1);
  TORCH_CHECK(K >= 1 && K - 1 <= tl_ln_canon_tile(), "too many taps");
  TORCH_CHECK(hist.dim() == 3 && hist.size(1) == K - 1 && hist.size(2) == W,
              "history must be [slots, K-1, W]");
  auto out = torch::empty_like(
      X, X.options().dtype(out_f32 ? torch::kFloat : torch::kBFloat16));
  tl_ln_canon(X.data_ptr(), w.data_ptr(), taps.data_ptr(), hist.data_ptr(),
              tiles.data_ptr(), (int)tiles.size(0), cu.data_ptr(),
              slots.data_ptr(), pos0.data_ptr(), out.data_ptr(), W, K,
              (float)eps, out_f32 ? 1 : 0, ssm_stream());
  return out;
}

void postln_add(Tensor X, Tensor y, Tensor w, double eps,
                c10::optional<Tensor> y2, c10::optional<Tensor> wy,
                c10::optional<Tensor> wy2) {
  SSM_F32(X);
  SSM_IN(y);
  SSM_F32(w);
  TORCH_CHECK(X.dim() == 2 && y.sizes() == X.sizes(), "X and y must be [T, W]");
  const int W = X.size(1);
  TORCH_CHECK(w.numel() == W && (size_t)W * 4 <= 64 * 1024,
              "norm weight must be [W], W <= 16384");
  const int is_f32 = ssm_is_f32(y);
  const void *p2 = nullptr, *pw = nullptr, *pw2 = nullptr;
  if (y2.has_value()) {
    TORCH_CHECK(wy.has_value() && wy2.has_value(), "two branches need weights");
    SSM_IN(y2.value());
    SSM_F32(wy.value());
    SSM_F32(wy2.value());
    TORCH_CHECK(y2->sizes() == X.sizes() &&
                    y2->scalar_type() == y.scalar_type() &&
                    wy->numel() == W && wy2->numel() == W,
                "second branch must match the first");
    p2 = y2->data_ptr();
    pw = wy->data_ptr();
    pw2 = wy2->data_ptr();
  }
  tl_postln_add(X.data_ptr(), y.data_ptr(), p2, w.data_ptr(), pw, pw2,
                X.size(0), W, (float)eps, is_f32, ssm_stream());
}

Tensor polynorm(Tensor z, Tensor coef, double eps) {
  SSM_IN(z);
  SSM_F32(coef);
  TORCH_CHECK(z.dim() == 2 && coef.numel() == 4, "z [T, N], coef [4]");
  auto out = torch::empty_like(z);
  tl_polynorm(z.data_ptr(), coef.data_ptr(), out.data_ptr(), z.size(0),
              (int)z.size(1), (float)eps, ssm_is_f32(z), ssm_stream());
  return out;
}

Tensor gated_group_rms(Tensor y, Tensor gate, int64_t gate_col, Tensor w,
                       int64_t groups, double eps, bool out_f32) {
  SSM_F32(y);
  SSM_IN(gate);
  SSM_F32(w);
  TORCH_CHECK(y.dim() == 2 && gate.dim() == 2 && gate.size(0) == y.size(0),
              "y [T, N], gate [T, L]");
  const int N = y.size(1);
  TORCH_CHECK(groups >= 1 && N % groups == 0 && w.numel() == N &&
                  gate_col >= 0 && gate_col + N <= gate.size(1),
              "groups / gate columns out of range");
  const int is_f32 = ssm_is_f32(gate);
  TORCH_CHECK(is_f32 == (out_f32 ? 1 : 0), "gate / output dtype mismatch");
  auto out = torch::empty({y.size(0), N}, gate.options());
  tl_gated_group_rms(y.data_ptr(), gate.data_ptr(), (int)gate.size(1),
                     (int)gate_col, w.data_ptr(), out.data_ptr(), y.size(0), N,
                     (int)groups, (float)eps, is_f32, ssm_stream());
  return out;
}

void conv_rope_rows(Tensor src, int64_t col, int64_t n_heads, int64_t D,
                    Tensor taps, c10::optional<Tensor> bias, bool act_silu,
                    Tensor hist, int64_t rot_dims,
                    c10::optional<Tensor> freqs, double mult, Tensor tiles,
                    Tensor cu, Tensor slots, Tensor pos0, Tensor table,
                    c10::optional<Tensor> out, c10::optional<Tensor> pool,
                    c10::optional<Tensor> raw_pool, int64_t pool_heads) {
  SSM_IN(src);
  SSM_F32(taps);
  SSM_F32(hist);
  SSM_I32(table);
  check_step(tiles, cu, slots, pos0, hist.size(0));
  const int is_f32 = ssm_is_f32(src);
  const int64_t T = src.size(0), N = n_heads * D;
  TORCH_CHECK(src.dim() == 2 && col >= 0 && col + N <= src.size(1),
              "columns out of range");
  TORCH_CHECK(taps.dim() == 2 && taps.size(0) == N, "taps must be [N, K]");
  const int K = taps.size(1);
  TORCH_CHECK(K >= 1 && K - 1 <= tl_conv_rope_tile(), "too many taps");
  TORCH_CHECK(hist.dim() == 3 && hist.size(1) == K - 1 && hist.size(2) == N,
              "history must be [slots, K-1, N]");
  TORCH_CHECK(pool_heads >= 0 && pool_heads <= n_heads && table.dim() == 2,
              "pool heads out of range");
  const int64_t dense = n_heads - pool_heads;
  if (bias.has_value()) {
    SSM_F32(bias.value());
    TORCH_CHECK(bias->numel() == N, "bias must be [N]");
  }
  if (rot_dims > 0) {
    TORCH_CHECK(freqs.has_value() && freqs->is_cuda() &&
                    freqs->is_contiguous() &&
                    freqs->scalar_type() == torch::kDouble &&
                    freqs->numel() == rot_dims / 2,
                "freqs must be float64 [rot_dims / 2]");
  }
  if (dense > 0) {
    TORCH_CHECK(out.has_value(), "dense heads need an output");
    SSM_F32(out.value());
    TORCH_CHECK(out->numel() == T * dense * D, "out must be [T, dense * D]");
  }
  if (pool_heads > 0) {
    TORCH_CHECK(pool.has_value(), "pool heads need a pool");
    SSM_IN(pool.value());
    TORCH_CHECK(pool->scalar_type() == src.scalar_type() && pool->dim() == 4 &&
                    pool->size(1) == pool_heads && pool->size(2) == 128 &&
                    pool->size(3) == D,
                "pool must be [pages, pool_heads, 128, D] in src's dtype");
    if (raw_pool.has_value()) {
      SSM_IN(raw_pool.value());
      TORCH_CHECK(raw_pool->scalar_type() == src.scalar_type() &&
                      raw_pool->sizes() == pool->sizes(),
                  "raw pool must match the pool");
    }
  }
  const int rc = tl_conv_rope_rows(
      src.data_ptr(), (int)src.size(1), (int)col, (int)n_heads, (int)D,
      taps.data_ptr(), bias.has_value() ? bias->data_ptr() : nullptr,
      act_silu ? 1 : 0, hist.data_ptr(), K, (int)rot_dims,
      rot_dims > 0 ? freqs->data_ptr() : nullptr, (float)mult,
      tiles.data_ptr(), (int)tiles.size(0), cu.data_ptr(), slots.data_ptr(),
      pos0.data_ptr(), table.data_ptr(), (int)table.size(1),
      dense > 0 ? out->data_ptr() : nullptr,
      pool_heads > 0 ? pool->data_ptr() : nullptr,
      (pool_heads > 0 && raw_pool.has_value()) ? raw_pool->data_ptr() : nullptr,
      (int)pool_heads, is_f32, ssm_stream());
  TORCH_CHECK(rc == 0, "conv_rope_rows: shape outside the kernel's range");
}

Tensor ssd_scan(Tensor xbc, int64_t x_off, int64_t b_off, int64_t c_off,
                Tensor dt_src, int64_t dt_col, Tensor dt_bias, Tensor A_log,
                Tensor skip, Tensor S, Tensor cu, Tensor slots, Tensor pos0,
                int64_t H, int64_t P, int64_t N, int64_t G) {
  SSM_F32(xbc);
  SSM_IN(dt_src);
  SSM_F32(dt_bias);
  SSM_F32(A_log);
  SSM_F32(skip);
  SSM_F32(S);
  SSM_I32(cu);
  SSM_I32(slots);
  SSM_I32(pos0);
  const int64_t T = xbc.size(0), L = xbc.size(1);
  TORCH_CHECK(xbc.dim() == 2 && dt_src.dim() == 2 && dt_src.size(0) == T,
              "xbc [T, L], dt_src [T, *]");
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && x_off >= 0 &&
                  x_off + H * P <= L && b_off >= 0 && b_off + G * N <= L &&
                  c_off >= 0 && c_off + G * N <= L && dt_col >= 0 &&
                  dt_col + H <= dt_src.size(1),
              "columns out of range");
  TORCH_CHECK(dt_bias.numel() == H && A_log.numel() == H && skip.numel() == H,
              "per-head constants must be [H]");
  TORCH_CHECK(S.dim() == 4 && S.size(1) == H && S.size(2) == N &&
                  S.size(3) == P,
              "state must be [slots, H, N, P]");
  const int B = slots.numel();
  TORCH_CHECK(cu.numel() == B + 1 && pos0.numel() == B, "ragged metadata");
  auto out = torch::empty({T, H * P}, xbc.options());
  if (T == 0 || B == 0) return out;
  const int rc = tl_ssd_scan(
      xbc.data_ptr(), (int)L, (int)x_off, (int)b_off, (int)c_off,
      dt_src.data_ptr(), (int)dt_src.size(1), (int)dt_col, dt_bias.data_ptr(),
      A_log.data_ptr(), skip.data_ptr(), S.data_ptr(), cu.data_ptr(),
      slots.data_ptr(), pos0.data_ptr(), out.data_ptr(), B, (int)H, (int)G,
      (int)N, (int)P, ssm_is_f32(dt_src), ssm_stream());
  TORCH_CHECK(rc == 0, "ssd_scan: launch refused");
  return out;
}

// per-(chunk, head) operands of the chunk form:
// Cs, Cd, Bs, Bw [chunks*H, C, N], Xd [chunks*H, C, P], L [chunks*H, C],
// tot [chunks*H]
std::vector<Tensor> ssd_chunk_prep(Tensor xbc, int64_t x_off, int64_t b_off,
                                   int64_t c_off, Tensor dt_src,
                                   int64_t dt_col, Tensor dt_bias,
                                   Tensor A_log, Tensor cu_c, int64_t H,
                                   int64_t P, int64_t N, int64_t G,
                                   int64_t C) {
  SSM_F32(xbc);
  SSM_IN(dt_src);
  SSM_F32(dt_bias);
  SSM_F32(A_log);
  SSM_I32(cu_c);
  const int64_t L = xbc.size(1), NC = cu_c.numel() - 1;
  TORCH_CHECK(xbc.dim() == 2 && dt_src.dim() == 2 &&
                  dt_src.size(0) == xbc.size(0) && NC >= 0 && C >= 1,
              "xbc [T, L], dt_src [T, *]");
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && x_off >= 0 &&
                  x_off + H * P <= L && b_off >= 0 && b_off + G * N <= L &&
                  c_off >= 0 && c_off + G * N <= L && dt_col >= 0 &&
                  dt_col + H <= dt_src.size(1) && dt_bias.numel() == H &&
                  A_log.numel() == H,
              "columns out of range");
  auto o = xbc.options();
  std::vector<Tensor> r;
  for (int i = 0; i < 4; ++i) r.push_back(torch::empty({NC * H, C, N}, o));
  r.push_back(torch::empty({NC * H, C, P}, o));
  r.push_back(torch::empty({NC * H, C}, o));
  r.push_back(torch::empty({NC * H}, o));
  tl_ssd_chunk_prep(xbc.data_ptr(), (int)L, (int)x_off, (int)b_off,
                    (int)c_off, dt_src.data_ptr(), (int)dt_src.size(1),
                    (int)dt_col, dt_bias.data_ptr(), A_log.data_ptr(),
                    cu_c.data_ptr(), r[0].data_ptr(), r[1].data_ptr(),
                    r[2].data_ptr(), r[3].data_ptr(), r[4].data_ptr(),
                    r[5].data_ptr(), r[6].data_ptr(), (int)NC, (int)H, (int)G,
                    (int)N, (int)P, (int)C, ssm_is_f32(dt_src), ssm_stream());
  return r;
}

void ssd_decay_mask_(Tensor A, Tensor Lc) {
  SSM_F32(A);
  SSM_F32(Lc);
  TORCH_CHECK(A.dim() == 3 && A.size(1) == A.size(2) && Lc.dim() == 2 &&
                  Lc.size(0) == A.size(0) && Lc.size(1) == A.size(1),
              "A must be [chunks*H, C, C], L [chunks*H, C]");
  tl_ssd_decay_mask(A.data_ptr(), Lc.data_ptr(), (int)A.size(0),
                    (int)A.size(1), ssm_stream());
}

void ssd_chain_(Tensor U, Tensor S, Tensor tot, Tensor chunk_base,
                Tensor n_chunks, Tensor slots, Tensor pos0) {
  SSM_F32(U);
  SSM_F32(S);
  SSM_F32(tot);
  SSM_I32(chunk_base);
  SSM_I32(n_chunks);
  SSM_I32(slots);
  SSM_I32(pos0);
  TORCH_CHECK(S.dim() == 4, "S pool [slots, H, N, P]");
  const int H = S.size(1);
  const int64_t NP = S.size(2) * S.size(3);
  TORCH_CHECK(tot.numel() % H == 0 && U.numel() == tot.numel() * NP,
              "U must be [chunks*H, N, P], tot [chunks*H]");
  const int B = slots.size(0);
  TORCH_CHECK(chunk_base.size(0) == B && n_chunks.size(0) == B &&
                  pos0.size(0) == B,
              "per-sequence chunk metadata");
  tl_ssd_chain(U.data_ptr(), S.data_ptr(), tot.data_ptr(),
               chunk_base.data_ptr(), n_chunks.data_ptr(), slots.data_ptr(),
               pos0.data_ptr(), B, H, (int)NP, ssm_stream());
}

}  // namespace

void register_ssm_ops(pybind11::module& mod) {
  mod.def("layer_norm_rows", &layer_norm_rows,
          "layer norm (weight, no bias) of fp32 rows");
  mod.def("ln_canon", &ln_canon,
          "layer norm + causal per-channel input convolution (slot history)");
  mod.def("postln_add", &postln_add,
          "X += layer_norm(u) * w, u = y or the half sum of two RMS-normed "
          "branches");
  mod.def("polynorm", &polynorm, "cubic in the row-normalised powers");
  mod.def("gated_group_rms", &gated_group_rms,
          "y * silu(gate), RMS norm in equal parts, times w");
  mod.def("conv_rope_rows", &conv_rope_rows,
          "short causal convolution + rotate-half positions, dense or "
          "scattered into page pools");
  mod.def("ssd_chunk_prep", &ssd_chunk_prep,
          "per-chunk operands of the chunk form of the state-space scan");
  mod.def("ssd_decay_mask_", &ssd_decay_mask_,
          "A[i][j] *= exp(L_i - L_j) below and on the diagonal, 0 above");
  mod.def("ssd_chain_", &ssd_chain_,
          "chunk summaries -> state before each chunk; final state to slot");
  mod.def("ssd_scan", &ssd_scan,
          "selective state-space scan over ragged sequences (slot state)");
}
