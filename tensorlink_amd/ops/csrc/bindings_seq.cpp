// Python bindings for the post-norm layered family's kernels: post-norm
// residual, RMS scaling, GELU, soft cap, row preparation (norm + rotation
// + page scatter), the flexible paged attention and the lightning scan.
// Host-side glue and shape checks only; registered into the main module by
// register_seq_ops().

#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

#include "flex_attn.hpp"

extern "C" {
void tl_postnorm_add(void* X, const void* y, const void* w, void* h,
                     int64_t rows, int W, float eps, int one_plus, int is_f32,
                     hipStream_t stream);
void tl_rms_scale(const void* x, const void* w, const void* gate, int ldg,
                  int gate_col, void* out, int64_t rows, int N, float eps,
                  int one_plus, int is_f32, hipStream_t stream);
void tl_add_rms(void* X, const void* y, const void* w, void* h, int64_t rows,
                int W, float eps, float x_scale, int is_f32,
                hipStream_t stream);
void tl_gelu_gate(const void* p, void* out, int64_t rows, int N,
                  int tanh_form, int is_f32, hipStream_t stream);
void tl_gelu(const void* x, void* out, int64_t n, int N, int tanh_form,
             const void* table, int ldt, int table_col, const void* tokens,
             int is_f32, hipStream_t stream);
void tl_soft_cap(void* z, int64_t n, float cap, hipStream_t stream);
void tl_norm_rope_rows(const void* src, int ld, int col, int n_heads,
                       int head_dim, const void* norm_w, int norm_cols,
                       float eps, int rot_off, int rot_dims,
                       const void* freqs, const void* tok_seq,
                       const void* tok_pos, const void* table, int P, int T,
                       void* out, void* pool, int is_f32, int head_norm,
                       int interleaved, float rot_mult, const void* mix_src,
                       int mix_ld, int mix_col, const void* mix_lam,
                       hipStream_t stream);
int tl_flex_attn_heads_per_block(int H, int G, int DK, int V, int has_talk);
int tl_flex_attn_rows(const void* q, const void* kpool, const void* vpool,
                      int vld, const void* tok_seq, const void* tok_pos,
                      const void* table, int P, const void* talk, void* out,
                      int out_f32, void* part, int ns, int T, int H, int G,
                      int DK, int V, float scale, int window, int sink,
                      int pool_f32, int hb_max, float softcap,
                      const void* sinks, TlFlexExtra ex, hipStream_t stream);
int tl_flex_attn_tiles_ok(int H, int G, int KG, int DK, int V);
void tl_stage_queries(const void* q, const void* talk, void* out, int T,
                      int H, int G, int DK, hipStream_t stream);
int tl_flex_attn_tiles(const void* q, const void* kpool, const void* vpool,
                       int vld, const void* tiles, int n_tiles,
                       const void* table, int P, void* out, int out_f32,
                       int H, int G, int KG, int DK, int V, float scale,
                       int window, int sink, float softcap, const void* sinks,
                       TlFlexExtra ex, hipStream_t stream);
int tl_lightning_scan(const void* proj, int ld, int q_off, int k_off,
                      int v_off, const void* decay, void* S, const void* cu,
                      const void* slots, const void* pos0, void* out, int B,
                      int H, int D, int V, int is_f32, hipStream_t stream);
void tl_lightning_chunk_prep(const void* proj, int ld, int q_off, int k_off,
                             int v_off, const void* decay, const void* cu_c,
                             void* Qs, void* Qd, void* Ks, void* Kw, void* Vs,
                             int NC, int H, int D, int V, int C, int is_f32,
                             hipStream_t stream);
void tl_lightning_decay_mask(void* A, const void* decay, int NCH, int H,
                             int C, hipStream_t stream);
void tl_lightning_chain(void* U, void* S, const void* decay, const void* cu_c,
                        const void* chunk_base, const void* n_chunks,
                        const void* slots, const void* pos0, int B, int H,
                        int DV, hipStream_t stream);
}

namespace {

using torch::Tensor;

hipStream_t seq_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define SEQ_IN(t)                                                    \
  TORCH_CHECK((t).is_cuda(), #t " must be on GPU");                  \
  TORCH_CHECK((t).is_contiguous(), #t " must be contiguous")
#define SEQ_F32(t) \
  SEQ_IN(t);       \
  TORCH_CHECK((t).scalar_type() == torch::kFloat, #t " must be fp32")
#define SEQ_I32(t) \
  SEQ_IN(t);       \
  TORCH_CHECK((t).scalar_type() == torch::kInt, #t " must be int32")

int act_is_f32(const Tensor& t) {
  TORCH_CHECK(t.scalar_type() == torch::kFloat ||
                  t.scalar_type() == torch::kBFloat16,
              "activations must be fp32 or bf16");
  return t.scalar_type() == torch::kFloat ? 1 : 0;
}

// X += y / rms(y) * (w | 1 + w); returns X in the serving dtype
Tensor postnorm_add(Tensor X, Tensor y, Tensor w, double eps, bool one_plus,
                    bool out_f32) {
  SEQ_F32(X);
  SEQ_IN(y);
  SEQ_F32(w);
  TORCH_CHECK(X.dim() == 2 && y.dim() == 2 && y.sizes() == X.sizes(),
              "X and y must be [T, W]");
  const int W = X.size(1);
  TORCH_CHECK(w.numel() == W, "norm weight must be [W]");
  const int is_f32 = act_is_f32(y);
  TORCH_CHECK(is_f32 == (out_f32 ? 1 : 0), "y / output dtype mismatch");
  Tensor h;
  if (!out_f32) h = torch::empty_like(y);
  tl_postnorm_add(X.data_ptr(), y.data_ptr(), w.data_ptr(),
                  out_f32 ? nullptr : h.data_ptr(), X.size(0), W, (float)eps,
                  one_plus ? 1 : 0, is_f32, seq_stream());
  return out_f32 ? X : h;
}

Tensor rms_scale(Tensor x, Tensor w, double eps, bool one_plus,
                 c10::optional<Tensor> gate, int64_t gate_col, bool out_f32) {
  SEQ_F32(x);
  SEQ_F32(w);
  TORCH_CHECK(x.dim() == 2, "x must be [T, N]");
  const int N = x.size(1);
  TORCH_CHECK(w.numel() == N, "norm weight must be [N]");
  int ldg = 0;
  if (gate.has_value()) {
    SEQ_IN(gate.value());
    TORCH_CHECK(act_is_f32(gate.value()) == (out_f32 ? 1 : 0),
                "gate / output dtype mismatch");
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == x.size(0) &&
                    gate_col >= 0 && gate_col + N <= gate->size(1),
                "gate columns out of range");
    ldg = gate->size(1);
  }
  auto out = torch::empty(
      {x.size(0), N},
      x.options().dtype(out_f32 ? torch::kFloat : torch::kBFloat16));
  tl_rms_scale(x.data_ptr(), w.data_ptr(),
               gate.has_value() ? gate->data_ptr() : nullptr, ldg,
               (int)gate_col, out.data_ptr(), x.size(0), N, (float)eps,
               one_plus ? 1 : 0, out_f32 ? 1 : 0, seq_stream());
  return out;
}

// X (*= x_scale) += y; returns rms(X) * w in the serving dtype, or,
// without a weight, X itself after the add
Tensor add_rms(Tensor X, c10::optional<Tensor> y, c10::optional<Tensor> w,
               double eps, double x_scale, bool out_f32) {
  SEQ_F32(X);
  TORCH_CHECK(X.dim() == 2, "X must be [T, W]");
  if (w.has_value()) {
    SEQ_F32(w.value());
    TORCH_CHECK(w->numel() == X.size(1), "the norm weight must be [W]");
  }
  if (y.has_value()) {
    SEQ_IN(y.value());
    TORCH_CHECK(y->sizes() == X.sizes(), "y must be [T, W]");
    TORCH_CHECK(act_is_f32(y.value()) == (out_f32 ? 1 : 0),
                "y / output dtype mismatch");
  }
  Tensor h = X;
  if (w.has_value())
    h = torch::empty(X.sizes(), X.options().dtype(out_f32 ? torch::kFloat
                                                          : torch::kBFloat16));
  tl_add_rms(X.data_ptr(), y.has_value() ? y->data_ptr() : nullptr,
             w.has_value() ? w->data_ptr() : nullptr,
             w.has_value() ? h.data_ptr() : nullptr, X.size(0), (int)X.size(1),
             (float)eps, (float)x_scale, out_f32 ? 1 : 0, seq_stream());
  return h;
}

// gelu(p[:, :N]) * p[:, N:] for p [T, 2N]
Tensor gelu_gate(Tensor p, bool tanh_form) {
  SEQ_IN(p);
  TORCH_CHECK(p.dim() == 2 && p.size(1) % 2 == 0, "p must be [T, 2N]");
  const int64_t N = p.size(1) / 2;
  auto out = torch::empty({p.size(0), N}, p.options());
  tl_gelu_gate(p.data_ptr(), out.data_ptr(), p.size(0), (int)N,
               tanh_form ? 1 : 0, act_is_f32(p), seq_stream());
  return out;
}

Tensor gelu_mul(Tensor x, bool tanh_form, c10::optional<Tensor> table,
                c10::optional<Tensor> tokens, int64_t table_col) {
  SEQ_IN(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, N]");
  const int N = x.size(1);
  auto out = torch::empty_like(x);
  int ldt = 0;
  if (table.has_value()) {
    SEQ_IN(table.value());
    TORCH_CHECK(tokens.has_value(), "a table needs token ids");
    SEQ_I32(tokens.value());
    TORCH_CHECK(table->scalar_type() == x.scalar_type(),
                "table dtype must match activations");
    TORCH_CHECK(table->dim() == 2 && table_col >= 0 &&
                    table_col + N <= table->size(1) &&
                    tokens->numel() == x.size(0),
                "table columns / token ids out of range");
    ldt = table->size(1);
  }
  tl_gelu(x.data_ptr(), out.data_ptr(), x.numel(), N, tanh_form ? 1 : 0,
          table.has_value() ? table->data_ptr() : nullptr, ldt,
          (int)table_col, tokens.has_value() ? tokens->data_ptr() : nullptr,
          act_is_f32(x), seq_stream());
  return out;
}

void soft_cap_(Tensor z, double cap) {
  SEQ_F32(z);
  tl_soft_cap(z.data_ptr(), z.numel(), (float)cap, seq_stream());
}

void norm_rope_rows(Tensor src, int64_t col, int64_t n_heads,
                    int64_t head_dim, c10::optional<Tensor> norm_w,
                    int64_t norm_cols, double eps, int64_t rot_off,
                    int64_t rot_dims, c10::optional<Tensor> freqs,
                    Tensor tok_seq, Tensor tok_pos, Tensor table,
                    c10::optional<Tensor> out, c10::optional<Tensor> pool,
                    bool head_norm, bool interleaved, double rot_mult,
                    c10::optional<Tensor> mix_src, int64_t mix_col,
                    c10::optional<Tensor> mix_lam) {
  SEQ_IN(src);
  SEQ_I32(tok_seq);
  SEQ_I32(tok_pos);
  SEQ_I32(table);
  TORCH_CHECK(src.dim() == 2 && table.dim() == 2, "src [T, L], table [B, P]");
  const int64_t T = src.size(0), ld = src.size(1);
  const int64_t N = n_heads * head_dim;
  TORCH_CHECK(col >= 0 && col + N <= ld, "columns out of range");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T,
              "ragged metadata");
  if (norm_w.has_value() && head_norm) {
    SEQ_F32(norm_w.value());
    TORCH_CHECK(norm_w->numel() == head_dim && n_heads <= 512,
                "a per-head norm has one weight [head_dim] (<= 512 heads)");
  } else if (norm_w.has_value()) {
    SEQ_F32(norm_w.value());
    TORCH_CHECK(norm_cols > 0 && norm_cols <= N &&
                    norm_w->numel() == norm_cols,
                "norm weight must cover the normed columns");
  }
  int mix_ld = 0;
  if (mix_src.has_value()) {
    SEQ_IN(mix_src.value());
    TORCH_CHECK(mix_lam.has_value(), "blending needs its weight");
    SEQ_F32(mix_lam.value());
    TORCH_CHECK(mix_src->scalar_type() == src.scalar_type() &&
                    mix_src->dim() == 2 && mix_src->size(0) == T &&
                    mix_col >= 0 && mix_col + N <= mix_src->size(1) &&
                    mix_lam->numel() == 1,
                "blend source must be [T, >= mix_col + N] of src's dtype");
    mix_ld = (int)mix_src->size(1);
  }
  if (rot_dims > 0) {
    TORCH_CHECK(freqs.has_value(), "rotation needs frequencies");
    SEQ_IN(freqs.value());
    TORCH_CHECK(freqs->scalar_type() == torch::kDouble &&
                    freqs->numel() == rot_dims / 2 && rot_dims % 2 == 0 &&
                    rot_off >= 0 && rot_off + rot_dims <= head_dim,
                "frequencies must be float64 [rot_dims / 2]");
    // a rotated pair must be normed alike
    TORCH_CHECK(!norm_w.has_value() || head_norm || norm_cols == N ||
                    (n_heads == 1 && (norm_cols <= rot_off)),
                "the norm range may not cut a rotated pair");
  }
  TORCH_CHECK(out.has_value() != pool.has_value(),
              "either a dense output or a pool");
  if (out.has_value()) {
    SEQ_F32(out.value());
    TORCH_CHECK(out->numel() == T * N, "out must be [T, N]");
  } else {
    SEQ_IN(pool.value());
    TORCH_CHECK(pool->scalar_type() == src.scalar_type(),
                "pool dtype must match activations");
    TORCH_CHECK(pool->dim() == 4 && pool->size(1) == n_heads &&
                    pool->size(2) == 128 && pool->size(3) == head_dim,
                "pool must be [pages, heads, 128, head_dim]");
  }
  tl_norm_rope_rows(
      src.data_ptr(), (int)ld, (int)col, (int)n_heads, (int)head_dim,
      norm_w.has_value() ? norm_w->data_ptr() : nullptr, (int)norm_cols,
      (float)eps, (int)rot_off, (int)rot_dims,
      rot_dims > 0 ? freqs->data_ptr() : nullptr, tok_seq.data_ptr(),
      tok_pos.data_ptr(), table.data_ptr(), (int)table.size(1), (int)T,
      out.has_value() ? out->data_ptr() : nullptr,
      pool.has_value() ? pool->data_ptr() : nullptr, act_is_f32(src),
      head_norm ? 1 : 0, interleaved ? 1 : 0, (float)rot_mult,
      mix_src.has_value() ? mix_src->data_ptr() : nullptr, mix_ld,
      (int)mix_col, mix_lam.has_value() ? mix_lam->data_ptr() : nullptr,
      seq_stream());
}

// checked options of the flexible attention beyond window / sink / cap
TlFlexExtra flex_extra(int64_t T, int64_t H, int64_t V, int64_t window,
                       int64_t chunk, int64_t keep,
                       const c10::optional<Tensor>& bias,
                       const c10::optional<Tensor>& gate, int64_t gate_col,
                       bool gate_heads) {
  TlFlexExtra ex{};
  TORCH_CHECK(chunk >= 0 && keep >= 0 && !(chunk > 0 && window > 0),
              "a chunked mask has no window");
  ex.chunk = (int)chunk;
  ex.keep = (int)keep;
  if (bias.has_value()) {
    SEQ_F32(bias.value());
    TORCH_CHECK(bias->dim() == 2 && bias->size(0) == H && bias->size(1) >= 1,
                "distance bias must be [H, n]");
    ex.bias = (const float*)bias->data_ptr();
    ex.nb = (int)bias->size(1);
  }
  if (gate.has_value()) {
    SEQ_IN(gate.value());
    const int64_t n = gate_heads ? H : H * V;
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T && gate_col >= 0 &&
                    gate_col + n <= gate->size(1),
                "gate columns out of range");
    ex.gate = gate->data_ptr();
    ex.gate_ld = (int)gate->size(1);
    ex.gate_col = (int)gate_col;
    ex.gate_heads = gate_heads ? 1 : 0;
    ex.gate_f32 = act_is_f32(gate.value());
  }
  return ex;
}

Tensor flex_attn_rows(Tensor q, Tensor kpool, c10::optional<Tensor> vpool,
                      Tensor tok_seq, Tensor tok_pos, Tensor table,
                      c10::optional<Tensor> talk, int64_t H, double scale,
                      int64_t window, bool sink, int64_t V, bool out_f32,
                      int64_t n_split, int64_t hb_max, double softcap,
                      c10::optional<Tensor> sinks, int64_t chunk,
                      int64_t keep, c10::optional<Tensor> bias,
                      c10::optional<Tensor> gate, int64_t gate_col,
                      bool gate_heads) {
  if (sinks.has_value()) {
    SEQ_F32(sinks.value());
    TORCH_CHECK(sinks->numel() == H && sink, "sink logits must be [H]");
  }
  SEQ_F32(q);
  SEQ_IN(kpool);
  SEQ_I32(tok_seq);
  SEQ_I32(tok_pos);
  SEQ_I32(table);
  TORCH_CHECK(kpool.dim() == 4 && kpool.size(2) == 128,
              "key pool must be [pages, G, 128, DK]");
  const int G = kpool.size(1), DK = kpool.size(3);
  const int64_t T = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) == H * DK, "q must be [T, H*DK]");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T && table.dim() == 2,
              "ragged metadata");
  const int pool_f32 = act_is_f32(kpool);
  const void* vp = kpool.data_ptr();
  int vld = DK;
  if (vpool.has_value()) {
    SEQ_IN(vpool.value());
    TORCH_CHECK(vpool->scalar_type() == kpool.scalar_type() &&
                    vpool->dim() == 4 && vpool->size(0) == kpool.size(0) &&
                    vpool->size(1) == G && vpool->size(2) == 128 &&
                    vpool->size(3) == V,
                "value pool must be [pages, G, 128, V]");
    vp = vpool->data_ptr();
    vld = V;
  } else {
    TORCH_CHECK(V >= 1 && V <= DK, "values are a prefix of the key row");
  }
  if (talk.has_value()) {
    SEQ_F32(talk.value());
    TORCH_CHECK(talk->numel() == H * H, "talk must be [H, H]");
  }
  TORCH_CHECK(window >= 0 && n_split >= 1 && n_split <= 64,
              "window / n_split out of range");
  const TlFlexExtra ex =
      flex_extra(T, H, V, window, chunk, keep, bias, gate, gate_col, gate_heads);
  TORCH_CHECK(tl_flex_attn_heads_per_block((int)H, G, DK, (int)V,
                                           talk.has_value() ? 1 : 0) > 0,
              "flex_attn_rows: shape outside the kernel's range (value size "
              "<= 512, heads divisible by key heads, staged queries within "
              "64 KiB of LDS)");
  auto out = torch::empty(
      {T, H * V}, q.options().dtype(out_f32 ? torch::kFloat
                                            : torch::kBFloat16));
  if (T == 0) return out;
  Tensor part;
  if (n_split > 1)
    part = torch::empty({T * H * n_split * (2 + V)}, q.options());
  const int rc = tl_flex_attn_rows(
      q.data_ptr(), kpool.data_ptr(), vp, vld, tok_seq.data_ptr(),
      tok_pos.data_ptr(), table.data_ptr(), (int)table.size(1),
      talk.has_value() ? talk->data_ptr() : nullptr, out.data_ptr(),
      out_f32 ? 1 : 0, n_split > 1 ? part.data_ptr() : nullptr, (int)n_split,
      (int)T, (int)H, G, DK, (int)V, (float)scale, (int)window, sink ? 1 : 0,
      pool_f32, (int)std::max<int64_t>(1, hb_max), (float)softcap,
      sinks.has_value() ? sinks->data_ptr() : nullptr, ex, seq_stream());
  TORCH_CHECK(rc == 0, "flex_attn_rows: launch refused");
  return out;
}

bool flex_attn_tiles_ok(int64_t H, int64_t G, bool has_talk, int64_t DK,
                        int64_t V) {
  return tl_flex_attn_tiles_ok((int)H, (int)G, has_talk ? (int)G : 1,
                               (int)DK, (int)V) != 0;
}

// MFMA path for prompt portions (bf16 pools): `tiles` [n, 4] int32 rows of
// (sequence, first flat token, token count <= 64, first position).
Tensor flex_attn_tiles(Tensor q, Tensor kpool, c10::optional<Tensor> vpool,
                       Tensor tiles, Tensor table,
                       c10::optional<Tensor> talk, int64_t H, double scale,
                       int64_t window, bool sink, int64_t V, bool out_f32,
                       double softcap, c10::optional<Tensor> sinks,
                       int64_t chunk, int64_t keep,
                       c10::optional<Tensor> bias, c10::optional<Tensor> gate,
                       int64_t gate_col, bool gate_heads) {
  if (sinks.has_value()) {
    SEQ_F32(sinks.value());
    TORCH_CHECK(sinks->numel() == H && sink, "sink logits must be [H]");
  }
  SEQ_F32(q);
  SEQ_IN(kpool);
  SEQ_I32(tiles);
  SEQ_I32(table);
  TORCH_CHECK(kpool.scalar_type() == torch::kBFloat16 && kpool.dim() == 4 &&
                  kpool.size(2) == 128,
              "key pool must be bf16 [pages, G, 128, DK]");
  const int G = kpool.size(1), DK = kpool.size(3);
  const int64_t T = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) == H * DK, "q must be [T, H*DK]");
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 4 && table.dim() == 2,
              "tiles must be [n, 4]");
  const void* vp = kpool.data_ptr();
  int vld = DK;
  if (vpool.has_value()) {
    SEQ_IN(vpool.value());
    TORCH_CHECK(vpool->scalar_type() == torch::kBFloat16 &&
                    vpool->dim() == 4 && vpool->size(0) == kpool.size(0) &&
                    vpool->size(1) == G && vpool->size(2) == 128 &&
                    vpool->size(3) == V,
                "value pool must be bf16 [pages, G, 128, V]");
    vp = vpool->data_ptr();
    vld = V;
  } else {
    TORCH_CHECK(G == 1 && V >= 1 && V <= DK,
                "values are a prefix of the single key head's row");
  }
  if (talk.has_value()) {
    SEQ_F32(talk.value());
    TORCH_CHECK(talk->numel() == H * H, "talk must be [H, H]");
  }
  const int KG = talk.has_value() ? G : 1;
  TORCH_CHECK(tl_flex_attn_tiles_ok((int)H, G, KG, DK, (int)V),
              "flex_attn_tiles: shape outside the kernel's range");
  const TlFlexExtra ex =
      flex_extra(T, H, V, window, chunk, keep, bias, gate, gate_col, gate_heads);
  auto qs = torch::empty({T, H * KG * DK},
                         q.options().dtype(torch::kBFloat16));
  auto out = torch::empty(
      {T, H * V}, q.options().dtype(out_f32 ? torch::kFloat
                                            : torch::kBFloat16));
  if (T == 0 || tiles.size(0) == 0) return out;
  tl_stage_queries(q.data_ptr(),
                   talk.has_value() ? talk->data_ptr() : nullptr,
                   qs.data_ptr(), (int)T, (int)H, G, DK, seq_stream());
  const int rc = tl_flex_attn_tiles(
      qs.data_ptr(), kpool.data_ptr(), vp, vld, tiles.data_ptr(),
      (int)tiles.size(0), table.data_ptr(), (int)table.size(1),
      out.data_ptr(), out_f32 ? 1 : 0, (int)H, G, KG, DK, (int)V,
      (float)scale, (int)window, sink ? 1 : 0, (float)softcap,
      sinks.has_value() ? sinks->data_ptr() : nullptr, ex, seq_stream());
  TORCH_CHECK(rc == 0, "flex_attn_tiles: launch refused");
  return out;
}

Tensor lightning_scan(Tensor proj, int64_t q_off, int64_t k_off,
                      int64_t v_off, Tensor decay, Tensor S, Tensor cu,
                      Tensor slots, Tensor pos0, int64_t H, int64_t D,
                      int64_t V) {
  SEQ_IN(proj);
  SEQ_F32(decay);
  SEQ_F32(S);
  SEQ_I32(cu);
  SEQ_I32(slots);
  SEQ_I32(pos0);
  TORCH_CHECK(proj.dim() == 2, "proj must be [T, L]");
  const int64_t T = proj.size(0), ld = proj.size(1);
  const int B = slots.size(0);
  TORCH_CHECK(cu.size(0) == B + 1 && pos0.size(0) == B, "ragged metadata");
  TORCH_CHECK(q_off + H * D <= ld && k_off + H * D <= ld &&
                  v_off + H * V <= ld,
              "projection columns out of range");
  TORCH_CHECK(decay.numel() == H, "one decay per head");
  TORCH_CHECK(S.dim() == 4 && S.size(1) == H && S.size(2) == D &&
                  S.size(3) == V,
              "S pool must be [slots, H, D, V]");
  auto out = torch::empty({T, H * V}, proj.options().dtype(torch::kFloat));
  if (T == 0 || B == 0) return out;
  const int rc = tl_lightning_scan(
      proj.data_ptr(), (int)ld, (int)q_off, (int)k_off, (int)v_off,
      decay.data_ptr(), S.data_ptr(), cu.data_ptr(), slots.data_ptr(),
      pos0.data_ptr(), out.data_ptr(), B, (int)H, (int)D, (int)V,
      act_is_f32(proj), seq_stream());
  TORCH_CHECK(rc == 0, "lightning_scan: head sizes outside the kernel's "
                       "range");
  return out;
}

// silu(q), a^(i+1) silu(q), silu(k), a^(n-1-j) silu(k), silu(v) per
// (chunk, head), zero-padded to C rows: five fp32 tensors [NC*H, C, D|V]
std::vector<Tensor> lightning_chunk_prep(Tensor proj, int64_t q_off,
                                         int64_t k_off, int64_t v_off,
                                         Tensor decay, Tensor cu_c,
                                         int64_t H, int64_t D, int64_t V,
                                         int64_t C) {
  SEQ_IN(proj);
  SEQ_F32(decay);
  SEQ_I32(cu_c);
  TORCH_CHECK(proj.dim() == 2 && cu_c.numel() >= 1, "proj [T, L], cu_c");
  const int64_t ld = proj.size(1), NC = cu_c.numel() - 1;
  TORCH_CHECK(q_off + H * D <= ld && k_off + H * D <= ld &&
                  v_off + H * V <= ld && decay.numel() == H && C >= 1,
              "projection columns out of range");
  auto o = proj.options().dtype(torch::kFloat);
  std::vector<Tensor> r;
  for (int i = 0; i < 4; ++i) r.push_back(torch::empty({NC * H, C, D}, o));
  r.push_back(torch::empty({NC * H, C, V}, o));
  tl_lightning_chunk_prep(proj.data_ptr(), (int)ld, (int)q_off, (int)k_off,
                          (int)v_off, decay.data_ptr(), cu_c.data_ptr(),
                          r[0].data_ptr(), r[1].data_ptr(), r[2].data_ptr(),
                          r[3].data_ptr(), r[4].data_ptr(), (int)NC, (int)H,
                          (int)D, (int)V, (int)C, act_is_f32(proj),
                          seq_stream());
  return r;
}

void lightning_decay_mask_(Tensor A, Tensor decay) {
  SEQ_F32(A);
  SEQ_F32(decay);
  const int H = decay.numel();
  TORCH_CHECK(A.dim() == 3 && A.size(1) == A.size(2) && A.size(0) % H == 0,
              "A must be [chunks*H, C, C]");
  tl_lightning_decay_mask(A.data_ptr(), decay.data_ptr(), (int)A.size(0), H,
                          (int)A.size(1), seq_stream());
}

void lightning_chain_(Tensor U, Tensor S, Tensor decay, Tensor cu_c,
                      Tensor chunk_base, Tensor n_chunks, Tensor slots,
                      Tensor pos0) {
  SEQ_F32(U);
  SEQ_F32(S);
  SEQ_F32(decay);
  SEQ_I32(cu_c);
  SEQ_I32(chunk_base);
  SEQ_I32(n_chunks);
  SEQ_I32(slots);
  SEQ_I32(pos0);
  const int H = decay.numel();
  TORCH_CHECK(S.dim() == 4 && S.size(1) == H, "S pool [slots, H, D, V]");
  const int64_t DV = S.size(2) * S.size(3);
  const int64_t NC = cu_c.numel() - 1;
  TORCH_CHECK(U.numel() == NC * H * DV, "U must be [chunks*H, D, V]");
  const int B = slots.size(0);
  TORCH_CHECK(chunk_base.size(0) == B && n_chunks.size(0) == B &&
                  pos0.size(0) == B,
              "per-sequence chunk metadata");
  tl_lightning_chain(U.data_ptr(), S.data_ptr(), decay.data_ptr(),
                     cu_c.data_ptr(), chunk_base.data_ptr(),
                     n_chunks.data_ptr(), slots.data_ptr(), pos0.data_ptr(),
                     B, H, (int)DV, seq_stream());
}

}  // namespace

void register_seq_ops(pybind11::module& mod) {
  mod.def("lightning_chunk_prep", &lightning_chunk_prep,
          "per-chunk activations of the chunk form of lightning attention");
  mod.def("lightning_decay_mask_", &lightning_decay_mask_,
          "A[i][j] *= a^(i-j) below and on the diagonal, 0 above");
  mod.def("lightning_chain_", &lightning_chain_,
          "chunk summaries -> state before each chunk; final state to slot");
  mod.def("postnorm_add", &postnorm_add,
          "X += y / rms(y) * g on the fp32 residual; returns the cast copy");
  mod.def("rms_scale", &rms_scale, "x / rms(x) * g [* sigmoid(gate)]");
  mod.def("add_rms", &add_rms,
          "X += y on the fp32 residual; returns rms(X) * w (pre-norm)");
  mod.def("gelu_gate", &gelu_gate, "gelu(gate) * up on a fused projection");
  mod.def("gelu_mul", &gelu_mul,
          "GELU (erf or tanh form) times an optional gathered table slice");
  mod.def("soft_cap_", &soft_cap_, "cap * tanh(z / cap) in place");
  mod.def("norm_rope_rows", &norm_rope_rows,
          "RMS norm (whole range or per head) + rotary positions (halves or "
          "interleaved) + optional blend on projection rows, dense or "
          "scattered into a page pool");
  mod.def("flex_attn_rows", &flex_attn_rows,
          "paged softmax attention: window / chunk / kept prefix, sink, "
          "distance bias, score mixing, latent rows, output gate");
  mod.def("flex_attn_tiles_ok", &flex_attn_tiles_ok,
          "whether the MFMA tile kernel serves a shape");
  mod.def("flex_attn_tiles", &flex_attn_tiles,
          "paged softmax attention on MFMA, 64-query tiles (bf16 pools)");
  mod.def("lightning_scan", &lightning_scan,
          "decayed linear attention over ragged sequences (slot state)");
}
