// Python bindings for the sequence-mixer kernels: hyper-connection +
// Dynamic-Tanh, matrix-memory recurrence, differential attention over the
// paged pool. Host-side glue and shape checks only; registered into the
// main module by register_mix_ops().

#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
void tl_hyper_dyt(void* X, const void* y, const void* mix, const void* outw,
                  const void* inw, const void* alpha, const void* w,
                  const void* b, void* h, void* usum, int ns, int64_t TW,
                  int W, int is_f32, hipStream_t stream);
void tl_relu_sq(const void* x, void* out, int64_t n, int is_f32,
                hipStream_t stream);
int tl_mlstm_seq(const void* proj, int ld, int q_off, int k_off, int v_off,
                 int g_off, const void* gates, const void* norm_w, void* S,
                 void* n, void* m, const void* cu, const void* slots,
                 const void* pos0, void* out, int B, int H, int D, int V,
                 float cap, float qscale, float eps, void* F, int summary,
                 int is_f32, hipStream_t stream);
int tl_mlstm_chain(void* S_tmp, void* n_tmp, void* m_tmp, const void* F_tmp,
                   void* S, void* n, void* m, const void* chunk_base,
                   const void* n_chunks, const void* slots, const void* pos0,
                   int B, int max_chunks, int H, int D, int V,
                   hipStream_t stream);
void tl_kv_append(const void* proj, int ld, int k_off, int v_off, void* kpool,
                  void* vpool, const void* tok_seq, const void* tok_pos,
                  const void* table, int P, int T, int G, int DK, int V,
                  int is_f32, hipStream_t stream);
int tl_diff_attn_rows(const void* q, int ldq, int q_off, const void* kpool,
                      const void* vpool, const void* tok_seq,
                      const void* tok_pos, const void* table, int P,
                      const void* lam, void* out, void* part, int ns, int T,
                      int H, int G, int D, int V, float scale, float diff,
                      float eps, int is_f32, hipStream_t stream);
int tl_diff_attn_tiles(const void* q, int ldq, int q_off, const void* kpool,
                       const void* vpool, const void* tiles, int n_tiles,
                       const void* table, int P, const void* lam, void* out,
                       int H, int G, int D, int V, float scale, float diff,
                       float eps, hipStream_t stream);
}

namespace {

using torch::Tensor;

hipStream_t mix_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define MIX_IN(t)                                                    \
  TORCH_CHECK((t).is_cuda(), #t " must be on GPU");                  \
  TORCH_CHECK((t).is_contiguous(), #t " must be contiguous")
#define MIX_F32(t) \
  MIX_IN(t);       \
  TORCH_CHECK((t).scalar_type() == torch::kFloat, #t " must be fp32")
#define MIX_I32(t) \
  MIX_IN(t);       \
  TORCH_CHECK((t).scalar_type() == torch::kInt, #t " must be int32")

int io_is_f32(const Tensor& t) {
  TORCH_CHECK(t.scalar_type() == torch::kFloat ||
                  t.scalar_type() == torch::kBFloat16,
              "activations must be fp32 or bf16");
  return t.scalar_type() == torch::kFloat ? 1 : 0;
}

const void* opt_ptr(const c10::optional<Tensor>& t) {
  return t.has_value() ? t->data_ptr() : nullptr;
}

std::vector<Tensor> hyper_dyt(Tensor X, c10::optional<Tensor> y,
                              c10::optional<Tensor> mix,
                              c10::optional<Tensor> outw,
                              c10::optional<Tensor> inw,
                              c10::optional<Tensor> alpha,
                              c10::optional<Tensor> w,
                              c10::optional<Tensor> b, bool out_f32,
                              bool want_sum) {
  MIX_F32(X);
  TORCH_CHECK(X.dim() == 3, "streams must be [ns, T, W]");
  const int ns = X.size(0);
  const int64_t TW = X.size(1) * X.size(2);
  const int W = X.size(2);
  TORCH_CHECK(ns >= 1 && ns <= 8, "1..8 residual streams supported");
  int is_f32 = out_f32 ? 1 : 0;
  if (y.has_value()) {
    MIX_IN(y.value());
    is_f32 = io_is_f32(y.value());
    TORCH_CHECK(is_f32 == (out_f32 ? 1 : 0), "y / output dtype mismatch");
    TORCH_CHECK(y->numel() == TW, "y must be [T, W]");
    TORCH_CHECK(mix.has_value() && outw.has_value(), "update needs mix/out");
    MIX_F32(mix.value());
    MIX_F32(outw.value());
    TORCH_CHECK(mix->numel() == ns * ns && outw->numel() == ns,
                "mix [ns, ns], out [ns]");
  }
  if (inw.has_value()) {
    MIX_F32(inw.value());
    TORCH_CHECK(inw->numel() == ns, "in [ns]");
  }
  Tensor h, usum;
  if (w.has_value()) {
    TORCH_CHECK(alpha.has_value() && b.has_value(), "norm needs alpha, b");
    MIX_F32(w.value());
    MIX_F32(b.value());
    MIX_F32(alpha.value());
    TORCH_CHECK(w->numel() == W && b->numel() == W && alpha->numel() == 1,
                "norm weight/bias [W], alpha scalar");
    h = torch::empty({X.size(1), X.size(2)},
                     X.options().dtype(out_f32 ? torch::kFloat
                                               : torch::kBFloat16));
  }
  if (want_sum) usum = torch::empty({X.size(1), X.size(2)}, X.options());
  if (TW > 0)
    tl_hyper_dyt(X.data_ptr(), opt_ptr(y), opt_ptr(mix), opt_ptr(outw),
                 opt_ptr(inw), opt_ptr(alpha), opt_ptr(w), opt_ptr(b),
                 h.defined() ? h.data_ptr() : nullptr,
                 usum.defined() ? usum.data_ptr() : nullptr, ns, TW, W,
                 is_f32, mix_stream());
  return {h.defined() ? h : torch::empty({0}, X.options()),
          usum.defined() ? usum : torch::empty({0}, X.options())};
}

Tensor relu_sq(Tensor x) {
  MIX_IN(x);
  auto out = torch::empty_like(x);
  if (x.numel() > 0)
    tl_relu_sq(x.data_ptr(), out.data_ptr(), x.numel(), io_is_f32(x),
               mix_stream());
  return out;
}

Tensor mlstm_seq(Tensor proj, int64_t q_off, int64_t k_off, int64_t v_off,
                 int64_t g_off, Tensor gates, Tensor norm_w, Tensor S,
                 Tensor n, Tensor m, Tensor cu, Tensor slots, Tensor pos0,
                 int64_t H, int64_t D, int64_t V, double cap, double qscale,
                 double eps, c10::optional<Tensor> F_sum) {
  // F_sum given = summary mode: every ragged entry is run from the empty
  // state, no output is produced, its slot receives the entry's summary
  // and F_sum [slots, H] the sum of its log forget gates
  MIX_IN(proj);
  MIX_F32(gates);
  MIX_F32(norm_w);
  MIX_F32(S);
  MIX_F32(n);
  MIX_F32(m);
  MIX_I32(cu);
  MIX_I32(slots);
  MIX_I32(pos0);
  TORCH_CHECK(proj.dim() == 2, "proj must be [T, L]");
  const int64_t T = proj.size(0), ld = proj.size(1);
  const int B = slots.size(0);
  TORCH_CHECK(cu.size(0) == B + 1 && pos0.size(0) == B, "ragged metadata");
  TORCH_CHECK(q_off + H * D <= ld && k_off + H * D <= ld &&
                  v_off + H * V <= ld && g_off + H * V <= ld,
              "projection columns out of range");
  TORCH_CHECK(gates.numel() == T * 2 * H, "gates must be [T, 2H]");
  TORCH_CHECK(norm_w.numel() == H * V, "norm weight must be [H*V]");
  TORCH_CHECK(S.dim() == 4 && S.size(1) == H && S.size(2) == D &&
                  S.size(3) == V,
              "S pool must be [slots, H, D, V]");
  TORCH_CHECK(n.numel() == S.size(0) * H * D && m.numel() == S.size(0) * H,
              "n / m pools do not match S");
  const bool summary = F_sum.has_value();
  if (summary) {
    MIX_F32(F_sum.value());
    TORCH_CHECK(F_sum->numel() == S.size(0) * H, "F_sum must be [slots, H]");
  }
  auto out = torch::empty({summary ? 0 : T, H * V}, proj.options());
  if (T == 0 || B == 0) return out;
  const int rc = tl_mlstm_seq(
      proj.data_ptr(), (int)ld, (int)q_off, (int)k_off, (int)v_off,
      (int)g_off, gates.data_ptr(), norm_w.data_ptr(), S.data_ptr(),
      n.data_ptr(), m.data_ptr(), cu.data_ptr(), slots.data_ptr(),
      pos0.data_ptr(), out.data_ptr(), B, (int)H, (int)D, (int)V, (float)cap,
      (float)qscale, (float)eps, summary ? F_sum->data_ptr() : nullptr,
      summary ? 1 : 0, io_is_f32(proj), mix_stream());
  TORCH_CHECK(rc == 0, "mlstm_seq: head sizes outside the kernel's range "
                       "(dim <= 256, vdim <= 1023)");
  return out;
}

void mlstm_chain(Tensor S_tmp, Tensor n_tmp, Tensor m_tmp, Tensor F_tmp,
                 Tensor S, Tensor n, Tensor m, Tensor chunk_base,
                 Tensor n_chunks, Tensor slots, Tensor pos0,
                 int64_t max_chunks) {
  MIX_F32(S_tmp);
  MIX_F32(n_tmp);
  MIX_F32(m_tmp);
  MIX_F32(F_tmp);
  MIX_F32(S);
  MIX_F32(n);
  MIX_F32(m);
  MIX_I32(chunk_base);
  MIX_I32(n_chunks);
  MIX_I32(slots);
  MIX_I32(pos0);
  TORCH_CHECK(S.dim() == 4 && S_tmp.dim() == 4, "S pools must be 4-d");
  const int H = S.size(1), D = S.size(2), V = S.size(3);
  TORCH_CHECK(S_tmp.size(1) == H && S_tmp.size(2) == D && S_tmp.size(3) == V,
              "chunk pool does not match the slot pool");
  const int64_t NC = S_tmp.size(0);
  TORCH_CHECK(n_tmp.numel() == NC * H * D && m_tmp.numel() == NC * H &&
                  F_tmp.numel() == NC * H,
              "chunk n / m / F pools do not match");
  const int B = slots.size(0);
  TORCH_CHECK(chunk_base.size(0) == B && n_chunks.size(0) == B &&
                  pos0.size(0) == B,
              "per-sequence chunk metadata");
  const int rc = tl_mlstm_chain(
      S_tmp.data_ptr(), n_tmp.data_ptr(), m_tmp.data_ptr(), F_tmp.data_ptr(),
      S.data_ptr(), n.data_ptr(), m.data_ptr(), chunk_base.data_ptr(),
      n_chunks.data_ptr(), slots.data_ptr(), pos0.data_ptr(), B,
      (int)max_chunks, H, D, V, mix_stream());
  TORCH_CHECK(rc == 0, "mlstm_chain: too many chunks in one sequence");
}

void kv_append(Tensor proj, int64_t k_off, int64_t v_off, Tensor kpool,
               Tensor vpool, Tensor tok_seq, Tensor tok_pos, Tensor table) {
  MIX_IN(proj);
  MIX_IN(kpool);
  MIX_IN(vpool);
  MIX_I32(tok_seq);
  MIX_I32(tok_pos);
  MIX_I32(table);
  TORCH_CHECK(kpool.scalar_type() == proj.scalar_type() &&
                  vpool.scalar_type() == proj.scalar_type(),
              "pool dtype must match activations");
  TORCH_CHECK(kpool.dim() == 4 && vpool.dim() == 4 && kpool.size(2) == 128 &&
                  vpool.size(2) == 128 && kpool.size(1) == vpool.size(1),
              "pools must be [pages, G, 128, *]");
  const int64_t T = proj.size(0), ld = proj.size(1);
  const int G = kpool.size(1), DK = kpool.size(3), V = vpool.size(3);
  TORCH_CHECK(k_off + G * DK <= ld && v_off + G * V <= ld,
              "projection columns out of range");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T && table.dim() == 2,
              "ragged metadata");
  tl_kv_append(proj.data_ptr(), (int)ld, (int)k_off, (int)v_off,
               kpool.data_ptr(), vpool.data_ptr(), tok_seq.data_ptr(),
               tok_pos.data_ptr(), table.data_ptr(), (int)table.size(1),
               (int)T, G, DK, V, io_is_f32(proj), mix_stream());
}

// n_split > 1 spreads every row's keys over that many blocks (few rows
// over long contexts: decoding) and merges them in a second kernel.
Tensor diff_attn_rows(Tensor q, int64_t q_off, Tensor kpool, Tensor vpool,
                      Tensor tok_seq, Tensor tok_pos, Tensor table,
                      Tensor lam, int64_t H, int64_t D, double scale,
                      double diff, double eps, int64_t n_split) {
  MIX_IN(q);
  MIX_IN(kpool);
  MIX_IN(vpool);
  MIX_I32(tok_seq);
  MIX_I32(tok_pos);
  MIX_I32(table);
  MIX_F32(lam);
  TORCH_CHECK(kpool.scalar_type() == q.scalar_type() &&
                  vpool.scalar_type() == q.scalar_type(),
              "pool dtype must match activations");
  TORCH_CHECK(kpool.dim() == 4 && vpool.dim() == 4 && kpool.size(2) == 128 &&
                  vpool.size(2) == 128 && kpool.size(1) == vpool.size(1) &&
                  kpool.size(3) == 2 * D,
              "pools must be [pages, G, 128, 2D] / [pages, G, 128, V]");
  const int64_t T = q.size(0), ld = q.size(1);
  const int G = kpool.size(1), V = vpool.size(3);
  TORCH_CHECK(q_off + H * 2 * D <= ld, "query columns out of range");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T && table.dim() == 2,
              "ragged metadata");
  auto out = torch::empty({T, H * V}, q.options());
  if (T == 0) return out;
  TORCH_CHECK(n_split >= 1 && n_split <= 64, "n_split out of range");
  Tensor part;
  if (n_split > 1)
    part = torch::empty({T * H * n_split * (4 + 2 * V)},
                        q.options().dtype(torch::kFloat));
  const int rc = tl_diff_attn_rows(
      q.data_ptr(), (int)ld, (int)q_off, kpool.data_ptr(), vpool.data_ptr(),
      tok_seq.data_ptr(), tok_pos.data_ptr(), table.data_ptr(),
      (int)table.size(1), lam.data_ptr(), out.data_ptr(),
      n_split > 1 ? part.data_ptr() : nullptr, (int)n_split, (int)T, (int)H,
      G, (int)D, V, (float)scale, (float)diff, (float)eps, io_is_f32(q),
      mix_stream());
  TORCH_CHECK(rc == 0, "diff_attn_rows: shape outside the kernel's range "
                       "(vdim <= 512, heads divisible by kv heads)");
  return out;
}

// MFMA path for prompt portions (bf16): `tiles` [n, 4] int32 rows of
// (sequence, first flat token, token count <= 64, first position).
// Returns false when the shape is outside the kernel's range.
bool diff_attn_tiles(Tensor q, int64_t q_off, Tensor kpool, Tensor vpool,
                     Tensor tiles, Tensor table, Tensor lam, Tensor out,
                     int64_t H, int64_t D, double scale, double diff,
                     double eps) {
  MIX_IN(q);
  MIX_IN(kpool);
  MIX_IN(vpool);
  MIX_IN(out);
  MIX_I32(tiles);
  MIX_I32(table);
  MIX_F32(lam);
  TORCH_CHECK(q.scalar_type() == torch::kBFloat16 &&
                  kpool.scalar_type() == torch::kBFloat16 &&
                  vpool.scalar_type() == torch::kBFloat16 &&
                  out.scalar_type() == torch::kBFloat16,
              "the tiled kernel is bf16 only");
  TORCH_CHECK(kpool.dim() == 4 && vpool.dim() == 4 && kpool.size(2) == 128 &&
                  vpool.size(2) == 128 && kpool.size(1) == vpool.size(1) &&
                  kpool.size(3) == 2 * D,
              "pools must be [pages, G, 128, 2D] / [pages, G, 128, V]");
  const int64_t T = q.size(0), ld = q.size(1);
  const int G = kpool.size(1), V = vpool.size(3);
  TORCH_CHECK(q_off + H * 2 * D <= ld, "query columns out of range");
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 4 && table.dim() == 2,
              "tiles must be [n, 4]");
  TORCH_CHECK(out.numel() == T * H * V, "out must be [T, H*V]");
  const int rc = tl_diff_attn_tiles(
      q.data_ptr(), (int)ld, (int)q_off, kpool.data_ptr(), vpool.data_ptr(),
      tiles.data_ptr(), (int)tiles.size(0), table.data_ptr(),
      (int)table.size(1), lam.data_ptr(), out.data_ptr(), (int)H, G, (int)D,
      V, (float)scale, (float)diff, (float)eps, mix_stream());
  return rc == 0;
}

}  // namespace

void register_mix_ops(pybind11::module& mod) {
  mod.def("hyper_dyt", &hyper_dyt,
          "hyper-connection update + Dynamic-Tanh norm over fp32 streams");
  mod.def("relu_sq", &relu_sq, "relu(x)^2");
  mod.def("mlstm_seq", &mlstm_seq,
          "matrix-memory recurrence over ragged sequences (slot state)");
  mod.def("mlstm_chain", &mlstm_chain,
          "chain per-chunk mLSTM summaries into per-chunk start states");
  mod.def("kv_append", &kv_append, "scatter new K/V rows into page pools");
  mod.def("diff_attn_tiles", &diff_attn_tiles,
          "differential attention on MFMA, 64-query tiles, paged KV (bf16)");
  mod.def("diff_attn_rows", &diff_attn_rows,
          "differential attention, one query token per block, paged KV");
}
