// torch.ops.hipserve_cell.* — the kernels of layer-list decoders built from parallel blocks with gated sublayer
// results: the block's residual update fused with the next norms (gated_block.hip), the mLSTM matrix memory
// (mlstm.hip), latent attention (latent_attention*.hip), window attention with capped scores, kept first keys and
// learned sinks (window_attention*.hip), the softmax router with group-limited selection (router.hip), the experts'
// GEMMs (expert_ffn.hip, moe.hip), PolyNorm, the gate multiply and the activations (elementwise.hip). Built as their
// own library (hipserve/_C_cell.so) so that a model compiles only what it runs.
// All ops write into caller-provided outputs (no allocation except moe_align's scratch, no host sync).
#include <torch/library.h>
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "hipserve/seq_kernels.h"
#include "hipserve/seq_shared_bindings.h"
#include "hipserve/seq_latent_bindings.h"
#include "hipserve/seq_window_bindings.h"

namespace {

using namespace hipserve_shared;

// One gated sublayer result: y [T, H] contiguous, g [T, H] with any row stride, b [H] fp32.
void check_sub(const at::Tensor& out, const c10::optional<at::Tensor>& g, const c10::optional<at::Tensor>& b, long T,
               long H) {
  TORCH_CHECK(g.has_value() && b.has_value(), "gated_add_norms: a sublayer result needs its gate and the gate's bias");
  TORCH_CHECK(g->scalar_type() == out.scalar_type() && rows2d(*g) && g->size(0) == T && g->size(1) == H);
  CHECK_F32(*b);
  TORCH_CHECK(b->numel() == H);
}

void gated_add_norms(at::Tensor& out1, const c10::optional<at::Tensor>& out2, at::Tensor& residual,
                     const at::Tensor& w1, const c10::optional<at::Tensor>& w2, double eps,
                     const c10::optional<at::Tensor>& y1, const c10::optional<at::Tensor>& g1,
                     const c10::optional<at::Tensor>& b1, const c10::optional<at::Tensor>& y2,
                     const c10::optional<at::Tensor>& g2, const c10::optional<at::Tensor>& b2,
                     const c10::optional<at::Tensor>& ye, const c10::optional<at::Tensor>& pair_slot,
                     const c10::optional<at::Tensor>& wts, const c10::optional<at::Tensor>& shared) {
  CHECK_DEV(out1); CHECK_CONTIG(out1); CHECK_F32(residual); CHECK_F32(w1);
  const bool f32 = is_f32(out1, "gated_add_norms");
  TORCH_CHECK(residual.dim() == 2 && out1.sizes() == residual.sizes());
  const long T = residual.size(0), H = residual.size(1);
  TORCH_CHECK(w1.numel() == 1 || w1.numel() == H, "gated_add_norms: one norm weight, or one per channel");
  TORCH_CHECK(out2.has_value() == w2.has_value());
  if (out2.has_value()) {
    CHECK_F32(*w2);
    TORCH_CHECK(out2->scalar_type() == out1.scalar_type() && out2->is_contiguous() && out2->sizes() == residual.sizes() &&
                (w2->numel() == 1 || w2->numel() == H));
  }
  auto same = [&](const at::Tensor& t) { return t.scalar_type() == out1.scalar_type() && t.is_contiguous(); };
  if (y1.has_value()) {
    TORCH_CHECK(same(*y1) && y1->sizes() == residual.sizes());
    check_sub(out1, g1, b1, T, H);
  }
  long top = 0;
  const bool second = g2.has_value();
  if (second) {
    check_sub(out1, g2, b2, T, H);
    if (y2.has_value()) {
      TORCH_CHECK(same(*y2) && y2->sizes() == residual.sizes());
    } else {
      TORCH_CHECK(ye.has_value() && pair_slot.has_value() && wts.has_value(),
                  "gated_add_norms: the second result is a row per token or the parts of a mixture's output");
      CHECK_I32(*pair_slot); CHECK_F32(*wts);
      TORCH_CHECK(wts->dim() == 2 && wts->size(0) == T);
      top = wts->size(1);
      TORCH_CHECK(same(*ye) && ye->dim() == 2 && ye->size(1) == H && pair_slot->numel() >= T * top);
      if (shared.has_value()) TORCH_CHECK(same(*shared) && shared->sizes() == residual.sizes());
    }
  }
  c10::hip::HIPGuardMasqueradingAsCUDA g(out1.device());
  hipserve::launch_gated_add_norms(
      out1.data_ptr(), out2.has_value() ? out2->data_ptr() : nullptr, residual.data_ptr<float>(), w1.data_ptr<float>(),
      w1.numel(), (const float*)opt_ptr(w2), w2.has_value() ? w2->numel() : 0, T, H, (float)eps, opt_ptr(y1),
      y1.has_value() ? g1->data_ptr() : nullptr, y1.has_value() ? g1->stride(0) : 0,
      y1.has_value() ? (const float*)opt_ptr(b1) : nullptr, second ? opt_ptr(y2) : nullptr,
      second ? g2->data_ptr() : nullptr, second ? g2->stride(0) : 0, second ? (const float*)opt_ptr(b2) : nullptr,
      opt_ptr(ye), (const int*)opt_ptr(pair_slot), (const float*)opt_ptr(wts), top,
      (second && !y2.has_value()) ? opt_ptr(shared) : nullptr, f32, cur_stream());
}

void mlstm(at::Tensor& out, at::Tensor& S, at::Tensor& N, at::Tensor& M, const at::Tensor& proj,
           const at::Tensor& gates, const at::Tensor& b_if, const at::Tensor& norm_w, const at::Tensor& seq_cu,
           const at::Tensor& seq_ctx, const at::Tensor& seq_state, at::Tensor& scratch, int64_t heads, int64_t dim,
           int64_t vdim, double cap, double eps, bool one_row_seqs) {
  CHECK_DEV(proj); CHECK_CONTIG(out); CHECK_F32(S); CHECK_F32(N); CHECK_F32(M); CHECK_F32(gates); CHECK_F32(b_if);
  CHECK_F32(norm_w); CHECK_F32(scratch); CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_state);
  const bool f32 = is_f32(proj, "mlstm");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type());
  TORCH_CHECK(heads >= 1 && dim >= 1 && dim <= hipserve::mlstm_max_dim() && vdim >= 1 && cap > 0.0, "mlstm: sizes");
  const long T = proj.size(0), nseq = seq_ctx.numel();
  TORCH_CHECK(rows2d(proj) && proj.size(1) >= 2 * heads * (dim + vdim) && out.numel() == T * heads * vdim);
  TORCH_CHECK(gates.dim() == 2 && gates.size(0) == T && gates.size(1) == 2 * heads && b_if.numel() == 2 * heads &&
              norm_w.numel() == heads * vdim);
  TORCH_CHECK(S.dim() == 4 && S.size(1) == heads && S.size(2) == dim && S.size(3) == vdim);
  TORCH_CHECK(N.dim() == 3 && N.size(0) == S.size(0) && N.size(1) == heads && N.size(2) == dim);
  TORCH_CHECK(M.dim() == 2 && M.size(0) == S.size(0) && M.size(1) == heads);
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_state.numel() >= nseq && nseq <= 65535);
  TORCH_CHECK(!one_row_seqs || T >= nseq, "mlstm: one row per sequence");
  TORCH_CHECK(scratch.numel() >= T * heads * (2 * dim + 2 * vdim + 6));
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_mlstm(out.data_ptr(), S.data_ptr<float>(), N.data_ptr<float>(), M.data_ptr<float>(), proj.data_ptr(),
                         proj.stride(0), gates.data_ptr<float>(), b_if.data_ptr<float>(), norm_w.data_ptr<float>(),
                         seq_cu.data_ptr<int>(), seq_ctx.data_ptr<int>(), seq_state.data_ptr<int>(), nseq, T,
                         scratch.data_ptr<float>(), heads, dim, vdim, (float)cap, (float)eps, one_row_seqs, f32,
                         cur_stream());
}

}  // namespace

TORCH_LIBRARY(hipserve_cell, m) {
  m.def("gated_add_norms(Tensor(a!) out1, Tensor(b!)? out2, Tensor(c!) residual, Tensor w1, Tensor? w2, float eps, "
        "Tensor? y1, Tensor? g1, Tensor? b1, Tensor? y2, Tensor? g2, Tensor? b2, Tensor? ye, Tensor? pair_slot, "
        "Tensor? wts, Tensor? shared) -> ()");
  m.def("mlstm(Tensor(a!) out, Tensor(b!) S, Tensor(c!) N, Tensor(d!) M, Tensor proj, Tensor gates, Tensor b_if, "
        "Tensor norm_w, Tensor seq_cu, Tensor seq_ctx, Tensor seq_state, Tensor(e!) scratch, int heads, int dim, "
        "int vdim, float cap, float eps, bool one_row_seqs) -> ()");
  m.def("polynorm(Tensor(a!) out, Tensor x, Tensor coef, float eps) -> ()");
  m.def("gate_mul(Tensor(a!) out, Tensor x, Tensor gate) -> ()");
  m.def("activation(Tensor(a!) out, Tensor x, int kind, float c0, float c1) -> ()");
  m.def("latent_prepare(Tensor(a!) cq, Tensor(b!) cache, Tensor proj, Tensor positions, Tensor slots, Tensor q_norm, "
        "Tensor kv_norm, Tensor inv_freq, int q_rank, int kv_rank, int rot_dim, float eps) -> ()");
  m.def("latent_attention(Tensor(a!) o_lat, Tensor q_abs, Tensor q, Tensor proj, Tensor cache, Tensor seq_cu, "
        "Tensor seq_ctx, Tensor seq_bt, int seq0, int seq1, int rows_bound, int tq, Tensor inv_freq, int heads, "
        "int dim, int rot_dim, int kv_rank, int gate_off, float scale, int window) -> ()");
  m.def("latent_attention_mfma(Tensor(a!) o_lat, Tensor(b!) qc, Tensor? q_abs, Tensor q, Tensor proj, Tensor positions, "
        "Tensor cache, Tensor seq_cu, Tensor seq_ctx, Tensor seq_bt, int seq0, int seq1, int rows_bound, "
        "Tensor inv_freq, int heads, int dim, int rot_dim, int kv_rank, int gate_off, float scale, int window, "
        "int nparts, int part_keys, Tensor(c!)? ws_acc, Tensor(d!)? ws_ml, int row_base, bool fill_qc) -> ()");
  m.def("latent_attention_mfma_ok(int kv_rank, int rot_dim) -> bool", &latent_attention_mfma_ok);
  m.def("attn_prepare(Tensor(a!) proj, Tensor(b!)? cache, Tensor positions, Tensor slots, Tensor inv_freq, int heads, "
        "int kv_heads, int maps, int dim, int vdim, Tensor? q_norm, Tensor? k_norm, int norm_mode, bool v_norm, "
        "float eps) -> ()");
  m.def("window_attention(Tensor(a!) out, Tensor proj, Tensor cache, Tensor seq_cu, Tensor seq_ctx, Tensor seq_bt, "
        "int seq0, int seq1, int rows_bound, int tq, int heads, int kv_heads, int dim, int vdim, int gate_off, "
        "float scale, int window, bool sink, float out_scale, int maps, float lam, float post, float eps, int keep, "
        "float softcap, Tensor? sink_w) -> ()");
  m.def("window_attention_mfma(Tensor(a!) out, Tensor proj, Tensor cache, Tensor seq_cu, Tensor seq_ctx, Tensor seq_bt, "
        "int seq0, int seq1, int rows_bound, int heads, int kv_heads, int dim, int vdim, int gate_off, float scale, "
        "int window, bool sink, float out_scale, int nparts, int part_keys, Tensor(b!)? ws_acc, Tensor(c!)? ws_ml, "
        "int row_base, int maps, float lam, float post, float eps, int keep, float softcap, Tensor? sink_w) -> ()");
  m.def("window_attention_mfma_ok(int dim, int vdim, int out_ld, int out_off, int maps) -> bool", &window_attention_mfma_ok);
  m.def("route_topk(Tensor(a!) ids, Tensor(b!) wts, Tensor logits, Tensor correction, int top, float scale, int E, "
        "int groups, int keep, bool renorm) -> ()");
  m.def("moe_align(Tensor ids, int E, int tile, Tensor(a!) slots, Tensor(b!) tile_expert, Tensor(c!) pair_slot) -> ()");
  m.def("expert_gemm(Tensor(a!) out, Tensor x, Tensor w, Tensor slots, Tensor tile_expert, int tile, int gather_k, "
        "int act) -> ()");
}

TORCH_LIBRARY_IMPL(hipserve_cell, CUDA, m) {
  m.impl("gated_add_norms", &gated_add_norms);
  m.impl("mlstm", &mlstm);
  m.impl("polynorm", &polynorm);
  m.impl("gate_mul", &gate_mul);
  m.impl("activation", &activation);
  m.impl("latent_prepare", &latent_prepare);
  m.impl("latent_attention", &latent_attention);
  m.impl("latent_attention_mfma", &latent_attention_mfma);
  m.impl("attn_prepare", &attn_prepare);
  m.impl("window_attention", &window_attention);
  m.impl("window_attention_mfma", &window_attention_mfma);
  m.impl("route_topk", &route_topk);
  m.impl("moe_align", &moe_align);
  m.impl("expert_gemm", &expert_gemm);
}
