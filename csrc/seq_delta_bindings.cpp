// torch.ops.hipserve_delta.* — window attention (with a sink, or differential with two maps per head), the
// delta-rule and decayed linear-attention recurrences, token shift, the softmax router and the experts' GEMMs, and
// the elementwise activations of the layer-list decoders (csrc/kernels/seq/window_attention*.hip, delta_scan.hip,
// router.hip, expert_ffn.hip), plus the residual + norm kernels; built as their own library (hipserve/_C_delta.so) so a model compiles only
// what it runs.
// All ops write into caller-provided outputs (no allocation except moe_align's scratch, no host sync).
#include <torch/library.h>
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "hipserve/seq_kernels.h"
#include "hipserve/seq_shared_bindings.h"
#include "hipserve/seq_window_bindings.h"

namespace {

using namespace hipserve_shared;

void scaled_add_group_rmsnorm(at::Tensor& out, at::Tensor& residual, const at::Tensor& w, int64_t groups, double eps,
                              const c10::optional<at::Tensor>& mix, const c10::optional<at::Tensor>& ls1,
                              const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& pair_slot,
                              int64_t top, const c10::optional<at::Tensor>& ls2,
                              const c10::optional<at::Tensor>& extra) {
  CHECK_DEV(out); CHECK_CONTIG(out); CHECK_F32(residual); CHECK_F32(w);
  const bool f32 = is_f32(out, "scaled_add_group_rmsnorm");
  TORCH_CHECK(residual.dim() == 2 && out.sizes() == residual.sizes());
  const long T = residual.size(0), H = residual.size(1);
  TORCH_CHECK(groups >= 1 && H % groups == 0 && w.numel() == H && H + groups <= 15000, "group norm shape");
  if (mix.has_value()) {
    TORCH_CHECK(mix->scalar_type() == out.scalar_type() && mix->is_contiguous() && mix->sizes() == residual.sizes());
    TORCH_CHECK(!ls1.has_value() || (ls1->scalar_type() == at::kFloat && ls1->is_contiguous() && ls1->numel() == H));
  }
  if (y.has_value()) {
    TORCH_CHECK(y->scalar_type() == out.scalar_type() && y->is_contiguous() && y->dim() == 2 && y->size(1) == H);
    TORCH_CHECK(top >= 1 && pair_slot.has_value() && pair_slot->scalar_type() == at::kInt &&
                pair_slot->is_contiguous() && pair_slot->numel() >= T * top);
    TORCH_CHECK(ls2.has_value() && ls2->scalar_type() == at::kFloat && ls2->numel() == H);
  }
  if (extra.has_value())
    TORCH_CHECK(extra->scalar_type() == out.scalar_type() && extra->is_contiguous() && extra->sizes() == residual.sizes());
  c10::hip::HIPGuardMasqueradingAsCUDA g(out.device());
  hipserve::launch_scaled_add_group_rmsnorm(
      out.data_ptr(), residual.data_ptr<float>(), w.data_ptr<float>(), T, H, groups, (float)eps, opt_ptr(mix),
      (const float*)opt_ptr(ls1), opt_ptr(y), (const int*)opt_ptr(pair_slot), y.has_value() ? top : 0,
      (const float*)opt_ptr(ls2), opt_ptr(extra), f32, cur_stream());
}


void gated_delta(at::Tensor& y, at::Tensor& S, at::Tensor& conv_state, const at::Tensor& proj,
                 const at::Tensor& conv_w, const at::Tensor& a_log, const at::Tensor& dt_bias,
                 const at::Tensor& norm_w, const at::Tensor& seq_cu, const at::Tensor& seq_ctx,
                 const at::Tensor& seq_state, at::Tensor& scratch, int64_t heads, int64_t kv_heads, int64_t dim,
                 int64_t vdim, int64_t taps, double eps) {
  CHECK_DEV(proj); CHECK_CONTIG(y); CHECK_F32(S); CHECK_F32(conv_state); CHECK_F32(conv_w); CHECK_F32(a_log);
  CHECK_F32(dt_bias); CHECK_F32(norm_w); CHECK_F32(scratch); CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_state);
  const bool f32 = is_f32(proj, "gated_delta");
  TORCH_CHECK(y.scalar_type() == proj.scalar_type());
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dim >= 1 && dim <= hipserve::delta_max_dim() &&
              vdim >= 1 && taps >= 1 && taps <= hipserve::delta_max_taps(), "gated_delta: sizes");
  const long T = proj.size(0), nseq = seq_ctx.numel(), C = 2 * kv_heads * dim + heads * vdim;
  TORCH_CHECK(C * 4 <= 60 * 1024, "gated_delta: too many convolution channels");
  TORCH_CHECK(rows2d(proj) && proj.size(1) == C + 2 * heads + heads * vdim && y.numel() == T * heads * vdim);
  TORCH_CHECK(S.dim() == 4 && S.size(1) == heads && S.size(2) == dim && S.size(3) == vdim);
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(0) == S.size(0) && conv_state.size(2) == C &&
              conv_state.size(1) == (taps > 1 ? taps - 1 : 1));
  TORCH_CHECK(conv_w.numel() == C * taps && a_log.numel() == heads && dt_bias.numel() == heads && norm_w.numel() == vdim);
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_state.numel() >= nseq && nseq <= 65535);
  TORCH_CHECK(scratch.numel() >= T * (2 * kv_heads * dim + 2 * heads * vdim + 2 * heads));
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_gated_delta(y.data_ptr(), S.data_ptr<float>(), conv_state.data_ptr<float>(), proj.data_ptr(),
                               proj.stride(0), conv_w.data_ptr<float>(), a_log.data_ptr<float>(),
                               dt_bias.data_ptr<float>(), norm_w.data_ptr<float>(), seq_cu.data_ptr<int>(),
                               seq_ctx.data_ptr<int>(), seq_state.data_ptr<int>(), nseq, T, scratch.data_ptr<float>(),
                               heads, kv_heads, dim, vdim, taps, (float)eps, f32, cur_stream());
}

void delta_rule(at::Tensor& out, at::Tensor& S, const at::Tensor& proj, const at::Tensor& wl, const at::Tensor& a_b,
                const at::Tensor& w0, const at::Tensor& norm_w, const at::Tensor& seq_cu, const at::Tensor& seq_ctx,
                const at::Tensor& seq_state, at::Tensor& scratch, int64_t heads, int64_t dim, double eps,
                double out_scale) {
  CHECK_DEV(proj); CHECK_F32(S); CHECK_F32(wl); CHECK_F32(a_b); CHECK_F32(w0); CHECK_F32(norm_w); CHECK_F32(scratch);
  CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_state);
  const bool f32 = is_f32(proj, "delta_rule");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type());
  TORCH_CHECK(heads >= 1 && dim >= 1 && dim <= hipserve::delta_max_dim(), "delta_rule: sizes");
  const long T = proj.size(0), nseq = seq_ctx.numel(), N = heads * dim;
  TORCH_CHECK(rows2d(proj) && proj.size(1) >= 5 * N && rows2d(out) && out.size(0) == T && out.size(1) == N);
  TORCH_CHECK(S.dim() == 4 && S.size(1) == heads && S.size(2) == dim && S.size(3) == dim);
  TORCH_CHECK(wl.numel() == T * N && a_b.numel() == N && w0.numel() == N && norm_w.numel() == N);
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_state.numel() >= nseq && nseq <= 65535 &&
              scratch.numel() >= T * 7 * N);
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_delta_rule(out.data_ptr(), out.stride(0), S.data_ptr<float>(), proj.data_ptr(), proj.stride(0),
                              wl.data_ptr<float>(), a_b.data_ptr<float>(), w0.data_ptr<float>(),
                              norm_w.data_ptr<float>(), seq_cu.data_ptr<int>(), seq_ctx.data_ptr<int>(),
                              seq_state.data_ptr<int>(), nseq, T, scratch.data_ptr<float>(), heads, dim, (float)eps,
                              (float)out_scale, f32, cur_stream());
}

void add_normed(at::Tensor& out, at::Tensor& residual, const at::Tensor& w, double eps,
                const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& ye,
                const c10::optional<at::Tensor>& pair_slot, const c10::optional<at::Tensor>& ids,
                const c10::optional<at::Tensor>& wts, int64_t E, const c10::optional<at::Tensor>& h,
                const c10::optional<at::Tensor>& shared) {
  CHECK_DEV(out); CHECK_CONTIG(out); CHECK_F32(residual); CHECK_F32(w);
  const bool f32 = is_f32(out, "add_normed");
  TORCH_CHECK(residual.dim() == 2 && out.sizes() == residual.sizes());
  const long T = residual.size(0), H = residual.size(1);
  TORCH_CHECK(w.numel() == H && H <= 15000, "add_normed shape");
  auto same = [&](const at::Tensor& t) { return t.scalar_type() == out.scalar_type() && t.is_contiguous(); };
  long top = 0;
  if (y.has_value()) {
    TORCH_CHECK(same(*y) && y->sizes() == residual.sizes());
  } else {
    TORCH_CHECK(ye.has_value() && pair_slot.has_value() && ids.has_value() && wts.has_value() && h.has_value(),
                "add_normed: an addend or the parts of a mixture's output");
    CHECK_I32(*pair_slot); CHECK_I32(*ids); CHECK_F32(*wts);
    TORCH_CHECK(ids->dim() == 2 && ids->size(0) == T && wts->sizes() == ids->sizes());
    top = ids->size(1);
    TORCH_CHECK(same(*ye) && ye->dim() == 2 && ye->size(1) == H && pair_slot->numel() >= T * top);
    TORCH_CHECK(same(*h) && h->sizes() == residual.sizes() && h->data_ptr() != out.data_ptr());
    if (shared.has_value()) TORCH_CHECK(same(*shared) && shared->sizes() == residual.sizes());
  }
  c10::hip::HIPGuardMasqueradingAsCUDA g(out.device());
  hipserve::launch_add_normed(out.data_ptr(), residual.data_ptr<float>(), w.data_ptr<float>(), T, H, (float)eps,
                              opt_ptr(y), opt_ptr(ye), (const int*)opt_ptr(pair_slot), (const int*)opt_ptr(ids),
                              (const float*)opt_ptr(wts), top, E, opt_ptr(h), y.has_value() ? nullptr : opt_ptr(shared),
                              f32, cur_stream());
}

void token_shift(at::Tensor& out, const at::Tensor& x, at::Tensor& state, const at::Tensor& mu,
                 const at::Tensor& seq_cu, const at::Tensor& seq_ctx, const at::Tensor& seq_state) {
  CHECK_DEV(x); CHECK_CONTIG(out); CHECK_F32(x); CHECK_F32(state); CHECK_F32(mu);
  CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_state);
  const bool f32 = is_f32(out, "token_shift");
  TORCH_CHECK(x.dim() == 2 && out.dim() == 3 && mu.dim() == 2 && state.dim() == 2);
  const long T = x.size(0), H = x.size(1), nb = out.size(0), nseq = seq_ctx.numel();
  TORCH_CHECK(out.size(1) == T && out.size(2) == H && mu.size(0) == nb && mu.size(1) == H && state.size(1) == H);
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_state.numel() >= nseq && nseq <= 65535);
  c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
  hipserve::launch_token_shift(out.data_ptr(), x.data_ptr<float>(), state.data_ptr<float>(), mu.data_ptr<float>(),
                               seq_cu.data_ptr<int>(), seq_ctx.data_ptr<int>(), seq_state.data_ptr<int>(), nseq, T, H,
                               nb, f32, cur_stream());
}

void wkv(at::Tensor& out, at::Tensor& S, const at::Tensor& proj, const at::Tensor& wl, const at::Tensor& w0,
         const at::Tensor& u, const at::Tensor& norm_w, const at::Tensor& seq_cu, const at::Tensor& seq_ctx,
         const at::Tensor& seq_state, at::Tensor& scratch, int64_t heads, int64_t dim, double eps) {
  CHECK_DEV(proj); CHECK_CONTIG(proj); CHECK_CONTIG(out); CHECK_F32(S); CHECK_F32(wl); CHECK_F32(w0); CHECK_F32(u);
  CHECK_F32(norm_w); CHECK_F32(scratch); CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_state);
  const bool f32 = is_f32(proj, "wkv");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type());
  TORCH_CHECK(heads >= 1 && dim >= 1 && dim <= hipserve::delta_max_dim(), "wkv: sizes");
  const long N = heads * dim, nseq = seq_ctx.numel();
  TORCH_CHECK(proj.dim() == 3 && proj.size(0) == 4 && proj.size(2) == N);
  const long T = proj.size(1);
  TORCH_CHECK(out.numel() == T * N && wl.numel() == T * N && w0.numel() == N && u.numel() == N && norm_w.numel() == N);
  TORCH_CHECK(S.dim() == 4 && S.size(1) == heads && S.size(2) == dim && S.size(3) == dim);
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_state.numel() >= nseq && nseq <= 65535 &&
              scratch.numel() >= T * (5 * N + heads));
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_wkv(out.data_ptr(), S.data_ptr<float>(), proj.data_ptr(), wl.data_ptr<float>(),
                       w0.data_ptr<float>(), u.data_ptr<float>(), norm_w.data_ptr<float>(), seq_cu.data_ptr<int>(),
                       seq_ctx.data_ptr<int>(), seq_state.data_ptr<int>(), nseq, T, scratch.data_ptr<float>(), heads,
                       dim, (float)eps, f32, cur_stream());
}

void wkv_step(at::Tensor& out, at::Tensor& S, const at::Tensor& proj, const at::Tensor& low, const at::Tensor& w2,
              const at::Tensor& w0, const at::Tensor& u, const at::Tensor& norm_w, const at::Tensor& seq_cu,
              const at::Tensor& seq_ctx, const at::Tensor& seq_state, int64_t heads, int64_t dim, double eps) {
  CHECK_DEV(proj); CHECK_CONTIG(proj); CHECK_CONTIG(out); CHECK_CONTIG(low); CHECK_CONTIG(w2); CHECK_F32(S); CHECK_F32(w0);
  CHECK_F32(u); CHECK_F32(norm_w); CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_state);
  const bool f32 = is_f32(proj, "wkv_step");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type() && low.scalar_type() == proj.scalar_type() &&
              w2.scalar_type() == proj.scalar_type());
  TORCH_CHECK(heads >= 1 && dim >= 1 && dim <= 256, "wkv_step: sizes");
  const long N = heads * dim, nseq = seq_ctx.numel();
  TORCH_CHECK(proj.dim() == 3 && proj.size(0) == 4 && proj.size(2) == N);
  const long T = proj.size(1);
  TORCH_CHECK(low.dim() == 2 && low.size(0) == T && w2.dim() == 2 && w2.size(0) == N && w2.size(1) == low.size(1));
  const long rank = low.size(1);
  TORCH_CHECK((rank + 3 * dim) * 4 <= 60 * 1024, "wkv_step: bottleneck too wide");
  TORCH_CHECK(out.numel() == T * N && w0.numel() == N && u.numel() == N && norm_w.numel() == N);
  TORCH_CHECK(S.dim() == 4 && S.size(1) == heads && S.size(2) == dim && S.size(3) == dim);
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_state.numel() >= nseq && nseq <= 65535);
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_wkv_step(out.data_ptr(), S.data_ptr<float>(), proj.data_ptr(), T, low.data_ptr(), w2.data_ptr(), rank,
                            w0.data_ptr<float>(), u.data_ptr<float>(), norm_w.data_ptr<float>(),
                            seq_cu.data_ptr<int>(), seq_ctx.data_ptr<int>(), seq_state.data_ptr<int>(), nseq, heads,
                            dim, (float)eps, f32, cur_stream());
}

}  // namespace

TORCH_LIBRARY(hipserve_delta, m) {
  m.def("scaled_add_group_rmsnorm(Tensor(a!) out, Tensor(b!) residual, Tensor w, int groups, float eps, Tensor? mix, "
        "Tensor? ls1, Tensor? y, Tensor? pair_slot, int top, Tensor? ls2, Tensor? extra) -> ()");
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
  m.def("gated_delta(Tensor(a!) y, Tensor(b!) S, Tensor(c!) conv_state, Tensor proj, Tensor conv_w, Tensor a_log, "
        "Tensor dt_bias, Tensor norm_w, Tensor seq_cu, Tensor seq_ctx, Tensor seq_state, Tensor(d!) scratch, "
        "int heads, int kv_heads, int dim, int vdim, int taps, float eps) -> ()");
  m.def("delta_rule(Tensor(a!) out, Tensor(b!) S, Tensor proj, Tensor wl, Tensor a_b, Tensor w0, Tensor norm_w, "
        "Tensor seq_cu, Tensor seq_ctx, Tensor seq_state, Tensor(c!) scratch, int heads, int dim, float eps, "
        "float out_scale) -> ()");
  m.def("activation(Tensor(a!) out, Tensor x, int kind, float c0, float c1) -> ()");
  m.def("add_normed(Tensor(a!) out, Tensor(b!) residual, Tensor w, float eps, Tensor? y, Tensor? ye, Tensor? pair_slot, "
        "Tensor? ids, Tensor? wts, int E, Tensor? h, Tensor? shared) -> ()");
  m.def("token_shift(Tensor(a!) out, Tensor x, Tensor(b!) state, Tensor mu, Tensor seq_cu, Tensor seq_ctx, "
        "Tensor seq_state) -> ()");
  m.def("wkv(Tensor(a!) out, Tensor(b!) S, Tensor proj, Tensor wl, Tensor w0, Tensor u, Tensor norm_w, Tensor seq_cu, "
        "Tensor seq_ctx, Tensor seq_state, Tensor(c!) scratch, int heads, int dim, float eps) -> ()");
  m.def("wkv_step(Tensor(a!) out, Tensor(b!) S, Tensor proj, Tensor low, Tensor w2, Tensor w0, Tensor u, Tensor norm_w, "
        "Tensor seq_cu, Tensor seq_ctx, Tensor seq_state, int heads, int dim, float eps) -> ()");
  m.def("route_topk(Tensor(a!) ids, Tensor(b!) wts, Tensor logits, Tensor correction, int top, float scale, int E, "
        "int groups, int keep, bool renorm) -> ()");
  m.def("moe_align(Tensor ids, int E, int tile, Tensor(a!) slots, Tensor(b!) tile_expert, Tensor(c!) pair_slot) -> ()");
  m.def("expert_gemm(Tensor(a!) out, Tensor x, Tensor w, Tensor slots, Tensor tile_expert, int tile, int gather_k, "
        "int act) -> ()");
}

TORCH_LIBRARY_IMPL(hipserve_delta, CUDA, m) {
  m.impl("scaled_add_group_rmsnorm", &scaled_add_group_rmsnorm);
  m.impl("attn_prepare", &attn_prepare);
  m.impl("window_attention", &window_attention);
  m.impl("window_attention_mfma", &window_attention_mfma);
  m.impl("gated_delta", &gated_delta);
  m.impl("delta_rule", &delta_rule);
  m.impl("activation", &activation);
  m.impl("add_normed", &add_normed);
  m.impl("token_shift", &token_shift);
  m.impl("wkv", &wkv);
  m.impl("wkv_step", &wkv_step);
  m.impl("route_topk", &route_topk);
  m.impl("moe_align", &moe_align);
  m.impl("expert_gemm", &expert_gemm);
}
