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

namespace {

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

#define CHECK_DEV(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU tensor")
#define CHECK_CONTIG(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_F32(x) TORCH_CHECK((x).scalar_type() == at::kFloat && (x).is_contiguous(), #x " must be contiguous fp32")
#define CHECK_I32(x) TORCH_CHECK((x).scalar_type() == at::kInt && (x).is_contiguous(), #x " must be contiguous int32")

bool is_f32(const at::Tensor& t, const char* who) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, who, ": bf16 or fp32 activations");
  return t.scalar_type() == at::kFloat;
}

const void* opt_ptr(const c10::optional<at::Tensor>& t) { return t.has_value() ? t->data_ptr() : nullptr; }

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

bool rows2d(const at::Tensor& t) { return t.dim() == 2 && t.stride(1) == 1; }

void attn_prepare(at::Tensor& proj, const c10::optional<at::Tensor>& cache, const at::Tensor& positions,
                  const at::Tensor& slots, const at::Tensor& inv_freq, int64_t heads, int64_t kv_heads, int64_t maps,
                  int64_t dim, int64_t vdim, const c10::optional<at::Tensor>& q_norm,
                  const c10::optional<at::Tensor>& k_norm, int64_t norm_mode, bool v_norm, double eps) {
  CHECK_DEV(proj); CHECK_F32(inv_freq);
  const bool f32 = is_f32(proj, "attn_prepare");
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dim >= 1 && vdim >= 1 && (maps == 1 || maps == 2));
  TORCH_CHECK(norm_mode >= 0 && norm_mode <= 2 && (heads + kv_heads) * maps <= 8192);
  const long T = proj.size(0), nq = heads * maps * dim, nk = kv_heads * maps * dim, nv = kv_heads * vdim;
  const bool own_kv = cache.has_value();
  TORCH_CHECK(rows2d(proj) && proj.size(1) >= nq + (own_kv ? nk + nv : 0));
  if (own_kv) {
    CHECK_CONTIG(*cache);
    TORCH_CHECK(cache->scalar_type() == proj.scalar_type() && cache->dim() == 3 && cache->size(2) == nk + nv);
  }
  TORCH_CHECK(positions.scalar_type() == at::kLong && slots.scalar_type() == at::kLong && positions.numel() >= T &&
              slots.numel() >= T && positions.is_contiguous() && slots.is_contiguous());
  TORCH_CHECK(2 * inv_freq.numel() <= dim, "rotated dims exceed the head size");
  TORCH_CHECK((norm_mode != 0) == q_norm.has_value() && (!own_kv || q_norm.has_value() == k_norm.has_value()));
  if (q_norm.has_value()) {
    CHECK_F32(*q_norm);
    TORCH_CHECK(q_norm->numel() == (norm_mode == 2 ? dim : nq));
    if (own_kv) {
      CHECK_F32(*k_norm);
      TORCH_CHECK(k_norm->numel() == (norm_mode == 2 ? dim : nk));
    }
  }
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_attn_prepare(proj.data_ptr(), proj.stride(0), own_kv ? cache->data_ptr() : nullptr,
                                positions.data_ptr<long>(), slots.data_ptr<long>(), inv_freq.data_ptr<float>(),
                                inv_freq.numel(), T, heads, kv_heads, maps, dim, vdim, (const float*)opt_ptr(q_norm),
                                own_kv ? (const float*)opt_ptr(k_norm) : nullptr, norm_mode, v_norm, (float)eps, f32,
                                cur_stream());
}

void window_attention(at::Tensor& out, const at::Tensor& proj, const at::Tensor& cache, const at::Tensor& seq_cu,
                      const at::Tensor& seq_ctx, const at::Tensor& seq_bt, int64_t seq0, int64_t seq1,
                      int64_t rows_bound, int64_t tq, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                      int64_t gate_off, double scale, int64_t window, bool sink, double out_scale, int64_t maps,
                      double lam, double post, double eps) {
  CHECK_DEV(proj); CHECK_CONTIG(cache); CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_bt);
  const bool f32 = is_f32(proj, "window_attention");
  TORCH_CHECK(maps == 1 || maps == 2);
  TORCH_CHECK(out.scalar_type() == proj.scalar_type() && cache.scalar_type() == proj.scalar_type());
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dim >= 1 && vdim >= 1 &&
              vdim <= hipserve::window_attention_max_vdim() && dim <= 1024, "window_attention: head sizes");
  const long T = proj.size(0);
  TORCH_CHECK(rows2d(proj) && proj.size(1) >= heads * maps * dim && (gate_off < 0 || proj.size(1) >= gate_off + heads));
  TORCH_CHECK(rows2d(out) && out.size(0) == T && out.size(1) == heads * vdim);
  TORCH_CHECK(cache.dim() == 3 && cache.size(2) == kv_heads * (maps * dim + vdim));
  const long nseq = seq_ctx.numel();
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_bt.dim() == 2 && seq_bt.size(0) >= nseq);
  TORCH_CHECK(0 <= seq0 && seq0 <= seq1 && seq1 <= nseq && rows_bound <= T && window >= 0);
  TORCH_CHECK(tq == 1 || tq == 2 || tq == 4 || tq == 8 || tq == 16, "tokens per workgroup: 1, 2, 4, 8 or 16");
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_window_attention(out.data_ptr(), out.stride(0), proj.data_ptr(), proj.stride(0), cache.data_ptr(),
                                    cache.size(1), seq_cu.data_ptr<int>(), seq_ctx.data_ptr<int>(),
                                    seq_bt.data_ptr<int>(), seq_bt.size(1), seq0, seq1, rows_bound, tq, heads, kv_heads,
                                    dim, vdim, gate_off, (float)scale, window, sink, (float)out_scale, maps, (float)lam,
                                    (float)post, (float)eps, f32, cur_stream());
}

bool window_attention_mfma_ok(int64_t dim, int64_t vdim, int64_t out_ld, int64_t out_off, int64_t maps) {
  return hipserve::window_attention_mfma_ok(dim, vdim, out_ld, out_off, maps);
}

void window_attention_mfma(at::Tensor& out, const at::Tensor& proj, const at::Tensor& cache, const at::Tensor& seq_cu,
                           const at::Tensor& seq_ctx, const at::Tensor& seq_bt, int64_t seq0, int64_t seq1,
                           int64_t rows_bound, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                           int64_t gate_off, double scale, int64_t window, bool sink, double out_scale, int64_t nparts,
                           int64_t part_keys, const c10::optional<at::Tensor>& ws_acc,
                           const c10::optional<at::Tensor>& ws_ml, int64_t row_base, int64_t maps, double lam,
                           double post, double eps) {
  CHECK_DEV(proj); CHECK_CONTIG(cache); CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_bt);
  TORCH_CHECK(proj.scalar_type() == at::kBFloat16 && out.scalar_type() == at::kBFloat16 &&
              cache.scalar_type() == at::kBFloat16, "window_attention_mfma: bf16 only");
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0);
  const long T = proj.size(0);
  TORCH_CHECK(rows2d(proj) && proj.size(1) >= heads * maps * dim && (gate_off < 0 || proj.size(1) >= gate_off + heads));
  TORCH_CHECK(rows2d(out) && out.size(0) == T && out.size(1) == heads * vdim);
  TORCH_CHECK(hipserve::window_attention_mfma_ok(dim, vdim, out.stride(0), out.storage_offset(), maps),
              "window_attention_mfma: unsupported head sizes or output alignment");
  TORCH_CHECK(cache.dim() == 3 && cache.size(2) == kv_heads * (maps * dim + vdim));
  const long nseq = seq_ctx.numel();
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_bt.dim() == 2 && seq_bt.size(0) >= nseq);
  TORCH_CHECK(0 <= seq0 && seq0 <= seq1 && seq1 <= nseq && window >= 0);
  TORCH_CHECK(nparts >= 1 && nparts <= 64 && row_base >= 0 && row_base + rows_bound <= T);
  float *wa = nullptr, *wm = nullptr;
  if (nparts > 1) {
    TORCH_CHECK(part_keys > 0 && part_keys % 32 == 0 && ws_acc.has_value() && ws_ml.has_value());
    TORCH_CHECK(ws_acc->scalar_type() == at::kFloat && ws_acc->is_contiguous() &&
                ws_acc->numel() >= nparts * heads * maps * rows_bound * vdim);
    TORCH_CHECK(ws_ml->scalar_type() == at::kFloat && ws_ml->is_contiguous() &&
                ws_ml->numel() >= nparts * heads * maps * rows_bound * 2);
    wa = ws_acc->data_ptr<float>();
    wm = ws_ml->data_ptr<float>();
  }
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_window_attention_mfma(out.data_ptr(), out.stride(0), proj.data_ptr(), proj.stride(0),
                                         cache.data_ptr(), cache.size(1), seq_cu.data_ptr<int>(),
                                         seq_ctx.data_ptr<int>(), seq_bt.data_ptr<int>(), seq_bt.size(1), seq0, seq1,
                                         rows_bound, heads, kv_heads, dim, vdim, gate_off, (float)scale, window, sink,
                                         (float)out_scale, nparts, part_keys, wa, wm, row_base, maps, (float)lam,
                                         (float)post, (float)eps, cur_stream());
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

void activation(at::Tensor& out, const at::Tensor& x, int64_t kind, double c0, double c1) {
  CHECK_DEV(x);
  const bool f32 = is_f32(x, "activation");
  TORCH_CHECK(kind >= 0 && kind <= 3, "activation: 0 = tanh, 1 = xielu, 2 = relu2, 3 = silu_mul");
  TORCH_CHECK(out.scalar_type() == x.scalar_type() && rows2d(x) && rows2d(out) && out.size(0) == x.size(0));
  TORCH_CHECK(kind == 3 ? (x.size(1) == 2 * out.size(1) && out.data_ptr() != x.data_ptr()) : out.size(1) == x.size(1));
  c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
  hipserve::launch_activation(out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), x.size(0), out.size(1), kind,
                              (float)c0, (float)c1, f32, cur_stream());
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

void route_topk(at::Tensor& ids, at::Tensor& wts, const at::Tensor& logits, const at::Tensor& correction, int64_t top,
                double scale, int64_t E) {
  CHECK_DEV(logits); CHECK_F32(logits); CHECK_F32(correction); CHECK_F32(wts); CHECK_I32(ids);
  TORCH_CHECK(logits.dim() == 2);
  const long T = logits.size(0), n = logits.size(1);
  TORCH_CHECK(n >= 1 && n <= hipserve::route_topk_max_outputs() && correction.numel() == n && top >= 1 && top <= n);
  TORCH_CHECK(ids.numel() == T * top && wts.numel() == T * top && E >= 0 && E <= n);
  c10::hip::HIPGuardMasqueradingAsCUDA g(logits.device());
  hipserve::launch_route_topk(ids.data_ptr<int>(), wts.data_ptr<float>(), logits.data_ptr<float>(),
                              correction.data_ptr<float>(), T, n, top, (float)scale, E, cur_stream());
}

using hipserve_shared::expert_gemm;
using hipserve_shared::moe_align;

}  // namespace

TORCH_LIBRARY(hipserve_delta, m) {
  m.def("scaled_add_group_rmsnorm(Tensor(a!) out, Tensor(b!) residual, Tensor w, int groups, float eps, Tensor? mix, "
        "Tensor? ls1, Tensor? y, Tensor? pair_slot, int top, Tensor? ls2, Tensor? extra) -> ()");
  m.def("attn_prepare(Tensor(a!) proj, Tensor(b!)? cache, Tensor positions, Tensor slots, Tensor inv_freq, int heads, "
        "int kv_heads, int maps, int dim, int vdim, Tensor? q_norm, Tensor? k_norm, int norm_mode, bool v_norm, "
        "float eps) -> ()");
  m.def("window_attention(Tensor(a!) out, Tensor proj, Tensor cache, Tensor seq_cu, Tensor seq_ctx, Tensor seq_bt, "
        "int seq0, int seq1, int rows_bound, int tq, int heads, int kv_heads, int dim, int vdim, int gate_off, "
        "float scale, int window, bool sink, float out_scale, int maps, float lam, float post, float eps) -> ()");
  m.def("window_attention_mfma(Tensor(a!) out, Tensor proj, Tensor cache, Tensor seq_cu, Tensor seq_ctx, Tensor seq_bt, "
        "int seq0, int seq1, int rows_bound, int heads, int kv_heads, int dim, int vdim, int gate_off, float scale, "
        "int window, bool sink, float out_scale, int nparts, int part_keys, Tensor(b!)? ws_acc, Tensor(c!)? ws_ml, "
        "int row_base, int maps, float lam, float post, float eps) -> ()");
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
  m.def("route_topk(Tensor(a!) ids, Tensor(b!) wts, Tensor logits, Tensor correction, int top, float scale, int E) -> ()");
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
