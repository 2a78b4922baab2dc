// Bindings of the window-attention kernels, the softmax router and the activations (window_attention*.hip, router.hip,
// elementwise.hip), shared by the kernel libraries that link them.
#pragma once
#include "hipserve/seq_shared_bindings.h"

namespace hipserve_shared {

inline void attn_prepare(at::Tensor& proj, const c10::optional<at::Tensor>& cache, const at::Tensor& positions,
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

inline void window_attention(at::Tensor& out, const at::Tensor& proj, const at::Tensor& cache, const at::Tensor& seq_cu,
                      const at::Tensor& seq_ctx, const at::Tensor& seq_bt, int64_t seq0, int64_t seq1,
                      int64_t rows_bound, int64_t tq, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                      int64_t gate_off, double scale, int64_t window, bool sink, double out_scale, int64_t maps,
                      double lam, double post, double eps, int64_t keep, double softcap,
                      const c10::optional<at::Tensor>& sink_w) {
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
  TORCH_CHECK(keep >= 0 && softcap >= 0.0, "window_attention: kept first keys and score cap are not negative");
  if (sink_w.has_value()) {
    CHECK_F32(*sink_w);
    TORCH_CHECK(sink && sink_w->numel() == heads, "window_attention: one sink logit per head");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_window_attention(out.data_ptr(), out.stride(0), proj.data_ptr(), proj.stride(0), cache.data_ptr(),
                                    cache.size(1), seq_cu.data_ptr<int>(), seq_ctx.data_ptr<int>(),
                                    seq_bt.data_ptr<int>(), seq_bt.size(1), seq0, seq1, rows_bound, tq, heads, kv_heads,
                                    dim, vdim, gate_off, (float)scale, window, sink, (float)out_scale, maps, (float)lam,
                                    (float)post, (float)eps, keep, (float)softcap, (const float*)opt_ptr(sink_w), f32,
                                    cur_stream());
}

inline bool window_attention_mfma_ok(int64_t dim, int64_t vdim, int64_t out_ld, int64_t out_off, int64_t maps) {
  return hipserve::window_attention_mfma_ok(dim, vdim, out_ld, out_off, maps);
}

inline void window_attention_mfma(at::Tensor& out, const at::Tensor& proj, const at::Tensor& cache, const at::Tensor& seq_cu,
                           const at::Tensor& seq_ctx, const at::Tensor& seq_bt, int64_t seq0, int64_t seq1,
                           int64_t rows_bound, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                           int64_t gate_off, double scale, int64_t window, bool sink, double out_scale, int64_t nparts,
                           int64_t part_keys, const c10::optional<at::Tensor>& ws_acc,
                           const c10::optional<at::Tensor>& ws_ml, int64_t row_base, int64_t maps, double lam,
                           double post, double eps, int64_t keep, double softcap,
                           const c10::optional<at::Tensor>& sink_w) {
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
  TORCH_CHECK(keep >= 0 && softcap >= 0.0, "window_attention_mfma: kept first keys and score cap are not negative");
  if (sink_w.has_value()) {
    CHECK_F32(*sink_w);
    TORCH_CHECK(sink && sink_w->numel() == heads, "window_attention_mfma: one sink logit per head");
  }
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
                                         (float)post, (float)eps, keep, (float)softcap, (const float*)opt_ptr(sink_w),
                                         cur_stream());
}

inline void activation(at::Tensor& out, const at::Tensor& x, int64_t kind, double c0, double c1) {
  CHECK_DEV(x);
  const bool f32 = is_f32(x, "activation");
  TORCH_CHECK(kind >= 0 && kind <= 3, "activation: 0 = tanh, 1 = xielu, 2 = relu2, 3 = silu_mul");
  TORCH_CHECK(out.scalar_type() == x.scalar_type() && rows2d(x) && rows2d(out) && out.size(0) == x.size(0));
  TORCH_CHECK(kind == 3 ? (x.size(1) == 2 * out.size(1) && out.data_ptr() != x.data_ptr()) : out.size(1) == x.size(1));
  c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
  hipserve::launch_activation(out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), x.size(0), out.size(1), kind,
                              (float)c0, (float)c1, f32, cur_stream());
}

inline void route_topk(at::Tensor& ids, at::Tensor& wts, const at::Tensor& logits, const at::Tensor& correction, int64_t top,
                double scale, int64_t E, int64_t groups, int64_t keep, bool renorm) {
  CHECK_DEV(logits); CHECK_F32(logits); CHECK_F32(correction); CHECK_F32(wts); CHECK_I32(ids);
  TORCH_CHECK(logits.dim() == 2);
  const long T = logits.size(0), n = logits.size(1);
  TORCH_CHECK(n >= 1 && n <= hipserve::route_topk_max_outputs() && correction.numel() == n && top >= 1 && top <= n);
  TORCH_CHECK(ids.numel() == T * top && wts.numel() == T * top && E >= 0 && E <= n);
  TORCH_CHECK(groups >= 1 && groups <= 64 && n % groups == 0 && keep >= 1 && keep <= groups &&
              (groups == 1 || keep * (n / groups) >= top), "route_topk: groups of equal size that can hold the choice");
  c10::hip::HIPGuardMasqueradingAsCUDA g(logits.device());
  hipserve::launch_route_topk(ids.data_ptr<int>(), wts.data_ptr<float>(), logits.data_ptr<float>(),
                              correction.data_ptr<float>(), T, n, top, (float)scale, E, groups, keep, renorm,
                              cur_stream());
}

inline void polynorm(at::Tensor& out, const at::Tensor& x, const at::Tensor& coef, double eps) {
  CHECK_DEV(x); CHECK_F32(coef);
  const bool f32 = is_f32(x, "polynorm");
  TORCH_CHECK(out.scalar_type() == x.scalar_type() && rows2d(x) && rows2d(out) && out.sizes() == x.sizes() &&
              coef.numel() == 4, "polynorm: rows of one size and four coefficients");
  c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
  hipserve::launch_polynorm(out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), x.size(0), x.size(1),
                            coef.data_ptr<float>(), (float)eps, f32, cur_stream());
}

inline void gate_mul(at::Tensor& out, const at::Tensor& x, const at::Tensor& gate) {
  CHECK_DEV(x); CHECK_CONTIG(x); CHECK_CONTIG(out);
  const bool f32 = is_f32(x, "gate_mul");
  TORCH_CHECK(x.dim() == 3 && out.dim() == 2 && out.scalar_type() == x.scalar_type() && gate.scalar_type() == x.scalar_type());
  const long heads = x.size(0), T = x.size(1), d = x.size(2);
  TORCH_CHECK(out.size(0) == T && out.size(1) == heads * d && rows2d(gate) && gate.size(0) == T && gate.size(1) == heads * d,
              "gate_mul: out and gate [T, heads * d] for x [heads, T, d]");
  c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
  hipserve::launch_gate_mul(out.data_ptr(), x.data_ptr(), gate.data_ptr(), gate.stride(0), T, heads, d, f32, cur_stream());
}

}  // namespace hipserve_shared
