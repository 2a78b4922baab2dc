// Bindings of the latent-attention kernels (latent_attention*.hip), shared by the kernel libraries that link them.
#pragma once
#include "hipserve/seq_shared_bindings.h"

namespace hipserve_shared {

inline void latent_prepare(at::Tensor& cq, at::Tensor& cache, const at::Tensor& proj, const at::Tensor& positions,
                    const at::Tensor& slots, const at::Tensor& q_norm, const at::Tensor& kv_norm,
                    const at::Tensor& inv_freq, int64_t q_rank, int64_t kv_rank, int64_t rot_dim, double eps) {
  CHECK_DEV(proj); CHECK_CONTIG(cq); CHECK_CONTIG(cache); CHECK_F32(q_norm); CHECK_F32(kv_norm); CHECK_F32(inv_freq);
  const bool f32 = is_f32(proj, "latent_prepare");
  TORCH_CHECK(cq.scalar_type() == proj.scalar_type() && cache.scalar_type() == proj.scalar_type());
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(1) >= q_rank + kv_rank + rot_dim);
  const long T = proj.size(0);
  TORCH_CHECK(cq.numel() == T * q_rank && cache.dim() == 3 && cache.size(2) == kv_rank + rot_dim);
  TORCH_CHECK(positions.scalar_type() == at::kLong && slots.scalar_type() == at::kLong && positions.numel() >= T &&
              slots.numel() >= T && positions.is_contiguous() && slots.is_contiguous());
  TORCH_CHECK(q_norm.numel() == q_rank && kv_norm.numel() == kv_rank && 2 * inv_freq.numel() <= rot_dim);
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_latent_prepare(cq.data_ptr(), cache.data_ptr(), proj.data_ptr(), proj.stride(0),
                                  positions.data_ptr<long>(), slots.data_ptr<long>(), q_norm.data_ptr<float>(),
                                  kv_norm.data_ptr<float>(), inv_freq.data_ptr<float>(), inv_freq.numel(), T, q_rank,
                                  kv_rank, rot_dim, (float)eps, f32, cur_stream());
}

inline void latent_attention(at::Tensor& o_lat, const at::Tensor& q_abs, const at::Tensor& q, const at::Tensor& proj,
                      const at::Tensor& cache, const at::Tensor& seq_cu, const at::Tensor& seq_ctx,
                      const at::Tensor& seq_bt, int64_t seq0, int64_t seq1, int64_t rows_bound, int64_t tq,
                      const at::Tensor& inv_freq, int64_t heads, int64_t dim, int64_t rot_dim, int64_t kv_rank,
                      int64_t gate_off, double scale, int64_t window) {
  CHECK_DEV(q); CHECK_CONTIG(o_lat); CHECK_F32(q_abs); CHECK_CONTIG(q); CHECK_CONTIG(cache); CHECK_F32(inv_freq);
  CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_bt);
  const bool f32 = is_f32(q, "latent_attention");
  TORCH_CHECK(o_lat.scalar_type() == q.scalar_type() && cache.scalar_type() == q.scalar_type() &&
              proj.scalar_type() == q.scalar_type());
  const long T = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) == heads * (dim + rot_dim));
  TORCH_CHECK(q_abs.numel() == heads * T * kv_rank && o_lat.numel() == heads * T * kv_rank);
  TORCH_CHECK(cache.dim() == 3 && cache.size(2) == kv_rank + rot_dim && kv_rank <= 1024);
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) == T && proj.size(1) >= gate_off + heads);
  const long nseq = seq_ctx.numel();
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_bt.dim() == 2 && seq_bt.size(0) >= nseq);
  TORCH_CHECK(0 <= seq0 && seq0 <= seq1 && seq1 <= nseq && rows_bound <= T);
  TORCH_CHECK(tq == 1 || tq == 2 || tq == 4 || tq == 8 || tq == 16, "tokens per workgroup: 1, 2, 4, 8 or 16");
  TORCH_CHECK(2 * inv_freq.numel() <= rot_dim);
  c10::hip::HIPGuardMasqueradingAsCUDA g(q.device());
  hipserve::launch_latent_attention(o_lat.data_ptr(), q_abs.data_ptr<float>(), q.data_ptr(), proj.data_ptr(),
                                    proj.stride(0), cache.data_ptr(), cache.size(1), seq_cu.data_ptr<int>(),
                                    seq_ctx.data_ptr<int>(), seq_bt.data_ptr<int>(), seq_bt.size(1), seq0, seq1,
                                    rows_bound, tq, inv_freq.data_ptr<float>(), inv_freq.numel(), T, heads, dim,
                                    rot_dim, kv_rank, gate_off, (float)scale, window, f32, cur_stream());
}

inline void latent_attention_mfma(at::Tensor& o_lat, at::Tensor& qc, const c10::optional<at::Tensor>& q_abs, const at::Tensor& q,
                           const at::Tensor& proj, const at::Tensor& positions, const at::Tensor& cache,
                           const at::Tensor& seq_cu, const at::Tensor& seq_ctx, const at::Tensor& seq_bt, int64_t seq0,
                           int64_t seq1, int64_t rows_bound, const at::Tensor& inv_freq, int64_t heads, int64_t dim,
                           int64_t rot_dim, int64_t kv_rank, int64_t gate_off, double scale, int64_t window,
                           int64_t nparts, int64_t part_keys, const c10::optional<at::Tensor>& ws_acc,
                           const c10::optional<at::Tensor>& ws_ml, int64_t row_base, bool fill_qc) {
  CHECK_DEV(q); CHECK_CONTIG(o_lat); CHECK_CONTIG(qc); CHECK_CONTIG(q); CHECK_CONTIG(cache);
  CHECK_F32(inv_freq); CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_bt);
  if (q_abs.has_value()) CHECK_F32(*q_abs);
  TORCH_CHECK(q.scalar_type() == at::kBFloat16 && o_lat.scalar_type() == at::kBFloat16 &&
              qc.scalar_type() == at::kBFloat16 && cache.scalar_type() == at::kBFloat16 &&
              proj.scalar_type() == at::kBFloat16, "latent_attention_mfma: bf16 only");
  TORCH_CHECK(hipserve::latent_attention_mfma_ok(kv_rank, rot_dim), "latent_attention_mfma: unsupported latent sizes");
  const long T = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) == heads * (dim + rot_dim));
  TORCH_CHECK((!q_abs.has_value() || q_abs->numel() == heads * T * kv_rank) && o_lat.numel() == heads * T * kv_rank &&
              qc.numel() == heads * T * (kv_rank + rot_dim));
  TORCH_CHECK(cache.dim() == 3 && cache.size(2) == kv_rank + rot_dim);
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) == T && proj.size(1) >= gate_off + heads);
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.is_contiguous() && positions.numel() >= T);
  const long nseq = seq_ctx.numel();
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_bt.dim() == 2 && seq_bt.size(0) >= nseq);
  TORCH_CHECK(0 <= seq0 && seq0 <= seq1 && seq1 <= nseq && rows_bound <= T && 2 * inv_freq.numel() <= rot_dim);
  float *wa = nullptr, *wm = nullptr;
  TORCH_CHECK(nparts >= 1 && nparts <= 64 && row_base >= 0 && row_base + rows_bound <= T);
  if (nparts > 1) {
    TORCH_CHECK(part_keys > 0 && part_keys % 32 == 0 && ws_acc.has_value() && ws_ml.has_value());
    TORCH_CHECK(ws_acc->scalar_type() == at::kFloat && ws_acc->is_contiguous() &&
                ws_acc->numel() >= nparts * heads * rows_bound * kv_rank && kv_rank % 4 == 0);
    TORCH_CHECK(ws_ml->scalar_type() == at::kFloat && ws_ml->is_contiguous() &&
                ws_ml->numel() >= nparts * heads * rows_bound * 2);
    wa = ws_acc->data_ptr<float>();
    wm = ws_ml->data_ptr<float>();
  }
  c10::hip::HIPGuardMasqueradingAsCUDA g(q.device());
  if (fill_qc)
    hipserve::launch_latent_q_cat(qc.data_ptr(), q_abs.has_value() ? q_abs->data_ptr<float>() : nullptr, q.data_ptr(),
                                  positions.data_ptr<long>(),
                                  inv_freq.data_ptr<float>(), inv_freq.numel(), T, heads, dim, rot_dim, kv_rank,
                                  cur_stream());
  hipserve::launch_latent_attention_mfma(o_lat.data_ptr(), qc.data_ptr(), proj.data_ptr(), proj.stride(0),
                                         cache.data_ptr(), cache.size(1), seq_cu.data_ptr<int>(),
                                         seq_ctx.data_ptr<int>(), seq_bt.data_ptr<int>(), seq_bt.size(1), seq0, seq1,
                                         rows_bound, T, heads, rot_dim, kv_rank, gate_off, (float)scale, window,
                                         nparts, part_keys, wa, wm, row_base, cur_stream());
}

inline bool latent_attention_mfma_ok(int64_t kv_rank, int64_t rot_dim) {
  return hipserve::latent_attention_mfma_ok(kv_rank, rot_dim);
}

}  // namespace hipserve_shared
