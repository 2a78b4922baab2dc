// torch.ops.hipserve_seq.* — the layer-list decoders' kernels (csrc/kernels/seq/*.hip), built as
// their own library (hipserve/_C_seq.so) so a model of these designs compiles only what it runs.
// All ops write into caller-provided outputs (no allocation except moe_align's scratch, no host sync).
#include <torch/library.h>
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "hipserve/kernels.h"
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

void latent_prepare(at::Tensor& cq, at::Tensor& cache, const at::Tensor& proj, const at::Tensor& positions,
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

void latent_attention(at::Tensor& o_lat, const at::Tensor& q_abs, const at::Tensor& q, const at::Tensor& proj,
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

// bf16 prompt portions on the matrix cores: qc (scratch) [heads, T, kv_rank + rot_dim] is filled here.
void latent_attention_mfma(at::Tensor& o_lat, at::Tensor& qc, const c10::optional<at::Tensor>& q_abs, const at::Tensor& q,
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

bool latent_attention_mfma_ok(int64_t kv_rank, int64_t rot_dim) {
  return hipserve::latent_attention_mfma_ok(kv_rank, rot_dim);
}

void mingru_scan(at::Tensor& y, at::Tensor& state, const at::Tensor& proj, const at::Tensor& b_z,
                 const at::Tensor& b_x, const at::Tensor& seq_cu, const at::Tensor& seq_ctx,
                 const at::Tensor& seq_state, int64_t max_q) {
  CHECK_DEV(proj); CHECK_CONTIG(proj); CHECK_CONTIG(y); CHECK_F32(state); CHECK_F32(b_z); CHECK_F32(b_x);
  CHECK_I32(seq_cu); CHECK_I32(seq_ctx); CHECK_I32(seq_state);
  const bool f32 = is_f32(proj, "mingru_scan");
  TORCH_CHECK(y.scalar_type() == proj.scalar_type());
  const long width = state.size(1), nseq = seq_ctx.numel();
  TORCH_CHECK(proj.dim() == 2 && proj.size(1) == 3 * width && y.numel() == proj.size(0) * width);
  TORCH_CHECK(b_z.numel() == width && b_x.numel() == width);
  TORCH_CHECK(seq_cu.numel() == nseq + 1 && seq_state.numel() >= nseq);
  c10::hip::HIPGuardMasqueradingAsCUDA g(proj.device());
  hipserve::launch_mingru_scan(y.data_ptr(), state.data_ptr<float>(), proj.data_ptr(), b_z.data_ptr<float>(),
                               b_x.data_ptr<float>(), seq_cu.data_ptr<int>(), seq_ctx.data_ptr<int>(),
                               seq_state.data_ptr<int>(), nseq, width, max_q, f32, cur_stream());
}

using hipserve_shared::expert_gemm;
using hipserve_shared::moe_align;

}  // namespace

TORCH_LIBRARY(hipserve_seq, m) {
  m.def("scaled_add_group_rmsnorm(Tensor(a!) out, Tensor(b!) residual, Tensor w, int groups, float eps, Tensor? mix, "
        "Tensor? ls1, Tensor? y, Tensor? pair_slot, int top, Tensor? ls2, Tensor? extra) -> ()");
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
  m.def("mingru_scan(Tensor(a!) y, Tensor(b!) state, Tensor proj, Tensor b_z, Tensor b_x, Tensor seq_cu, "
        "Tensor seq_ctx, Tensor seq_state, int max_q) -> ()");
  m.def("moe_align(Tensor ids, int E, int tile, Tensor(a!) slots, Tensor(b!) tile_expert, Tensor(c!) pair_slot) -> ()");
  m.def("expert_gemm(Tensor(a!) out, Tensor x, Tensor w, Tensor slots, Tensor tile_expert, int tile, int gather_k, "
        "int act) -> ()");
}

TORCH_LIBRARY_IMPL(hipserve_seq, CUDA, m) {
  m.impl("scaled_add_group_rmsnorm", &scaled_add_group_rmsnorm);
  m.impl("latent_prepare", &latent_prepare);
  m.impl("latent_attention", &latent_attention);
  m.impl("latent_attention_mfma", &latent_attention_mfma);
  m.impl("mingru_scan", &mingru_scan);
  m.impl("moe_align", &moe_align);
  m.impl("expert_gemm", &expert_gemm);
}
