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
#include "hipserve/seq_latent_bindings.h"

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

// bf16 prompt portions on the matrix cores: qc (scratch) [heads, T, kv_rank + rot_dim] is filled here.
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
