// Bindings shared by the layer-list decoders' kernel libraries (each library links its own copy of the
// kernels): the expert alignment and the expert GEMMs of the mixtures of experts.
#pragma once
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include "hipserve/kernels.h"
#include "hipserve/seq_kernels.h"

namespace hipserve_shared {

inline hipStream_t cur_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

#define CHECK_DEV(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU tensor")
#define CHECK_CONTIG(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_F32(x) TORCH_CHECK((x).scalar_type() == at::kFloat && (x).is_contiguous(), #x " must be contiguous fp32")
#define CHECK_I32(x) TORCH_CHECK((x).scalar_type() == at::kInt && (x).is_contiguous(), #x " must be contiguous int32")

inline bool is_f32(const at::Tensor& t, const char* who) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, who, ": bf16 or fp32 activations");
  return t.scalar_type() == at::kFloat;
}

inline const void* opt_ptr(const c10::optional<at::Tensor>& t) { return t.has_value() ? t->data_ptr() : nullptr; }
inline bool rows2d(const at::Tensor& t) { return t.dim() == 2 && t.stride(1) == 1; }

inline void moe_align(const at::Tensor& ids, int64_t E, int64_t tile, at::Tensor& slots, at::Tensor& tile_expert,
                      at::Tensor& pair_slot) {
  auto i32 = [](const at::Tensor& t) { return t.scalar_type() == at::kInt && t.is_contiguous(); };
  TORCH_CHECK(ids.is_cuda() && i32(ids) && i32(slots) && i32(tile_expert) && i32(pair_slot), "moe_align: int32 GPU tensors");
  TORCH_CHECK(E >= 1 && E <= 128, "moe_align: at most 128 experts");
  TORCH_CHECK(tile == 16 || tile == 32 || tile == 64 || tile == 128 || tile == 256);
  const int npairs = ids.numel();
  TORCH_CHECK(slots.numel() >= npairs + E * (tile - 1) && slots.numel() % tile == 0,
              "slots capacity must cover padding and be a multiple of the tile");
  TORCH_CHECK(tile_expert.numel() * tile >= slots.numel() && pair_slot.numel() >= npairs);
  c10::hip::HIPGuardMasqueradingAsCUDA g(ids.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  const int nb = hipserve::moe_align_blocks(npairs);
  at::Tensor scratch = at::empty({(long)(nb > 1 ? nb : 0) * 128 + 1}, ids.options());  // [hist | tile count]
  hipserve::launch_moe_align(ids.data_ptr<int>(), npairs, E, tile, slots.data_ptr<int>(), slots.numel(),
                             tile_expert.data_ptr<int>(), tile_expert.numel(),
                             scratch.data_ptr<int>() + (scratch.numel() - 1), pair_slot.data_ptr<int>(), nullptr,
                             stream, nb > 1 ? scratch.data_ptr<int>() : nullptr);
}

inline void expert_gemm(at::Tensor& out, const at::Tensor& x, const at::Tensor& w, const at::Tensor& slots,
                        const at::Tensor& tile_expert, int64_t tile, int64_t gather_k, int64_t act) {
  auto i32 = [](const at::Tensor& t) { return t.scalar_type() == at::kInt && t.is_contiguous(); };
  TORCH_CHECK(x.is_cuda() && out.is_contiguous() && w.is_contiguous() && i32(slots) && i32(tile_expert));
  TORCH_CHECK(x.scalar_type() == at::kFloat || x.scalar_type() == at::kBFloat16, "expert_gemm: bf16 or fp32 activations");
  const bool f32 = x.scalar_type() == at::kFloat;
  TORCH_CHECK(out.scalar_type() == x.scalar_type() && w.scalar_type() == x.scalar_type());
  TORCH_CHECK(w.dim() == 3 && x.dim() == 2 && x.stride(1) == 1 && out.dim() == 2);
  const long N = w.size(1), K = w.size(2), cap = slots.numel();
  TORCH_CHECK(act >= 0 && act <= 2 && (act != 2 || N % 2 == 0), "expert_gemm: act 0 (none), 1 (relu^2), 2 (silu gate)");
  TORCH_CHECK(x.size(1) == K && out.size(1) == (act == 2 ? N / 2 : N) && out.size(0) >= cap);
  TORCH_CHECK(tile % 32 == 0 && cap % tile == 0 && tile_expert.numel() * tile >= cap, "tiles of a multiple of 32 slots");
  TORCH_CHECK(gather_k > 0 || x.size(0) >= cap, "ungathered x needs one row per slot");
  c10::hip::HIPGuardMasqueradingAsCUDA g(x.device());
  hipserve::launch_expert_gemm(out.data_ptr(), x.data_ptr(), x.stride(0), w.data_ptr(), slots.data_ptr<int>(),
                               tile_expert.data_ptr<int>(), cap / tile, tile, gather_k, N, K, act, w.size(0), f32,
                               c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
}

}  // namespace hipserve_shared
