// Residual update of a parallel block whose sublayers' results are gated per channel, fused with the
// norms that read the stream next, one workgroup per token row:
//   r = residual + sigmoid(g1 + b1) * y1 + sigmoid(g2 + b2) * y2                  (fp32, written back)
//   y2 = a dense feed-forward's row, or a mixture's output
//        shared + sum_j wts[t, j] * ye[pair_slot[t * top + j]]
//   out1 = r / sqrt(mean(r^2) + eps) * w1,   out2 = r / sqrt(mean(r^2) + eps) * w2
// Both norms read the same stream, so one mean square serves both; a norm weight is one number or a
// number per channel. g1 / g2 are column slices of the sublayers' merged projections (row strides
// of their own). Every addend is optional: without any the launch only norms the stream (the
// embedding output before the first block).
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kNT = 256;
constexpr int kPer = 8;   // channels per thread held in registers (H <= 2048); wider rows re-read the stream

template <typename T, bool REG>
__global__ __launch_bounds__(kNT) void gated_add_norms_kernel(
    T* __restrict__ out1, T* __restrict__ out2, float* __restrict__ residual, const float* __restrict__ w1, int w1n,
    const float* __restrict__ w2, int w2n, int H, float eps, const T* __restrict__ y1, const T* __restrict__ g1,
    long g1_ld, const float* __restrict__ b1, const T* __restrict__ y2, const T* __restrict__ g2, long g2_ld,
    const float* __restrict__ b2, const T* __restrict__ ye, const int* __restrict__ pair_slot,
    const float* __restrict__ wts, int top, const T* __restrict__ shared) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  float* r = residual + t * H;
  float keep[REG ? kPer : 1];
  float sq = 0.f;
  auto update = [&](int e) {
    float v = r[e];
    if (y1 != nullptr) v += sigmoid_f(ldf<T>(g1, t * g1_ld + e) + b1[e]) * ldf<T>(y1, t * H + e);
    if (g2 != nullptr) {
      float y;
      if (y2 != nullptr) {
        y = ldf<T>(y2, t * H + e);
      } else {
        y = shared != nullptr ? ldf<T>(shared, t * H + e) : 0.f;
        for (int j = 0; j < top; ++j) y += wts[t * top + j] * ldf<T>(ye, (long)pair_slot[t * top + j] * H + e);
      }
      v += sigmoid_f(ldf<T>(g2, t * g2_ld + e) + b2[e]) * y;
    }
    return v;
  };
  if constexpr (REG) {
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int e = tid + kNT * i;
      keep[i] = 0.f;
      if (e < H) {
        keep[i] = update(e);
        r[e] = keep[i];
        sq += keep[i] * keep[i];
      }
    }
  } else {
    for (int e = tid; e < H; e += kNT) {
      const float v = update(e);
      r[e] = v;
      sq += v * v;
    }
  }
  sq = block_sum(sq, red);
  const float inv = 1.f / sqrtf(sq / (float)H + eps);
  if constexpr (REG) {
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int e = tid + kNT * i;
      if (e < H) {
        const float v = keep[i] * inv;
        stf<T>(out1, t * H + e, v * w1[w1n == 1 ? 0 : e]);
        if (out2 != nullptr) stf<T>(out2, t * H + e, v * w2[w2n == 1 ? 0 : e]);
      }
    }
  } else {
    for (int e = tid; e < H; e += kNT) {  // the thread re-reads what it wrote itself
      const float v = r[e] * inv;
      stf<T>(out1, t * H + e, v * w1[w1n == 1 ? 0 : e]);
      if (out2 != nullptr) stf<T>(out2, t * H + e, v * w2[w2n == 1 ? 0 : e]);
    }
  }
}

}  // namespace

void launch_gated_add_norms(void* out1, void* out2, float* residual, const float* w1, int w1n, const float* w2, int w2n,
                            int T, int H, float eps, const void* y1, const void* g1, long g1_ld, const float* b1,
                            const void* y2, const void* g2, long g2_ld, const float* b2, const void* ye,
                            const int* pair_slot, const float* wts, int top, const void* shared, bool f32,
                            hipStream_t s) {
  if (T <= 0) return;
  const bool reg = H <= kNT * kPer;
#define HS_GB(TT, R)                                                                                                 \
  gated_add_norms_kernel<TT, R><<<T, kNT, 0, s>>>((TT*)out1, (TT*)out2, residual, w1, w1n, w2, w2n, H, eps,           \
                                                  (const TT*)y1, (const TT*)g1, g1_ld, b1, (const TT*)y2,             \
                                                  (const TT*)g2, g2_ld, b2, (const TT*)ye, pair_slot, wts, top,       \
                                                  (const TT*)shared)
  if (f32) { if (reg) HS_GB(float, true); else HS_GB(float, false); }
  else { if (reg) HS_GB(unsigned short, true); else HS_GB(unsigned short, false); }
#undef HS_GB
}

}  // namespace hipserve
