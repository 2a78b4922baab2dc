// Residual update + grouped RMSNorm of the layer-list decoders, one workgroup per token row:
//   r = residual + ls1 * mix (ls1 null: 1) + ls2 * (1/top) * sum_j y[pair_slot[t*top + j]] + extra     (fp32, written back)
//   out = r / sqrt(mean over the element's group of r^2 + eps) * w
// The row is split into `groups` equal consecutive parts with their own mean square. The MoE
// combine (rows of the expert-sorted y picked through pair_slot) and the embedding re-added at
// the start of a loop pass (`extra`) ride along, so one launch sits between two layers.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kNT = 256;

template <typename T>
__global__ __launch_bounds__(kNT) void scaled_add_group_rmsnorm_kernel(
    T* __restrict__ out, float* __restrict__ residual, const float* __restrict__ w, int H, int groups, float eps,
    const T* __restrict__ mix, const float* __restrict__ ls1, const T* __restrict__ y,
    const int* __restrict__ pair_slot, int top, const float* __restrict__ ls2, const T* __restrict__ extra) {
  extern __shared__ float sm[];  // [H] squares, then [groups] inverse rms
  float* sq = sm;
  float* ginv = sm + H;
  const long t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* r = residual + t * H;
  const float wtop = top > 0 ? 1.f / (float)top : 0.f;
  for (int e = tid; e < H; e += kNT) {
    float v = r[e];
    if (mix != nullptr) v += ls1 != nullptr ? ldf<T>(mix, t * H + e) * ls1[e] : ldf<T>(mix, t * H + e);
    if (y != nullptr) {
      float f = 0.f;
      for (int j = 0; j < top; ++j) f += ldf<T>(y, (long)pair_slot[t * top + j] * H + e);
      v += f * wtop * ls2[e];
    }
    if (extra != nullptr) v += ldf<T>(extra, t * H + e);
    r[e] = v;
    sq[e] = v * v;
  }
  __syncthreads();
  const int gs = H / groups;
  for (int g = wave; g < groups; g += kNT / 64) {  // one wave sums a group, in a fixed order
    float a = 0.f;
    for (int e = lane; e < gs; e += 64) a += sq[g * gs + e];
    a = wave_sum(a);
    if (lane == 0) ginv[g] = 1.f / sqrtf(a / (float)gs + eps);
  }
  __syncthreads();
  for (int e = tid; e < H; e += kNT) stf<T>(out, t * H + e, r[e] * ginv[e / gs] * w[e]);
}

// Residual update with the norm on the sublayer's OUTPUT, one workgroup per token row:
//   y = addend row, or the mixture's output
//       shared + sum_j wts[t, j] * (ids[t, j] < E ? ye[pair_slot[t * top + j]] : h[t])      (fp32)
//   residual += y / sqrt(mean(y^2) + eps) * w        (fp32, written back);  out = residual in T
template <typename T>
__global__ __launch_bounds__(kNT) void add_normed_kernel(
    T* __restrict__ out, float* __restrict__ residual, const float* __restrict__ w, int H, float eps,
    const T* __restrict__ y, const T* __restrict__ ye, const int* __restrict__ pair_slot, const int* __restrict__ ids,
    const float* __restrict__ wts, int top, int E, const T* __restrict__ h, const T* __restrict__ shared) {
  extern __shared__ float sm[];  // [H] the addend
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  float sq = 0.f;
  float wsum_id = 0.f;  // weight of the token's identity experts
  if (y == nullptr)
    for (int j = 0; j < top; ++j)
      if (ids[t * top + j] >= E) wsum_id += wts[t * top + j];
  for (int e = tid; e < H; e += kNT) {
    float v;
    if (y != nullptr) {
      v = ldf<T>(y, t * H + e);
    } else {
      v = shared != nullptr ? ldf<T>(shared, t * H + e) : 0.f;
      for (int j = 0; j < top; ++j)
        if (ids[t * top + j] < E) v = __builtin_fmaf(wts[t * top + j], ldf<T>(ye, (long)pair_slot[t * top + j] * H + e), v);
      if (wsum_id != 0.f) v = __builtin_fmaf(wsum_id, ldf<T>(h, t * H + e), v);
    }
    sm[e] = v;
    sq += v * v;
  }
  sq = block_sum(sq, red);
  const float inv = 1.f / sqrtf(sq / (float)H + eps);
  float* r = residual + t * H;
  for (int e = tid; e < H; e += kNT) {
    const float v = r[e] + sm[e] * inv * w[e];
    r[e] = v;
    stf<T>(out, t * H + e, v);
  }
}

}  // namespace

void launch_add_normed(void* out, float* residual, const float* w, int T, int H, float eps, const void* y,
                       const void* ye, const int* pair_slot, const int* ids, const float* wts, int top, int E,
                       const void* h, const void* shared, bool f32, hipStream_t s) {
  if (T <= 0) return;
  const size_t smem = (size_t)H * sizeof(float);
  if (f32)
    add_normed_kernel<float><<<T, kNT, smem, s>>>((float*)out, residual, w, H, eps, (const float*)y, (const float*)ye,
                                                  pair_slot, ids, wts, top, E, (const float*)h, (const float*)shared);
  else
    add_normed_kernel<unsigned short><<<T, kNT, smem, s>>>(
        (unsigned short*)out, residual, w, H, eps, (const unsigned short*)y, (const unsigned short*)ye, pair_slot, ids,
        wts, top, E, (const unsigned short*)h, (const unsigned short*)shared);
}

void launch_scaled_add_group_rmsnorm(void* out, float* residual, const float* w, int T, int H, int groups, float eps,
                                     const void* mix, const float* ls1, const void* y, const int* pair_slot, int top,
                                     const float* ls2, const void* extra, bool f32, hipStream_t s) {
  if (T <= 0) return;
  const size_t smem = (size_t)(H + groups) * sizeof(float);
  if (f32)
    scaled_add_group_rmsnorm_kernel<float><<<T, kNT, smem, s>>>(
        (float*)out, residual, w, H, groups, eps, (const float*)mix, ls1, (const float*)y, pair_slot, top, ls2,
        (const float*)extra);
  else
    scaled_add_group_rmsnorm_kernel<unsigned short><<<T, kNT, smem, s>>>(
        (unsigned short*)out, residual, w, H, groups, eps, (const unsigned short*)mix, ls1, (const unsigned short*)y,
        pair_slot, top, ls2, (const unsigned short*)extra);
}

}  // namespace hipserve
