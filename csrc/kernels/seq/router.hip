// Softmax router with a selection correction: per token, s = softmax(logits) over all n router
// outputs (fp32); the `top` outputs with the largest s + correction are chosen (ties: the lower
// index); wts = s * scale of the chosen ones, ids = their index, where every index >= E (an
// expert without weights) is written as E, so the expert alignment sees them as one bucket that
// no GEMM tile serves. One wave per token, output e on lane e % 64, slot e / 64 (n <= 256).
// groups > 1 (at most 64): the outputs form equal groups of neighbours; a group scores the largest
// corrected score in it (group g's on lane g), and the outputs outside the `keep` best groups (ties:
// the lower group) cannot be chosen. renorm: the chosen scores are divided by their sum + 1e-20.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kSlots = 4;

__global__ __launch_bounds__(256) void route_topk_kernel(int* __restrict__ ids, float* __restrict__ wts,
                                                         const float* __restrict__ logits,
                                                         const float* __restrict__ correction, int T, int n, int top,
                                                         float scale, int E, int groups, int keep, bool renorm) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= T) return;
  float p[kSlots], c[kSlots];
  float mx = -INFINITY;
#pragma unroll
  for (int s = 0; s < kSlots; ++s) {
    const int e = lane + 64 * s;
    p[s] = e < n ? logits[(long)t * n + e] : -INFINITY;
    mx = fmaxf(mx, p[s]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int s = 0; s < kSlots; ++s) {
    p[s] = lane + 64 * s < n ? expf(p[s] - mx) : 0.f;
    sum += p[s];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int s = 0; s < kSlots; ++s) {
    const int e = lane + 64 * s;
    p[s] = p[s] / sum;
    c[s] = e < n ? p[s] + correction[e] : -INFINITY;
  }
  if (groups > 1) {
    const int per = n / groups;
    float gbest = -INFINITY;   // lane g: group g's score
    for (int g = 0; g < groups; ++g) {
      float v = -INFINITY;
#pragma unroll
      for (int s = 0; s < kSlots; ++s)
        if ((lane + 64 * s) / per == g) v = fmaxf(v, c[s]);
      v = wave_max(v);
      if (lane == g) gbest = v;
    }
    unsigned long long allowed = 0;
    for (int j = 0; j < keep; ++j) {
      const float best = wave_max(gbest);
      const unsigned long long b = __ballot(gbest == best && lane < groups);
      if (!b) break;
      const int who = __builtin_ctzll(b);
      allowed |= 1ull << who;
      if (lane == who) gbest = -INFINITY;
    }
#pragma unroll
    for (int s = 0; s < kSlots; ++s) {
      const int e = lane + 64 * s;
      if (e < n && !((allowed >> (e / per)) & 1ull)) c[s] = -INFINITY;
    }
  }
  int mine[kSlots];
#pragma unroll
  for (int s = 0; s < kSlots; ++s) mine[s] = -1;
  float chosen = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
#pragma unroll
    for (int s = 0; s < kSlots; ++s) best = fmaxf(best, c[s]);
    best = wave_max(best);
    // the lowest index holding the best value: slot 0 holds outputs 0..63, slot 1 the next 64, ...
    int who = -1;
#pragma unroll
    for (int s = 0; s < kSlots; ++s) {
      const unsigned long long b = __ballot(c[s] == best);
      if (who < 0 && b) who = 64 * s + __builtin_ctzll(b);
    }
#pragma unroll
    for (int s = 0; s < kSlots; ++s) {
      if (who == lane + 64 * s) {
        ids[(long)t * top + j] = min(who, E);
        mine[s] = j;
        chosen += p[s];
        c[s] = -INFINITY;
      }
    }
  }
  const float f = renorm ? scale / (wave_sum(chosen) + 1e-20f) : scale;
#pragma unroll
  for (int s = 0; s < kSlots; ++s)
    if (mine[s] >= 0) wts[(long)t * top + mine[s]] = p[s] * f;
}

}  // namespace

int route_topk_max_outputs() { return 64 * kSlots; }

void launch_route_topk(int* ids, float* wts, const float* logits, const float* correction, int T, int n, int top,
                       float scale, int E, int groups, int keep, bool renorm, hipStream_t s) {
  if (T <= 0) return;
  route_topk_kernel<<<(T + 3) / 4, 256, 0, s>>>(ids, wts, logits, correction, T, n, top, scale, E, groups, keep, renorm);
}

}  // namespace hipserve
