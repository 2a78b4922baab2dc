// Expert GEMMs of the mixtures of experts over moe_align tiles: out[slot, :] = act(W[e] . x[row(slot)])
// where a tile is `tile` consecutive expert-sorted slots of one expert (tile_expert[t]; -1 = unused, and a
// value >= E, a bucket of pairs whose expert has no weights, is skipped too),
// row(slot) = slots[slot] / gather_k (the token row of the pair; first GEMM) or the slot itself
// (second GEMM) and act = none (0), squared ReLU (1) or a SiLU gate (2): W[e] = [gate rows; up rows], N / 2 each,
// and out[slot, c] = silu(gate_c . x) * (up_c . x) has N / 2 columns (a thread / lane holds a column's pair). Any N and K: edges are bounds-checked. A workgroup
// computes a [32 slots x 64 columns] block, x and W staged through LDS in K-chunks of 32, fp32
// accumulation; bf16 and fp32 element types.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kTM = 32, kTN = 64, kTK = 32;

template <typename T>
__global__ __launch_bounds__(256) void expert_gemm_kernel(T* __restrict__ out, const T* __restrict__ x, long x_ld,
                                                          const T* __restrict__ w, const int* __restrict__ slots,
                                                          const int* __restrict__ tile_expert, int tile, int gather_k,
                                                          int N, int K, int act, int E) {
  __shared__ float xs[kTM][kTK + 1], ws[kTN][kTK + 1];
  __shared__ long xrow[kTM];
  const int e = tile_expert[(blockIdx.y * kTM) / tile];
  if (e < 0 || e >= E) return;
  const int tid = threadIdx.x;
  const bool glu = act == 2;
  const int No = glu ? N / 2 : N;   // output columns
  // gated: the block's 64 weight rows are 32 gate rows and the 32 up rows of the same output columns
  const int slot0 = blockIdx.y * kTM, n0 = blockIdx.x * (glu ? kTN / 2 : kTN);
  if (tid < kTM) {
    const int p = slots[slot0 + tid];
    xrow[tid] = p < 0 ? -1 : (gather_k > 0 ? (long)(p / gather_k) : (long)(slot0 + tid)) * x_ld;
  }
  const T* we = w + (long)e * N * K;
  const int tx = tid & 15, ty = tid >> 4;  // 4 columns x 2 slots per thread
  float acc[2][4] = {};
  for (int k0 = 0; k0 < K; k0 += kTK) {
    __syncthreads();
    for (int idx = tid; idx < kTM * kTK; idx += 256) {
      const int r = idx / kTK, k = idx % kTK;
      const long xr = xrow[r];
      xs[r][k] = (xr >= 0 && k0 + k < K) ? ldf<T>(x, xr + k0 + k) : 0.f;
    }
    for (int idx = tid; idx < kTN * kTK; idx += 256) {
      const int c = idx / kTK, k = idx % kTK;
      const int col = glu ? n0 + (c & 31) : n0 + c;              // output column
      const long wrow = glu && c >= 32 ? (long)No + col : col;   // its weight row (the up row for c >= 32)
      ws[c][k] = (col < No && k0 + k < K) ? ldf<T>(we, wrow * K + k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < kTK; ++k) {
      const float a0 = xs[ty * 2][k], a1 = xs[ty * 2 + 1][k];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b = ws[tx + 16 * j][k];
        acc[0][j] = __builtin_fmaf(a0, b, acc[0][j]);
        acc[1][j] = __builtin_fmaf(a1, b, acc[1][j]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = ty * 2 + i;
    if (xrow[r] < 0) continue;
    if (glu) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {   // columns tx, tx + 16: gates in acc[.][j], ups in acc[.][j + 2]
        const int c = n0 + tx + 16 * j;
        if (c < No) stf<T>(out, (long)(slot0 + r) * No + c, acc[i][j] * sigmoid_f(acc[i][j]) * acc[i][j + 2]);
      }
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + tx + 16 * j;
      if (c >= N) continue;
      float v = acc[i][j];
      if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
      stf<T>(out, (long)(slot0 + r) * N + c, v);
    }
  }
}

// bf16 on the matrix cores: a workgroup (4 waves) computes [16 ST slots x 128 columns]; wave w owns
// columns 32 w .. 32 w + 31. Operands go from global memory straight into the MFMA registers (16 bytes
// per lane and step: 8 consecutive k of one W row / one x row); W rows are read once per slot tile, the
// x rows of the tile are shared by the four waves through L1. Needs K % 8 == 0, N % 8 == 0.
template <int ST>
__global__ __launch_bounds__(256) void expert_gemm_mfma_kernel(
    unsigned short* __restrict__ out, const unsigned short* __restrict__ x, long x_ld,
    const unsigned short* __restrict__ w, const int* __restrict__ slots, const int* __restrict__ tile_expert,
    int gather_k, int N, int K, int act, int E) {
  const int e = tile_expert[blockIdx.y];
  if (e < 0 || e >= E) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int slot0 = blockIdx.y * 16 * ST;
  const bool glu = act == 2;
  const int No = glu ? N / 2 : N;
  // gated: the wave's two 16-column tiles are the gate rows and the up rows of the SAME 16 output columns
  const int n0 = glu ? blockIdx.x * 64 + 16 * wave : blockIdx.x * 128 + 32 * wave;
  if (n0 >= No) return;
  const unsigned short* xr[ST];
  bool live[ST];
#pragma unroll
  for (int st = 0; st < ST; ++st) {
    const int slot = slot0 + 16 * st + c;
    const int p = slots[slot];
    live[st] = p >= 0;
    xr[st] = x + (p < 0 ? 0 : (gather_k > 0 ? (long)(p / gather_k) : (long)slot)) * x_ld + 8 * g;
  }
  const unsigned short* wr[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
    wr[nt] = w + ((long)e * N + (glu ? nt * No + min(n0 + c, No - 1) : min(n0 + 16 * nt + c, N - 1))) * K + 8 * g;
  f32x4 acc[2][ST];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int st = 0; st < ST; ++st) acc[nt][st] = f32x4{0.f, 0.f, 0.f, 0.f};
  const u16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int kU = 4;  // k steps whose operand loads are in flight together
  for (int k0 = 0; k0 < K; k0 += 32 * kU) {
    u16x8 a[kU][2], b[kU][ST];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int k = k0 + 32 * u;
      const bool in = k + 8 * g < K;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) a[u][nt] = in ? *reinterpret_cast<const u16x8*>(wr[nt] + k) : zero;
#pragma unroll
      for (int st = 0; st < ST; ++st) b[u][st] = (in && live[st]) ? *reinterpret_cast<const u16x8*>(xr[st] + k) : zero;
    }
#pragma unroll
    for (int u = 0; u < kU; ++u)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int st = 0; st < ST; ++st)
          acc[nt][st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[u][nt]),
                                                                __builtin_bit_cast(bf16x8, b[u][st]), acc[nt][st], 0, 0, 0);
  }
  // lane (c, g): columns n0 + 16 nt + 4 g .. + 3 of slot 16 st + c
#pragma unroll
  for (int st = 0; st < ST; ++st) {
    if (!live[st]) continue;
    const long slot = slot0 + 16 * st + c;
    if (glu) {
      const int n = n0 + 4 * g;
      if (n >= No) continue;  // No % 4 == 0: the four columns are inside together
      u16x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = f32_to_bf16(acc[0][st][j] * sigmoid_f(acc[0][st][j]) * acc[1][st][j]);
      *reinterpret_cast<u16x4*>(out + slot * No + n) = o;
      continue;
    }
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int n = n0 + 16 * nt + 4 * g;
      if (n >= N) continue;  // N % 8 == 0: the four columns are inside together
      u16x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float v = acc[nt][st][j];
        if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
        o[j] = f32_to_bf16(v);
      }
      *reinterpret_cast<u16x4*>(out + slot * N + n) = o;
    }
  }
}

}  // namespace

void launch_expert_gemm(void* out, const void* x, long x_ld, const void* w, const int* slots, const int* tile_expert,
                        int ntiles_cap, int tile, int gather_k, int N, int K, int act, int E, bool f32, hipStream_t s) {
  if (ntiles_cap <= 0) return;
  const int No = act == 2 ? N / 2 : N;
  if (!f32 && K % 8 == 0 && No % 8 == 0 && x_ld % 8 == 0 && (tile == 32 || tile == 64)) {
    dim3 mg(act == 2 ? (No + 63) / 64 : (N + 127) / 128, ntiles_cap);
    auto o = (unsigned short*)out;
    auto xi = (const unsigned short*)x, wi = (const unsigned short*)w;
    if (tile == 32) expert_gemm_mfma_kernel<2><<<mg, 256, 0, s>>>(o, xi, x_ld, wi, slots, tile_expert, gather_k, N, K, act, E);
    else expert_gemm_mfma_kernel<4><<<mg, 256, 0, s>>>(o, xi, x_ld, wi, slots, tile_expert, gather_k, N, K, act, E);
    return;
  }
  dim3 grid(act == 2 ? (No + kTN / 2 - 1) / (kTN / 2) : (N + kTN - 1) / kTN, (long)ntiles_cap * tile / kTM);
  if (f32)
    expert_gemm_kernel<float><<<grid, 256, 0, s>>>((float*)out, (const float*)x, x_ld, (const float*)w, slots,
                                                   tile_expert, tile, gather_k, N, K, act, E);
  else
    expert_gemm_kernel<unsigned short><<<grid, 256, 0, s>>>((unsigned short*)out, (const unsigned short*)x, x_ld,
                                                            (const unsigned short*)w, slots, tile_expert, tile,
                                                            gather_k, N, K, act, E);
}

}  // namespace hipserve
