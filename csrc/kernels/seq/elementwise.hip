// Elementwise and per-row activations of the layer-list decoders' feed-forwards and output gates
// (bf16 or fp32 rows, fp32 arithmetic):
//   activation  tanh, xIELU, squared ReLU, SiLU gate ([gate | up] rows)
//   polynorm    a N(z) + b N(z^2) + c N(z^3) + e per row, N(u) = u / sqrt(mean(u^2) + eps): one workgroup
//               per row keeps its elements in registers between the three sums of powers and the output
//   gate_mul    out[t, h * d + j] = x[h, t, j] * sigmoid(gate[t, h * d + j]): the heads of a head-major
//               batched product side by side per token, each element gated, in one pass
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void activation_kernel(T* __restrict__ out, long out_ld, const T* __restrict__ x,
                                                         long x_ld, int cols, int kind, float c0, float c1) {
  const long t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= cols) return;
  const float z = ldf<T>(x, t * x_ld + c);
  float r;
  if (kind == 0) r = tanhf(z);
  else if (kind == 2) { r = fmaxf(z, 0.f); r *= r; }
  else if (kind == 3) r = z * sigmoid_f(z) * ldf<T>(x, t * x_ld + cols + c);   // x rows = [gate | up]
  else r = z > 0.f ? c0 * z * z + 0.5f * z : c1 * (expm1f(z) - z) + 0.5f * z;
  stf<T>(out, t * out_ld + c, r);
}

// bf16 rows whose length, strides and base addresses are multiples of 8 elements: 8 elements per thread.
__global__ __launch_bounds__(256) void activation_vec_kernel(unsigned short* __restrict__ out, long out_ld,
                                                             const unsigned short* __restrict__ x, long x_ld,
                                                             int cols8, int kind, float c0, float c1) {
  const long t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= cols8) return;
  const u16x8 z8 = *reinterpret_cast<const u16x8*>(x + t * x_ld + 8 * c);
  u16x8 u8 = z8;
  if (kind == 3) u8 = *reinterpret_cast<const u16x8*>(x + t * x_ld + 8 * (cols8 + c));
  u16x8 r8;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float z = bf16_to_f32(z8[e]);
    float r;
    if (kind == 0) r = tanhf(z);
    else if (kind == 2) { r = fmaxf(z, 0.f); r *= r; }
    else if (kind == 3) r = z * sigmoid_f(z) * bf16_to_f32(u8[e]);
    else r = z > 0.f ? c0 * z * z + 0.5f * z : c1 * (expm1f(z) - z) + 0.5f * z;
    r8[e] = f32_to_bf16(r);
  }
  *reinterpret_cast<u16x8*>(out + t * out_ld + 8 * c) = r8;
}

constexpr int kPolyPer = 16;  // elements per thread held in registers (rows up to 256 * 16 = 4096 wide)

// REG: the row fits the registers of one workgroup (cols <= 256 * kPolyPer); else the row is read twice.
template <typename T, bool REG>
__global__ __launch_bounds__(256) void polynorm_kernel(T* __restrict__ out, long out_ld, const T* __restrict__ x,
                                                       long x_ld, int cols, const float* __restrict__ coef,
                                                       float eps) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  const T* row = x + t * x_ld;
  float z[REG ? kPolyPer : 1];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  if constexpr (REG) {
#pragma unroll
    for (int i = 0; i < kPolyPer; ++i) {
      const int c = tid + 256 * i;
      z[i] = c < cols ? ldf<T>(row, c) : 0.f;
      const float q = z[i] * z[i];
      s2 += q; s4 += q * q; s6 += q * q * q;
    }
  } else {
    for (int c = tid; c < cols; c += 256) {
      const float v = ldf<T>(row, c), q = v * v;
      s2 += q; s4 += q * q; s6 += q * q * q;
    }
  }
  s2 = block_sum(s2, red);
  s4 = block_sum(s4, red);
  s6 = block_sum(s6, red);
  const float n = (float)cols;
  const float a = coef[0] / sqrtf(s2 / n + eps), b = coef[1] / sqrtf(s4 / n + eps), c3 = coef[2] / sqrtf(s6 / n + eps);
  const float e = coef[3];
  if constexpr (REG) {
#pragma unroll
    for (int i = 0; i < kPolyPer; ++i) {
      const int c = tid + 256 * i;
      if (c < cols) stf<T>(out, t * out_ld + c, ((c3 * z[i] + b) * z[i] + a) * z[i] + e);
    }
  } else {
    for (int c = tid; c < cols; c += 256) {
      const float v = ldf<T>(row, c);
      stf<T>(out, t * out_ld + c, ((c3 * v + b) * v + a) * v + e);
    }
  }
}

// bf16 rows whose length, strides and base addresses are multiples of 8 elements: NV 16-byte vectors per thread
// (rows up to 2048 NV wide), read once.
template <int NV>
__global__ __launch_bounds__(256) void polynorm_vec_kernel(unsigned short* __restrict__ out, long out_ld,
                                                           const unsigned short* __restrict__ x, long x_ld, int cols,
                                                           const float* __restrict__ coef, float eps) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  u16x8 z[NV];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = 8 * (tid + 256 * i);
    z[i] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (c < cols) z[i] = *reinterpret_cast<const u16x8*>(x + t * x_ld + c);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = bf16_to_f32(z[i][e]), q = v * v;
      s2 += q; s4 += q * q; s6 += q * q * q;
    }
  }
  s2 = block_sum(s2, red);
  s4 = block_sum(s4, red);
  s6 = block_sum(s6, red);
  const float n = (float)cols;
  const float a = coef[0] / sqrtf(s2 / n + eps), b = coef[1] / sqrtf(s4 / n + eps), c3 = coef[2] / sqrtf(s6 / n + eps);
  const float e0 = coef[3];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = 8 * (tid + 256 * i);
    if (c >= cols) continue;
    u16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = bf16_to_f32(z[i][e]);
      r[e] = f32_to_bf16(((c3 * v + b) * v + a) * v + e0);
    }
    *reinterpret_cast<u16x8*>(out + t * out_ld + c) = r;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gate_mul_kernel(T* __restrict__ out, const T* __restrict__ x,
                                                       const T* __restrict__ gate, long gate_ld, int T_rows, int d,
                                                       int cols) {
  const long t = blockIdx.x;
  for (int c = threadIdx.x; c < cols; c += 256) {
    const int h = c / d, j = c - h * d;
    const float v = ldf<T>(x, ((long)h * T_rows + t) * d + j);
    stf<T>(out, t * cols + c, v * sigmoid_f(ldf<T>(gate, t * gate_ld + c)));
  }
}

}  // namespace

void launch_activation(void* out, long out_ld, const void* x, long x_ld, int rows, int cols, int kind, float c0,
                       float c1, bool f32, hipStream_t s) {
  if (rows <= 0 || cols <= 0) return;
  dim3 grid(rows, (cols + 255) / 256);
  if (f32) activation_kernel<float><<<grid, 256, 0, s>>>((float*)out, out_ld, (const float*)x, x_ld, cols, kind, c0, c1);
  else if (cols % 8 == 0 && out_ld % 8 == 0 && x_ld % 8 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)x % 16 == 0)
    activation_vec_kernel<<<dim3(rows, (cols / 8 + 255) / 256), 256, 0, s>>>(
        (unsigned short*)out, out_ld, (const unsigned short*)x, x_ld, cols / 8, kind, c0, c1);
  else
    activation_kernel<unsigned short><<<grid, 256, 0, s>>>((unsigned short*)out, out_ld, (const unsigned short*)x, x_ld,
                                                           cols, kind, c0, c1);
}

void launch_polynorm(void* out, long out_ld, const void* x, long x_ld, int rows, int cols, const float* coef,
                     float eps, bool f32, hipStream_t s) {
  if (rows <= 0 || cols <= 0) return;
  if (!f32 && cols % 8 == 0 && out_ld % 8 == 0 && x_ld % 8 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)x % 16 == 0 &&
      cols <= 2048 * 4) {
    auto o = (unsigned short*)out;
    auto in = (const unsigned short*)x;
    if (cols <= 2048) polynorm_vec_kernel<1><<<rows, 256, 0, s>>>(o, out_ld, in, x_ld, cols, coef, eps);
    else if (cols <= 4096) polynorm_vec_kernel<2><<<rows, 256, 0, s>>>(o, out_ld, in, x_ld, cols, coef, eps);
    else polynorm_vec_kernel<4><<<rows, 256, 0, s>>>(o, out_ld, in, x_ld, cols, coef, eps);
    return;
  }
  const bool reg = cols <= 256 * kPolyPer;
#define HS_PN(T, R) polynorm_kernel<T, R><<<rows, 256, 0, s>>>((T*)out, out_ld, (const T*)x, x_ld, cols, coef, eps)
  if (f32) { if (reg) HS_PN(float, true); else HS_PN(float, false); }
  else { if (reg) HS_PN(unsigned short, true); else HS_PN(unsigned short, false); }
#undef HS_PN
}

void launch_gate_mul(void* out, const void* x, const void* gate, long gate_ld, int rows, int heads, int d, bool f32,
                     hipStream_t s) {
  if (rows <= 0) return;
  if (f32)
    gate_mul_kernel<float><<<rows, 256, 0, s>>>((float*)out, (const float*)x, (const float*)gate, gate_ld, rows, d, heads * d);
  else
    gate_mul_kernel<unsigned short><<<rows, 256, 0, s>>>((unsigned short*)out, (const unsigned short*)x,
                                                         (const unsigned short*)gate, gate_ld, rows, d, heads * d);
}

}  // namespace hipserve
