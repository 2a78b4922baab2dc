// mLSTM matrix memory over per-sequence state slots: per head a state S [dim, vdim], a normaliser
// n [dim] and the running maximum m of the log gates, all fp32.
//   i = cap tanh((gi + bi) / cap),  f = logsigmoid(cap tanh((gf + bf) / cap))      (log gates, per head and token)
//   m' = max(f + m, i);  a = exp(f + m - m'),  b = exp(i - m')
//   S <- a S + b k v^T;  n <- a n + b k;  m <- m'
//   o = S^T q / (max(|n . q|, exp(-m)) + 1e-6),  q scaled by dim^-1/2
//   out = o / sqrt(mean_head(o^2) + eps) * w * sigmoid(gate)
// A step that starts at position 0 starts from S = 0, n = 0, m = 0.
//
// Prompt portions run four kernels:
//   mlstm_stage  one workgroup per token: q (scaled), k and v of every head as dense fp32 rows, the value row one
//                element longer with a 1 at its end (the normaliser's value), so the scan stages everything with
//                contiguous 4-byte loads whatever the element type and the row stride of the projection
//   mlstm_gates  one wave per (sequence, head): the gates of 64 tokens at a time and the running maximum by a
//                wave scan in the (max, +) semiring (m' = max(m + F, I) composes as F = F1 + F2,
//                I = max(I1 + F2, I2)); writes a, b and exp(-m) per token and the last m into the slot.
//                Whatever rounding the scan leaves in m cancels: a and b are formed from the SAME m values the
//                state is scaled by, so S and n stay exp(-m) times the unscaled sums.
//   mlstm_scan   the recurrence, laid out as the delta-rule scans: a state column (all key channels of one value
//                channel) in the registers of the 16 lanes of a DPP row, tokens staged through LDS eight at a
//                time and loaded one batch ahead. The normaliser is one more column whose value is 1, so
//                n . q falls out as that column's read-out.
//   mlstm_out    one wave per (token, head): the division, the head's RMS norm, weight and sigmoid gate.
// Steps in which every sequence brings one row (decoding) run mlstm_step: everything above for one
// (sequence, head) in one workgroup, thread v owning state column v, so the state is read and written once,
// coalesced.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

HS_DEVICE float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// scr[t, h] = (a, b, exp(-m), 0)
__global__ __launch_bounds__(64) void mlstm_gates_kernel(f32x4* __restrict__ scr, float* __restrict__ M,
                                                        const float* __restrict__ gates,
                                                        const float* __restrict__ b_if, const int* __restrict__ seq_cu,
                                                        const int* __restrict__ seq_ctx,
                                                        const int* __restrict__ seq_state, int heads, float cap) {
  const int s = blockIdx.y, h = blockIdx.x, lane = threadIdx.x;
  const int r0 = seq_cu[s], n = seq_cu[s + 1] - r0;
  if (n <= 0) return;
  float* mp = M + (long)seq_state[s] * heads + h;
  float carry = seq_ctx[s] - n > 0 ? *mp : 0.f;
  const float bi = b_if[h], bf = b_if[heads + h], icap = 1.f / cap;
  for (int t0 = 0; t0 < n; t0 += 64) {
    const int t = t0 + lane;
    const bool in = t < n;
    const float* g = gates + (long)(r0 + (in ? t : 0)) * 2 * heads;
    const float ig = cap * tanhf((g[h] + bi) * icap);
    const float fg = log_sigmoid(cap * tanhf((g[heads + h] + bf) * icap));
    float F = in ? fg : 0.f, I = in ? ig : -INFINITY;   // past the end: the identity of the composition
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float Fp = __shfl_up(F, off, 64), Ip = __shfl_up(I, off, 64);
      if (lane >= off) {
        I = fmaxf(Ip + F, I);
        F = Fp + F;
      }
    }
    const float m = fmaxf(carry + F, I);
    float mprev = __shfl_up(m, 1, 64);
    if (lane == 0) mprev = carry;
    if (in) scr[(long)(r0 + t) * heads + h] = f32x4{expf(fg + mprev - m), expf(ig - m), expf(-m), 0.f};
    carry = __shfl(m, min(63, n - t0 - 1), 64);
  }
  if (lane == 0) *mp = carry;
}

// qk[t, h] = [q * qscale (dim) | k (dim)], vv[t, h] = [v (vdim) | 1]
template <typename T>
__global__ __launch_bounds__(256) void mlstm_stage_kernel(float* __restrict__ qk, float* __restrict__ vv,
                                                         const T* __restrict__ proj, long ld, int heads, int dim,
                                                         int vdim, float qscale) {
  const long t = blockIdx.x;
  const T* row = proj + t * ld;
  const int nqk = heads * dim, nv = heads * vdim;
  for (int e = threadIdx.x; e < nqk; e += 256) {
    const int h = e / dim, i = e - h * dim;
    float* dst = qk + (t * heads + h) * 2 * dim;
    dst[i] = ldf<T>(row, e) * qscale;
    dst[dim + i] = ldf<T>(row, nqk + e);
  }
  for (int e = threadIdx.x; e < nv + heads; e += 256) {
    if (e < nv) {
      const int h = e / vdim, c = e - h * vdim;
      vv[(t * heads + h) * (vdim + 1) + c] = ldf<T>(row, 2L * nqk + e);
    } else {
      vv[(t * heads + (e - nv)) * (vdim + 1) + vdim] = 1.f;
    }
  }
}

constexpr int kTB = 8;     // tokens staged at a time
constexpr int kSeg = 16;   // lanes that share a state column (one DPP row)
constexpr int kScanThreads = 256;
constexpr int kCols = kScanThreads / kSeg;  // state columns per workgroup

HS_DEVICE float row_sum(float v) {
  v = dpp_step<0xB1, 0xf, false>(v);   // quad_perm [1, 0, 3, 2]
  v = dpp_step<0x4E, 0xf, false>(v);   // quad_perm [2, 3, 0, 1]
  v = dpp_step<0x141, 0xf, false>(v);  // row_half_mirror
  return dpp_step<0x140, 0xf, false>(v);  // row_mirror
}

// grid (heads, ceil((vdim + 1) / kCols), sequences). Column c < vdim is S[:, c]; column vdim is the normaliser.
// o [T, heads, vdim + 1]: the unnormalised read-outs, the last one n . q.
template <int DS>
__global__ __launch_bounds__(kScanThreads) void mlstm_scan_kernel(
    float* __restrict__ o, float* __restrict__ S, float* __restrict__ N, const float* __restrict__ qk,
    const float* __restrict__ vv, const f32x4* __restrict__ scr, const int* __restrict__ seq_cu,
    const int* __restrict__ seq_ctx, const int* __restrict__ seq_state, int heads, int dim, int vdim) {
  constexpr int DP = kSeg * DS;
  __shared__ __attribute__((aligned(16))) float sq[kTB][DP], sk[kTB][DP];
  __shared__ float sab[kTB][2];
  const int s = blockIdx.z, h = blockIdx.x, zb = blockIdx.y, tid = threadIdx.x;
  const int r0 = seq_cu[s], n = seq_cu[s + 1] - r0;
  if (n <= 0) return;
  const int seg = tid & (kSeg - 1), k0 = seg * DS;
  const int c = zb * kCols + tid / kSeg;   // this lane row's column
  const bool is_s = c < vdim, is_n = c == vdim;
  const long slot = seq_state[s];
  float* Sp = S + ((slot * heads + h) * dim) * vdim;
  float* Np = N + (slot * heads + h) * dim;
  const bool carried = seq_ctx[s] - n > 0;
  float st[DS];
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    st[i] = 0.f;
    if (carried && k0 + i < dim) {
      if (is_s) st[i] = Sp[(long)(k0 + i) * vdim + c];
      else if (is_n) st[i] = Np[k0 + i];
    }
  }
  const int ow = vdim + 1;
  const bool has_col = c <= vdim;
  constexpr int kLd = (kTB * DP + kScanThreads - 1) / kScanThreads;
  float rq[kLd], rk[kLd], rv[kTB], rab = 0.f;
  auto fetch = [&](int t0) {
    const int nt = min(kTB, n - t0);
#pragma unroll
    for (int it = 0; it < kLd; ++it) {
      const int i = it * kScanThreads + tid;
      const int tt = i / DP, k = i % DP;
      const float* row = qk + ((long)(r0 + t0 + tt) * heads + h) * 2 * dim;
      const bool in = tt < nt && k < dim;
      rq[it] = in ? row[k] : 0.f;
      rk[it] = in ? row[dim + k] : 0.f;
    }
    if (tid < 2 * nt) {
      const f32x4 g = scr[(long)(r0 + t0 + (tid >> 1)) * heads + h];
      rab = (tid & 1) ? g[1] : g[0];
    }
#pragma unroll
    for (int tt = 0; tt < kTB; ++tt)
      rv[tt] = (tt < nt && has_col) ? vv[((long)(r0 + t0 + tt) * heads + h) * ow + c] : 0.f;
  };
  float* po = o + ((long)r0 * heads + h) * ow + c;
  fetch(0);
  for (int t0 = 0; t0 < n; t0 += kTB) {
    const int nt = min(kTB, n - t0);
    __syncthreads();
#pragma unroll
    for (int it = 0; it < kLd; ++it) {
      const int i = it * kScanThreads + tid;
      if (i < kTB * DP) {
        sq[i / DP][i % DP] = rq[it];
        sk[i / DP][i % DP] = rk[it];
      }
    }
    if (tid < 2 * kTB) sab[tid >> 1][tid & 1] = rab;
    float val[kTB];
#pragma unroll
    for (int tt = 0; tt < kTB; ++tt) val[tt] = rv[tt];
    __syncthreads();
    if (t0 + kTB < n) fetch(t0 + kTB);
#pragma unroll
    for (int tt = 0; tt < kTB; ++tt) {
      if (tt < nt) {
        const float a = sab[tt][0], bv = sab[tt][1] * val[tt];
        float out = 0.f, out2 = 0.f;
#pragma unroll
        for (int i = 0; i < DS; ++i) {
          st[i] = __builtin_fmaf(a, st[i], bv * sk[tt][k0 + i]);
          if (i & 1) out2 = __builtin_fmaf(st[i], sq[tt][k0 + i], out2);
          else out = __builtin_fmaf(st[i], sq[tt][k0 + i], out);
        }
        const float r = row_sum(out + out2);
        if (seg == 0 && c <= vdim) po[(long)(t0 + tt) * heads * ow] = r;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < DS; ++i)
    if (k0 + i < dim) {
      if (is_s) Sp[(long)(k0 + i) * vdim + c] = st[i];
      else if (is_n) Np[k0 + i] = st[i];
    }
}

// One wave per (token, head): out = (o / den) / rms * w * sigmoid(gate), den = max(|n . q|, exp(-m)) + 1e-6.
template <typename T>
__global__ __launch_bounds__(256) void mlstm_out_kernel(T* __restrict__ out, const float* __restrict__ o,
                                                        const f32x4* __restrict__ scr, const T* __restrict__ proj,
                                                        long ld, int gate_off, const float* __restrict__ w, int rows,
                                                        int heads, int vdim, float eps) {
  const long idx = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (idx >= (long)rows * heads) return;
  const long t = idx / heads;
  const int h = idx % heads;
  const float* src = o + idx * (vdim + 1);
  const float iden = 1.f / (fmaxf(fabsf(src[vdim]), scr[idx][2]) + 1e-6f);
  float a = 0.f;
  for (int e = lane; e < vdim; e += 64) { const float x = src[e] * iden; a += x * x; }
  const float inv = iden / sqrtf(wave_sum(a) / (float)vdim + eps);
  const T* gate = proj + t * ld + gate_off + (long)h * vdim;
  for (int e = lane; e < vdim; e += 64)
    stf<T>(out, (t * heads + h) * vdim + e, src[e] * inv * w[h * vdim + e] * sigmoid_f(ldf<T>(gate, e)));
}

constexpr int kStepCols = 4;   // state columns per thread of the one-row kernel (vdim <= 4 * 256)

// grid (heads, sequences), 256 G threads (G = 1, 2 or 4 row groups); sequence s brings the one row seq_cu[s].
// Thread (g, c) walks its quarter of the key channels of state column c (+ 256 per pass), eight rows' loads in
// flight before their updates are stored; the groups' partial read-outs meet in LDS. Dynamic LDS: q, k [dim]
// each, then (G - 1) x 256 partial sums.
template <typename T>
__global__ __launch_bounds__(1024) void mlstm_step_kernel(
    T* __restrict__ out, float* __restrict__ S, float* __restrict__ N, float* __restrict__ M,
    const T* __restrict__ proj, long ld, const float* __restrict__ gates, const float* __restrict__ b_if,
    const float* __restrict__ w, const int* __restrict__ seq_cu, const int* __restrict__ seq_ctx,
    const int* __restrict__ seq_state, int heads, int dim, int vdim, float cap, float qscale, float eps) {
  extern __shared__ float sm[];
  __shared__ float red[16];
  float* sq = sm;
  float* sk = sm + dim;
  float* part = sm + 2 * dim;
  const int s = blockIdx.y, h = blockIdx.x, tid = threadIdx.x;
  const int G = blockDim.x >> 8, g = tid >> 8, c0 = tid & 255;
  const long t = seq_cu[s];
  if (seq_cu[s + 1] - t <= 0) return;
  const bool carried = seq_ctx[s] - 1 > 0;
  const long slot = seq_state[s];
  float* Sp = S + ((slot * heads + h) * dim) * vdim;
  float* Np = N + (slot * heads + h) * dim;
  float* mp = M + slot * heads + h;
  const T* row = proj + t * ld;
  const float icap = 1.f / cap;
  const float ig = cap * tanhf((gates[t * 2 * heads + h] + b_if[h]) * icap);
  const float fg = log_sigmoid(cap * tanhf((gates[t * 2 * heads + heads + h] + b_if[heads + h]) * icap));
  const float m0 = carried ? *mp : 0.f;
  const float m1 = fmaxf(fg + m0, ig);
  const float a = expf(fg + m0 - m1), b = expf(ig - m1);
  float nq = 0.f;
  for (int i = tid; i < dim; i += blockDim.x) {
    const float q = ldf<T>(row, (long)h * dim + i) * qscale, k = ldf<T>(row, (long)(heads + h) * dim + i);
    sq[i] = q;
    sk[i] = k;
    const float nn = __builtin_fmaf(a, carried ? Np[i] : 0.f, b * k);
    Np[i] = nn;
    nq = __builtin_fmaf(nn, q, nq);
  }
  nq = block_sum(nq, red);   // also the barrier after which sq / sk are read and every thread has read *mp
  if (tid == 0) *mp = m1;
  const float iden = 1.f / (fmaxf(fabsf(nq), expf(-m1)) + 1e-6f);
  const long voff = 2L * heads * dim + (long)h * vdim;
  const int per = (dim + G - 1) / G, lo = g * per, hi = min(dim, lo + per);
  float ov[kStepCols];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kStepCols; ++j) {
    const int c = c0 + 256 * j;
    ov[j] = 0.f;
    if (256 * j >= vdim) break;   // uniform over the workgroup
    float acc = 0.f;
    if (c < vdim) {
      const float bv = b * ldf<T>(row, voff + c);
      float* col = Sp + c;
      for (int i0 = lo; i0 < hi; i0 += 8) {
        float sv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) sv[u] = (carried && i0 + u < hi) ? col[(long)(i0 + u) * vdim] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (i0 + u < hi) {
            const float st = __builtin_fmaf(a, sv[u], bv * sk[i0 + u]);
            col[(long)(i0 + u) * vdim] = st;
            acc = __builtin_fmaf(st, sq[i0 + u], acc);
          }
        }
      }
    }
    if (G > 1) {
      if (g > 0) part[(g - 1) * 256 + c0] = acc;
      __syncthreads();
      if (g == 0)
        for (int gg = 1; gg < G; ++gg) acc += part[(gg - 1) * 256 + c0];
      __syncthreads();
    }
    if (g == 0 && c < vdim) {
      ov[j] = acc * iden;
      ss += ov[j] * ov[j];
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)vdim + eps);
  const long goff = voff + (long)heads * vdim;
  if (g != 0) return;
#pragma unroll
  for (int j = 0; j < kStepCols; ++j) {
    const int c = c0 + 256 * j;
    if (c < vdim)
      stf<T>(out, (t * heads + h) * vdim + c, ov[j] * inv * w[h * vdim + c] * sigmoid_f(ldf<T>(row, goff + c)));
  }
}

int ds_of(int dim) { return dim <= 16 ? 1 : dim <= 32 ? 2 : dim <= 64 ? 4 : dim <= 128 ? 8 : dim <= 256 ? 16 : 32; }

template <typename T>
void run(void* out, float* S, float* N, float* M, const void* proj, long ld, const float* gates, const float* b_if,
         const float* norm_w, const int* seq_cu, const int* seq_ctx, const int* seq_state, int nseq, int T_rows,
         float* scratch, int heads, int dim, int vdim, float cap, float eps, bool one_row_seqs, hipStream_t s) {
  const float qscale = 1.f / sqrtf((float)dim);
  if (one_row_seqs && vdim <= 256 * kStepCols) {
    const int G = dim >= 64 ? 4 : dim >= 16 ? 2 : 1;
    mlstm_step_kernel<T><<<dim3(heads, nseq), 256 * G, (2 * dim + (G - 1) * 256) * sizeof(float), s>>>(
        (T*)out, S, N, M, (const T*)proj, ld, gates, b_if, norm_w, seq_cu, seq_ctx, seq_state, heads, dim, vdim, cap,
        qscale, eps);
    return;
  }
  f32x4* scr = reinterpret_cast<f32x4*>(scratch);          // [T, heads] (a, b, exp(-m), 0)
  float* o = scratch + (long)T_rows * heads * 4;             // [T, heads, vdim + 1]
  float* vv = o + (long)T_rows * heads * (vdim + 1);         // [T, heads, vdim + 1]
  float* qk = vv + (long)T_rows * heads * (vdim + 1);        // [T, heads, 2 dim]
  mlstm_stage_kernel<T><<<T_rows, 256, 0, s>>>(qk, vv, (const T*)proj, ld, heads, dim, vdim, qscale);
  mlstm_gates_kernel<<<dim3(heads, nseq), 64, 0, s>>>(scr, M, gates, b_if, seq_cu, seq_ctx, seq_state, heads, cap);
  dim3 grid(heads, (vdim + 1 + kCols - 1) / kCols, nseq);
  switch (ds_of(dim)) {
#define HS_ML(D)                                                                                                    \
  case D:                                                                                                           \
    mlstm_scan_kernel<D><<<grid, kScanThreads, 0, s>>>(o, S, N, qk, vv, scr, seq_cu, seq_ctx, seq_state, heads, dim,  \
                                                      vdim);                                                        \
    break;
    HS_ML(1) HS_ML(2) HS_ML(4) HS_ML(8) HS_ML(16) HS_ML(32)
#undef HS_ML
  }
  const long nrow = (long)T_rows * heads;
  mlstm_out_kernel<T><<<(unsigned)((nrow + 3) / 4), 256, 0, s>>>((T*)out, o, scr, (const T*)proj, ld,
                                                               2 * heads * dim + heads * vdim, norm_w, T_rows, heads,
                                                               vdim, eps);
}

}  // namespace

int mlstm_max_dim() { return 512; }

void launch_mlstm(void* out, float* S, float* N, float* M, const void* proj, long ld, const float* gates,
                  const float* b_if, const float* norm_w, const int* seq_cu, const int* seq_ctx, const int* seq_state,
                  int nseq, int T, float* scratch, int heads, int dim, int vdim, float cap, float eps,
                  bool one_row_seqs, bool f32, hipStream_t s) {
  if (nseq <= 0 || T <= 0) return;
  if (f32)
    run<float>(out, S, N, M, proj, ld, gates, b_if, norm_w, seq_cu, seq_ctx, seq_state, nseq, T, scratch, heads, dim,
               vdim, cap, eps, one_row_seqs, s);
  else
    run<unsigned short>(out, S, N, M, proj, ld, gates, b_if, norm_w, seq_cu, seq_ctx, seq_state, nseq, T, scratch,
                        heads, dim, vdim, cap, eps, one_row_seqs, s);
}

}  // namespace hipserve
