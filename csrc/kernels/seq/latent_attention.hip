// Latent attention on a paged latent cache [blocks, block_size, kv_rank + rot_dim].
//
// latent_prepare: per token, the two latent RMSNorms (query latent -> cq, key/value latent ->
// cache row), the rotary key part (rotate-half over the first 2 * nfreq dims, angle = pos *
// inv_freq[i] in fp32) and the paged cache write.
//
// latent_attention: the key up-projection is absorbed into the query on the host side
// (q_abs[h, t, :] = W_uk_h^T q_unrot), so every head scores directly against the cached row:
//   score = (q_abs . latent + RoPE(q_rot) . rotary key) * scale,  keys 0 <= pos - j < window
// and the output stays in latent space (sum_j p_j latent_j), times the head's sigmoid gate; the
// value up-projection is a batched GEMM afterwards. All heads share one "key head", so a
// workgroup stages each 64-key tile once for all its (token, head) rows: one wave per row,
// lane = key for the scores (online softmax per wave), lane = latent dim for the output.
// Scores, softmax and accumulation are fp32; bf16 / fp32 only differ in the element type of
// q, the cache and the output.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    T* __restrict__ cq, T* __restrict__ cache, const T* __restrict__ proj, long ld, const long* __restrict__ positions,
    const long* __restrict__ slots, const float* __restrict__ q_norm, const float* __restrict__ kv_norm,
    const float* __restrict__ inv_freq, int nfreq, int q_rank, int kv_rank, int rot_dim, float eps) {
  __shared__ float scratch[8];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  const T* row = proj + t * ld;
  float a = 0.f, b = 0.f;
  for (int e = tid; e < q_rank; e += 256) { const float v = ldf<T>(row, e); a += v * v; }
  for (int e = tid; e < kv_rank; e += 256) { const float v = ldf<T>(row, q_rank + e); b += v * v; }
  a = block_sum(a, scratch);
  b = block_sum(b, scratch);
  const float ia = 1.f / sqrtf(a / (float)q_rank + eps), ib = 1.f / sqrtf(b / (float)kv_rank + eps);
  for (int e = tid; e < q_rank; e += 256) stf<T>(cq, t * q_rank + e, ldf<T>(row, e) * ia * q_norm[e]);
  const long slot = slots[t];
  if (slot < 0) return;
  T* dst = cache + slot * (kv_rank + rot_dim);
  for (int e = tid; e < kv_rank; e += 256) stf<T>(dst, e, ldf<T>(row, q_rank + e) * ib * kv_norm[e]);
  const T* kr = row + q_rank + kv_rank;
  const float pos = (float)positions[t];
  for (int e = tid; e < rot_dim; e += 256) {
    float v;
    if (e < 2 * nfreq) {
      const int i = e < nfreq ? e : e - nfreq;
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      const float u = ldf<T>(kr, i), w = ldf<T>(kr, i + nfreq);
      v = e < nfreq ? u * cs - w * sn : w * cs + u * sn;
    } else {
      v = ldf<T>(kr, e);
    }
    stf<T>(dst, kv_rank + e, v);
  }
}

constexpr int kKT = 64;       // keys per tile (one per lane)
constexpr int kDC = 64;       // cache dims per staged chunk
constexpr int kMaxCh = 16;    // kv_rank <= kMaxCh * 64
constexpr int kMaxRows = 16;  // waves per workgroup

// Finds the workgroup's (sequence, first token) among sequences seq0..seq1-1, `tq` tokens per workgroup.
HS_DEVICE bool find_tile(const int* __restrict__ seq_cu, int seq0, int seq1, int tq, int wg, int& s, int& tok0) {
  int acc = 0;
  for (int i = seq0; i < seq1; ++i) {
    const int n = seq_cu[i + 1] - seq_cu[i];
    const int nt = (n + tq - 1) / tq;
    if (wg < acc + nt) {
      s = i;
      tok0 = (wg - acc) * tq;
      return true;
    }
    acc += nt;
  }
  return false;
}

template <typename T>
__global__ __launch_bounds__(64 * kMaxRows) void latent_attention_kernel(
    T* __restrict__ o_lat, const float* __restrict__ q_abs, const T* __restrict__ q, const T* __restrict__ proj,
    long proj_ld, const T* __restrict__ cache, int block_size, const int* __restrict__ seq_cu,
    const int* __restrict__ seq_ctx, const int* __restrict__ seq_bt, int bt_width, int seq0, int seq1, int tq, int hc,
    const float* __restrict__ inv_freq, int nfreq, int T_rows, int heads, int dim, int rot_dim, int kv_rank,
    int gate_off, float scale, int window) {
  extern __shared__ float sm[];
  const int Dk = kv_rank + rot_dim;
  const int nrows = blockDim.x >> 6;
  long* krow = reinterpret_cast<long*>(sm);        // [kKT] cache row offsets (elements), -1 = no key
  float* qs = sm + 2 * kKT;                        // [nrows][Dk]
  float* kc = qs + nrows * Dk;                     // [kKT][kDC + 1]
  float* ps = kc + kKT * (kDC + 1);                // [nrows][kKT]
  int s, tok0;
  if (!find_tile(seq_cu, seq0, seq1, tq, blockIdx.x, s, tok0)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r0 = seq_cu[s], n = seq_cu[s + 1] - r0, ctx = seq_ctx[s];
  const int ntok = min(tq, n - tok0);
  const int h0 = blockIdx.y * hc;
  const int nh = min(hc, heads - h0);
  // row of this wave: token wave / hc, head wave % hc
  const int wt = wave / hc, wh = wave % hc;
  const bool active = wt < ntok && wh < nh;
  const int trow = r0 + tok0 + (active ? wt : 0);           // batch row of the token
  const int head = h0 + (active ? wh : 0);
  const int pos = ctx - n + tok0 + (active ? wt : 0);        // position of the token
  // stage the row's query: absorbed part, then the rotary part rotated at its position
  if (active) {
    const float* qa = q_abs + ((long)head * T_rows + trow) * kv_rank;
    for (int e = lane; e < kv_rank; e += 64) qs[wave * Dk + e] = qa[e];
    const T* qr = q + (long)trow * heads * (dim + rot_dim) + (long)head * (dim + rot_dim) + dim;
    const float fp = (float)pos;
    for (int e = lane; e < rot_dim; e += 64) {
      float v;
      if (e < 2 * nfreq) {
        const int i = e < nfreq ? e : e - nfreq;
        float sn, cs;
        sincosf(fp * inv_freq[i], &sn, &cs);
        const float u = ldf<T>(qr, i), w = ldf<T>(qr, i + nfreq);
        v = e < nfreq ? u * cs - w * sn : w * cs + u * sn;
      } else {
        v = ldf<T>(qr, e);
      }
      qs[wave * Dk + kv_rank + e] = v;
    }
  }
  const int p_first = ctx - n + tok0, p_last = p_first + ntok - 1;
  const int lo = window > 0 ? max(0, p_first - window + 1) : 0;
  const int my_lo = window > 0 ? max(0, pos - window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[kMaxCh];
#pragma unroll
  for (int c = 0; c < kMaxCh; ++c) acc[c] = 0.f;
  const int nkc = (kv_rank + kDC - 1) / kDC, ndc = (Dk + kDC - 1) / kDC;
  for (int j0 = lo; j0 <= p_last; j0 += kKT) {
    __syncthreads();  // previous tile's chunk reads are done (and qs is staged, first time)
    if (tid < kKT) {
      const int j = j0 + tid;
      krow[tid] = j <= p_last ? ((long)seq_bt[(long)s * bt_width + j / block_size] * block_size + j % block_size) * Dk
                              : -1;
    }
    // scores: lane = key, chunks of the cache row staged through LDS
    float sc = 0.f;
    for (int c = 0; c < ndc; ++c) {
      __syncthreads();
      const int d0 = c * kDC, dn = min(kDC, Dk - d0);
      for (int idx = tid; idx < kKT * kDC; idx += blockDim.x) {
        const int k = idx / kDC, d = idx % kDC;
        const long kr = krow[k];
        kc[k * (kDC + 1) + d] = (kr >= 0 && d < dn) ? ldf<T>(cache, kr + d0 + d) : 0.f;
      }
      __syncthreads();
      if (active) {
        const float* qv = qs + wave * Dk + d0;
        const float* kv = kc + lane * (kDC + 1);
        for (int d = 0; d < dn; ++d) sc = __builtin_fmaf(qv[d], kv[d], sc);
      }
    }
    const int j = j0 + lane;
    const bool vis = active && j <= pos && j >= my_lo;
    sc = vis ? sc * scale : -INFINITY;
    const float tmax = wave_max(sc);
    float p = 0.f, alpha = 1.f;
    if (tmax > -INFINITY) {  // wave-uniform: some key of the tile is visible to this row
      const float mn = fmaxf(m, tmax);
      alpha = expf(m - mn);   // m = -inf the first time: 0
      p = vis ? expf(sc - mn) : 0.f;
      l = l * alpha + wave_sum(p);
      m = mn;
    }
    ps[wave * kKT + lane] = p;
    // output: lane = latent dim within the chunk
    for (int c = 0; c < nkc; ++c) {
      __syncthreads();
      const int d0 = c * kDC, dn = min(kDC, kv_rank - d0);
      for (int idx = tid; idx < kKT * kDC; idx += blockDim.x) {
        const int k = idx / kDC, d = idx % kDC;
        const long kr = krow[k];
        kc[k * (kDC + 1) + d] = (kr >= 0 && d < dn) ? ldf<T>(cache, kr + d0 + d) : 0.f;
      }
      __syncthreads();
      float o = 0.f;
      const float* pv = ps + wave * kKT;
      for (int k = 0; k < kKT; ++k) o = __builtin_fmaf(pv[k], kc[k * (kDC + 1) + lane], o);
#pragma unroll
      for (int cc = 0; cc < kMaxCh; ++cc)
        if (cc == c) acc[cc] = acc[cc] * alpha + o;
    }
  }
  if (!active) return;
  const float g = gate_off >= 0 ? sigmoid_f(ldf<T>(proj, (long)trow * proj_ld + gate_off + head)) : 1.f;
  const float inv = l > 0.f ? g / l : 0.f;
  T* dst = o_lat + ((long)head * T_rows + trow) * kv_rank;
#pragma unroll
  for (int c = 0; c < kMaxCh; ++c) {
    const int e = c * kDC + lane;
    if (c < nkc && e < kv_rank) stf<T>(dst, e, acc[c] * inv);
  }
}

}  // namespace

void launch_latent_prepare(void* cq, void* cache, const void* proj, long ld, const long* positions, const long* slots,
                           const float* q_norm, const float* kv_norm, const float* inv_freq, int nfreq, int T,
                           int q_rank, int kv_rank, int rot_dim, float eps, bool f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    latent_prepare_kernel<float><<<T, 256, 0, s>>>((float*)cq, (float*)cache, (const float*)proj, ld, positions, slots,
                                                   q_norm, kv_norm, inv_freq, nfreq, q_rank, kv_rank, rot_dim, eps);
  else
    latent_prepare_kernel<unsigned short><<<T, 256, 0, s>>>((unsigned short*)cq, (unsigned short*)cache,
                                                            (const unsigned short*)proj, ld, positions, slots, q_norm,
                                                            kv_norm, inv_freq, nfreq, q_rank, kv_rank, rot_dim, eps);
}

void launch_latent_attention(void* o_lat, const float* q_abs, const void* q, const void* proj, long proj_ld,
                             const void* cache, int block_size, const int* seq_cu, const int* seq_ctx,
                             const int* seq_bt, int bt_width, int seq0, int seq1, int rows_bound, int tq,
                             const float* inv_freq, int nfreq, int T, int heads, int dim, int rot_dim, int kv_rank,
                             int gate_off, float scale, int window, bool f32, hipStream_t s) {
  if (seq1 <= seq0 || rows_bound <= 0) return;
  const int Dk = kv_rank + rot_dim;
  auto lds = [&](int rows) {
    return ((size_t)rows * Dk + kKT * (kDC + 1) + (size_t)rows * kKT) * sizeof(float) + kKT * sizeof(long);
  };
  int hc = min(heads, kMaxRows / tq);
  while (lds(tq * hc) > 60 * 1024 && tq > 1) { tq /= 2; hc = min(heads, kMaxRows / tq); }
  while (lds(tq * hc) > 60 * 1024 && hc > 1) hc /= 2;
  const int nrows = tq * hc;
  // workgroups: at most ceil(n_s / tq) per sequence <= rows_bound / tq + number of sequences
  dim3 grid(rows_bound / tq + (seq1 - seq0), (heads + hc - 1) / hc), block(64 * nrows);
  const size_t smem = lds(nrows);
  if (f32)
    latent_attention_kernel<float><<<grid, block, smem, s>>>(
        (float*)o_lat, q_abs, (const float*)q, (const float*)proj, proj_ld, (const float*)cache, block_size, seq_cu,
        seq_ctx, seq_bt, bt_width, seq0, seq1, tq, hc, inv_freq, nfreq, T, heads, dim, rot_dim, kv_rank, gate_off,
        scale, window);
  else
    latent_attention_kernel<unsigned short><<<grid, block, smem, s>>>(
        (unsigned short*)o_lat, q_abs, (const unsigned short*)q, (const unsigned short*)proj, proj_ld,
        (const unsigned short*)cache, block_size, seq_cu, seq_ctx, seq_bt, bt_width, seq0, seq1, tq, hc, inv_freq,
        nfreq, T, heads, dim, rot_dim, kv_rank, gate_off, scale, window);
}

}  // namespace hipserve
