// Grouped-query attention over a sliding window on a paged cache [blocks, block_size, keys | values]
// (all key heads of a token, then all its value heads), with an optional softmax sink and an
// optional per-head output gate.
//
// attn_prepare: per token, on the merged projection row [q | k | v | ...] (biases already added):
// the optional RMS norm of q and k (over the WHOLE projection with a weight per element, or over
// every head of `dim` elements with one weight of `dim` elements for all heads), the
// rotate-half rotation of the first 2 * nfreq dims of every q / k head (angle = pos * inv_freq[i],
// fp32), the optional division of every value head by its root mean square, q written back in
// place, k and v into the cache row. Without a cache (a layer that reads another layer's keys and
// values) the row is [q | ...] and only q is prepared.
//
// Two maps per head (differential attention): a query / key head holds [map 1 | map 2], `dim` each,
// so for the norm and the rotation there are simply twice as many heads; the attention kernel runs
// both maps of a (token, head) row in one wave over the same staged value tile and writes
// (a1 - lam a2) / rms(a1 - lam a2) * post.
//
// window_attention: one wave per (token, query head) row; a workgroup holds `tq` tokens x the
// query heads of ONE key/value head, so each 64-key tile is staged once for all of them. Scores:
// lane = key, the head's key dims staged in chunks of 64 through LDS; online softmax per wave;
// output: lane = value dim. With the sink the running (max, sum) start at (sink logit, 1): a key
// without a value whose score is a learned number per head (0 without sink weights). Options:
// softcap > 0 passes the scaled scores through softcap * tanh(. / softcap); keep > 0 keeps the
// sequence's first `keep` keys visible behind the window. The kernel then walks a compacted key
// index u: the kept keys below the workgroup's window first (u < nk), then the window's keys
// (key = u - nk + lo), so tiles, runs of keys and the split over workgroups need no second loop.
// Scores, softmax and accumulation are fp32 for both element types.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

// One head's rotation work items: `dim - nfreq` per head; item i < nfreq is the pair (i, i + nfreq),
// item i >= nfreq the unrotated element i + nfreq. Every element belongs to exactly one item.
// `hinv` (per-head inverse rms, or null: `inv` for all) and `w` (null: none; wmod > 0: one weight of wmod
// elements shared by all heads, else a weight per element of the projection).
template <typename T, typename F>
HS_DEVICE void rotate_heads(const T* __restrict__ src, int nheads, int dim, int nfreq, float pos,
                            const float* __restrict__ inv_freq, float inv, const float* __restrict__ hinv,
                            const float* __restrict__ w, int wmod, int tid, F&& store) {
  const int per = dim - nfreq;
  for (int it = tid; it < nheads * per; it += 256) {
    const int h = it / per, i = it % per;
    const int off = i < nfreq ? i : i + nfreq;
    const int e0 = h * dim + off;
    const float sc = hinv != nullptr ? hinv[h] : inv;
    float a = ldf<T>(src, e0) * sc;
    if (w != nullptr) a *= w[wmod > 0 ? off : e0];
    if (i < nfreq) {
      const int e1 = e0 + nfreq;
      float b = ldf<T>(src, e1) * sc;
      if (w != nullptr) b *= w[wmod > 0 ? off + nfreq : e1];
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      store(e0, a * cs - b * sn);
      store(e1, b * cs + a * sn);
    } else {
      store(e0, a);
    }
  }
}

// heads / kv_heads count the maps (twice the head counts for two maps per head). norm_mode 0: none, 1: over the
// whole q (k) projection, 2: per head with one shared weight of `dim` elements. cache null: q only.
template <typename T>
__global__ __launch_bounds__(256) void attn_prepare_kernel(
    T* __restrict__ proj, long ld, T* __restrict__ cache, const long* __restrict__ positions,
    const long* __restrict__ slots, const float* __restrict__ inv_freq, int nfreq, int heads, int kv_heads, int vheads,
    int dim, int vdim, const float* __restrict__ q_norm, const float* __restrict__ k_norm, int norm_mode, bool v_norm,
    float eps) {
  extern __shared__ float hinv[];  // norm_mode 2: [heads + kv_heads] inverse rms per head
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool own_kv = cache != nullptr;
  const int nq = heads * dim, nk = own_kv ? kv_heads * dim : 0, nv = vheads * vdim;
  T* row = proj + t * ld;
  float iq = 1.f, ik = 1.f;
  if (norm_mode == 1) {
    float a = 0.f, b = 0.f;
    for (int e = tid; e < nq; e += 256) { const float v = ldf<T>(row, e); a += v * v; }
    for (int e = tid; e < nk; e += 256) { const float v = ldf<T>(row, nq + e); b += v * v; }
    a = block_sum(a, scratch);
    b = block_sum(b, scratch);
    iq = 1.f / sqrtf(a / (float)nq + eps);
    ik = 1.f / sqrtf(b / (float)max(nk, 1) + eps);
  } else if (norm_mode == 2) {
    const int nh = heads + (own_kv ? kv_heads : 0);   // the key heads follow the query heads in the row
    for (int h = wave; h < nh; h += 4) {
      float a = 0.f;
      for (int e = lane; e < dim; e += 64) { const float v = ldf<T>(row, (long)h * dim + e); a += v * v; }
      a = wave_sum(a);
      if (lane == 0) hinv[h] = 1.f / sqrtf(a / (float)dim + eps);
    }
    __syncthreads();
  }
  const float* hq = norm_mode == 2 ? hinv : nullptr;
  const int wmod = norm_mode == 2 ? dim : 0;
  const float pos = (float)positions[t];
  rotate_heads<T>(row, heads, dim, nfreq, pos, inv_freq, iq, hq, q_norm, wmod, tid,
                  [&](int e, float v) { stf<T>(row, e, v); });
  if (!own_kv) return;
  const long slot = slots[t];
  if (slot < 0) return;
  T* dst = cache + slot * (long)(nk + nv);
  rotate_heads<T>(row + nq, kv_heads, dim, nfreq, pos, inv_freq, ik, hq != nullptr ? hq + heads : nullptr, k_norm,
                  wmod, tid, [&](int e, float v) { stf<T>(dst, e, v); });
  const T* vr = row + nq + nk;
  for (int g = wave; g < vheads; g += 4) {  // one wave per value head
    float inv = 1.f;
    if (v_norm) {
      float a = 0.f;
      for (int e = lane; e < vdim; e += 64) { const float v = ldf<T>(vr, g * vdim + e); a += v * v; }
      inv = 1.f / sqrtf(wave_sum(a) / (float)vdim + eps);
    }
    for (int e = lane; e < vdim; e += 64) stf<T>(dst, nk + g * vdim + e, ldf<T>(vr, g * vdim + e) * inv);
  }
}

constexpr int kKT = 64;       // keys per tile (one per lane)
constexpr int kDC = 64;       // key / value dims per staged chunk
constexpr int kMaxCh = 8;     // vdim <= kMaxCh * 64
constexpr int kMaxRows = 16;  // waves per workgroup

HS_DEVICE bool find_row_tile(const int* __restrict__ seq_cu, int seq0, int seq1, int tq, int wg, int& s, int& tok0) {
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

// grid.y = kv_heads * hchunks: workgroup y serves query heads g * group + c * hc .. of key/value head g.
// MAPS = 2: the row's two maps (queries [map 1 | map 2], keys alike) run side by side with their own
// running (max, sum) and accumulators over the same value chunks; the output is
// o = a1 - lam a2,  o / sqrt(mean(o^2) + eps) * post.
template <typename T, int MAPS>
__global__ __launch_bounds__(64 * kMaxRows) void window_attention_kernel(
    T* __restrict__ out, long out_ld, const T* __restrict__ proj, long proj_ld, const T* __restrict__ cache,
    int block_size, const int* __restrict__ seq_cu, const int* __restrict__ seq_ctx, const int* __restrict__ seq_bt,
    int bt_width, int seq0, int seq1, int tq, int hc, int hchunks, int heads, int kv_heads, int dim, int vdim,
    int gate_off, float scale, int window, bool sink, float out_scale, float lam, float post, float eps, int keep,
    float softcap, const float* __restrict__ sink_w) {
  extern __shared__ float sm[];
  const int nrows = blockDim.x >> 6;
  const int qd = MAPS * dim;                       // a row's query elements
  long* krow = reinterpret_cast<long*>(sm);        // [kKT] cache row offsets (elements), -1 = no key
  float* qs = sm + 2 * kKT;                        // [nrows][qd]
  float* kc = qs + nrows * qd;                     // [kKT][kDC + 1]
  float* ps = kc + kKT * (kDC + 1);                // [nrows][MAPS][kKT]
  int s, tok0;
  if (!find_row_tile(seq_cu, seq0, seq1, tq, blockIdx.x, s, tok0)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int group = heads / kv_heads;
  const int g = blockIdx.y / hchunks, h0 = (blockIdx.y % hchunks) * hc;
  const int nh = min(hc, group - h0);
  const int r0 = seq_cu[s], n = seq_cu[s + 1] - r0, ctx = seq_ctx[s];
  const int ntok = min(tq, n - tok0);
  const int wt = wave / hc, wh = wave % hc;
  const bool active = wt < ntok && wh < nh;
  const int trow = r0 + tok0 + (active ? wt : 0);
  const int head = g * group + h0 + (active ? wh : 0);
  const int pos = ctx - n + tok0 + (active ? wt : 0);
  const long Dc = (long)kv_heads * (qd + vdim);
  const long koff = (long)g * qd, voff = (long)kv_heads * qd + (long)g * vdim;
  if (active) {
    const T* q = proj + (long)trow * proj_ld + (long)head * qd;
    for (int e = lane; e < qd; e += 64) qs[wave * qd + e] = ldf<T>(q, e);
  }
  const int p_first = ctx - n + tok0, p_last = p_first + ntok - 1;
  const int lo = window > 0 ? max(0, p_first - window + 1) : 0;
  const int my_lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int nk = (window > 0 && keep > 0) ? min(keep, lo) : 0;   // kept keys below the workgroup's window
  const int total = nk + p_last - lo + 1;
  const float sink0 = (sink && sink_w != nullptr) ? sink_w[head] : 0.f;
  const float icap = softcap > 0.f ? 1.f / softcap : 0.f;
  float m[MAPS], l[MAPS], acc[MAPS][kMaxCh];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp) {
    m[mp] = sink ? sink0 : -INFINITY;
    l[mp] = sink ? 1.f : 0.f;
#pragma unroll
    for (int c = 0; c < kMaxCh; ++c) acc[mp][c] = 0.f;
  }
  const int nkc = (dim + kDC - 1) / kDC, nvc = (vdim + kDC - 1) / kDC;
  for (int u0 = 0; u0 < total; u0 += kKT) {
    __syncthreads();  // the previous tile's chunk reads are done (and qs is staged, the first time)
    if (tid < kKT) {
      const int u = u0 + tid;
      const int j = u < nk ? u : u - nk + lo;
      krow[tid] = u < total ? ((long)seq_bt[(long)s * bt_width + j / block_size] * block_size + j % block_size) * Dc
                            : -1;
    }
    const int u = u0 + lane;
    const int j = u < nk ? u : u - nk + lo;
    const bool vis = active && u < total && j <= pos && (j >= my_lo || j < keep);
    float alpha[MAPS];
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      float sc = 0.f;
      for (int c = 0; c < nkc; ++c) {
        __syncthreads();
        const int d0 = c * kDC, dn = min(kDC, dim - d0);
        for (int idx = tid; idx < kKT * kDC; idx += blockDim.x) {
          const int k = idx / kDC, d = idx % kDC;
          const long kr = krow[k];
          kc[k * (kDC + 1) + d] = (kr >= 0 && d < dn) ? ldf<T>(cache, kr + koff + mp * dim + d0 + d) : 0.f;
        }
        __syncthreads();
        if (active) {
          const float* qv = qs + wave * qd + mp * dim + d0;
          const float* kv = kc + lane * (kDC + 1);
          for (int d = 0; d < dn; ++d) sc = __builtin_fmaf(qv[d], kv[d], sc);
        }
      }
      sc *= scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc * icap);
      sc = vis ? sc : -INFINITY;
      const float tmax = wave_max(sc);
      float p = 0.f;
      alpha[mp] = 1.f;
      if (tmax > -INFINITY) {  // wave-uniform: some key of the tile is visible to this row
        const float mn = fmaxf(m[mp], tmax);
        alpha[mp] = expf(m[mp] - mn);   // m = -inf the first time (no sink): 0
        p = vis ? expf(sc - mn) : 0.f;
        l[mp] = l[mp] * alpha[mp] + wave_sum(p);
        m[mp] = mn;
      }
      ps[(wave * MAPS + mp) * kKT + lane] = p;
    }
    for (int c = 0; c < nvc; ++c) {
      __syncthreads();
      const int d0 = c * kDC, dn = min(kDC, vdim - d0);
      for (int idx = tid; idx < kKT * kDC; idx += blockDim.x) {
        const int k = idx / kDC, d = idx % kDC;
        const long kr = krow[k];
        kc[k * (kDC + 1) + d] = (kr >= 0 && d < dn) ? ldf<T>(cache, kr + voff + d0 + d) : 0.f;
      }
      __syncthreads();
#pragma unroll
      for (int mp = 0; mp < MAPS; ++mp) {
        float o = 0.f;
        const float* pv = ps + (wave * MAPS + mp) * kKT;
        for (int k = 0; k < kKT; ++k) o = __builtin_fmaf(pv[k], kc[k * (kDC + 1) + lane], o);
#pragma unroll
        for (int cc = 0; cc < kMaxCh; ++cc)
          if (cc == c) acc[mp][cc] = acc[mp][cc] * alpha[mp] + o;
      }
    }
  }
  if (!active) return;
  float f = out_scale;
  if (gate_off >= 0) f *= sigmoid_f(ldf<T>(proj, (long)trow * proj_ld + gate_off + head));
  T* dst = out + (long)trow * out_ld + (long)head * vdim;
  if constexpr (MAPS == 2) {
    const float i0 = l[0] > 0.f ? 1.f / l[0] : 0.f, i1 = l[1] > 0.f ? lam / l[1] : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < kMaxCh; ++c) {
      acc[0][c] = acc[0][c] * i0 - acc[1][c] * i1;
      if (c < nvc && c * kDC + lane < vdim) ss += acc[0][c] * acc[0][c];
    }
    f *= post / sqrtf(wave_sum(ss) / (float)vdim + eps);
#pragma unroll
    for (int c = 0; c < kMaxCh; ++c) {
      const int e = c * kDC + lane;
      if (c < nvc && e < vdim) stf<T>(dst, e, acc[0][c] * f);
    }
  } else {
    const float inv = l[0] > 0.f ? f / l[0] : 0.f;
#pragma unroll
    for (int c = 0; c < kMaxCh; ++c) {
      const int e = c * kDC + lane;
      if (c < nvc && e < vdim) stf<T>(dst, e, acc[0][c] * inv);
    }
  }
}

}  // namespace

void launch_attn_prepare(void* proj, long ld, void* cache, const long* positions, const long* slots,
                         const float* inv_freq, int nfreq, int T, int heads, int kv_heads, int maps, int dim, int vdim,
                         const float* q_norm, const float* k_norm, int norm_mode, bool v_norm, float eps, bool f32,
                         hipStream_t s) {
  if (T <= 0) return;
  const int qh = heads * maps, kh = kv_heads * maps;
  const size_t smem = (size_t)(qh + kh) * sizeof(float);
  if (f32)
    attn_prepare_kernel<float><<<T, 256, smem, s>>>((float*)proj, ld, (float*)cache, positions, slots, inv_freq, nfreq,
                                                    qh, kh, kv_heads, dim, vdim, q_norm, k_norm, norm_mode, v_norm, eps);
  else
    attn_prepare_kernel<unsigned short><<<T, 256, smem, s>>>((unsigned short*)proj, ld, (unsigned short*)cache,
                                                             positions, slots, inv_freq, nfreq, qh, kh, kv_heads, dim,
                                                             vdim, q_norm, k_norm, norm_mode, v_norm, eps);
}

int window_attention_max_vdim() { return kMaxCh * kDC; }

namespace {
template <typename T, int MAPS>
void launch_generic(void* out, long out_ld, const void* proj, long proj_ld, const void* cache, int block_size,
                    const int* seq_cu, const int* seq_ctx, const int* seq_bt, int bt_width, int seq0, int seq1,
                    int rows_bound, int tq, int heads, int kv_heads, int dim, int vdim, int gate_off, float scale,
                    int window, bool sink, float out_scale, float lam, float post, float eps, int keep, float softcap,
                    const float* sink_w, hipStream_t s) {
  const int group = heads / kv_heads;
  auto lds = [&](int rows) {
    return ((size_t)rows * MAPS * dim + kKT * (kDC + 1) + (size_t)rows * MAPS * kKT) * sizeof(float) +
           kKT * sizeof(long);
  };
  while (tq > 1 && tq > kMaxRows) tq /= 2;
  int hc = min(group, kMaxRows / tq);
  while (lds(tq * hc) > 60 * 1024 && tq > 1) { tq /= 2; hc = min(group, kMaxRows / tq); }
  while (lds(tq * hc) > 60 * 1024 && hc > 1) hc /= 2;
  const int hchunks = (group + hc - 1) / hc;
  const int nrows = tq * hc;
  dim3 grid(rows_bound / tq + (seq1 - seq0), kv_heads * hchunks), block(64 * nrows);
  window_attention_kernel<T, MAPS><<<grid, block, lds(nrows), s>>>(
      (T*)out, out_ld, (const T*)proj, proj_ld, (const T*)cache, block_size, seq_cu, seq_ctx, seq_bt, bt_width, seq0,
      seq1, tq, hc, hchunks, heads, kv_heads, dim, vdim, gate_off, scale, window, sink, out_scale, lam, post, eps, keep,
      softcap, sink_w);
}
}  // namespace

void launch_window_attention(void* out, long out_ld, const void* proj, long proj_ld, const void* cache, int block_size,
                             const int* seq_cu, const int* seq_ctx, const int* seq_bt, int bt_width, int seq0, int seq1,
                             int rows_bound, int tq, int heads, int kv_heads, int dim, int vdim, int gate_off,
                             float scale, int window, bool sink, float out_scale, int maps, float lam, float post,
                             float eps, int keep, float softcap, const float* sink_w, bool f32, hipStream_t s) {
  if (seq1 <= seq0 || rows_bound <= 0) return;
#define HS_GA(T, M)                                                                                                  \
  launch_generic<T, M>(out, out_ld, proj, proj_ld, cache, block_size, seq_cu, seq_ctx, seq_bt, bt_width, seq0, seq1,  \
                       rows_bound, tq, heads, kv_heads, dim, vdim, gate_off, scale, window, sink, out_scale, lam, post, \
                       eps, keep, softcap, sink_w, s)
  if (f32) { if (maps == 2) HS_GA(float, 2); else HS_GA(float, 1); }
  else { if (maps == 2) HS_GA(unsigned short, 2); else HS_GA(unsigned short, 1); }
#undef HS_GA
}

}  // namespace hipserve
