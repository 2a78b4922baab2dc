// Window attention on the matrix cores (bf16 activations and cache), same interface as the generic
// kernel of window_attention.hip: paged cache rows [all key heads | all value heads], sliding
// window, optional softmax sink, optional per-head sigmoid output gate, output scale.
//
// A workgroup (4 waves) owns 64 or 128 (token, query head) rows of ONE key/value head: consecutive
// tokens of one sequence x the query heads of the group, so all rows share one run of keys and a
// key / value tile is staged once for the whole group. A wave owns its 16 or 32 rows from the scores
// to the output, so the weights P never leave its registers. Per 32-key tile:
//   1. the head's key rows go to LDS row-major, its value rows TRANSPOSED (value dim major, the 32
//      keys of a row permuted into the order the score registers hold them, the row's four 8-key
//      chunks XOR-swizzled by the row index so the 2-byte transposing stores spread over the
//      banks), loaded one tile ahead;
//   2. S^T = K . Q^T per wave (mfma_f32_16x16x32_bf16, Q operands in registers): lane (c, g) holds
//      the scores of row c against keys 16 nt + 4 g + i;
//   3. masked online softmax in fp32 (log2 domain) in registers (a row's scores sit in four lanes); the
//      sink starts the running (max, sum) at (its logit, 1): 0, or a learned number per head; softcap > 0
//      passes the scaled scores through softcap * tanh(. / softcap) first;
//   4. O^T += V^T . P^T: the MFMA's k slot (g, e) stands for key 16 (e / 4) + 4 g + e % 4, which is
//      both where P's registers already are and one 16-byte read of the transposed value tile.
// Rows with few tokens and many keys (decode) split their keys over grid.z; the runs' unnormalised
// outputs and (max, sum) are merged by window_attention_reduce.
// keep > 0: the sequence's first `keep` keys stay visible behind the window. Tiles and runs walk a compacted
// key index u: the nk kept keys below the workgroup's window first, then the window (key = u - nk + lo).
//
// DIFF (differential attention): a query / key head holds two maps [map 1 | map 2]. The wave's two
// 16-row MFMA tiles are then the two MAPS of the same 16 (token, head) rows: each has its own key
// tile, scores, running (max, sum) and accumulators, and both multiply the one transposed value
// tile. The epilogue (or the reduce kernel of split rows) forms o = a1 - lam a2 and writes
// o / sqrt(mean(o^2) + eps) * post.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kKeys = 32;   // keys per tile
constexpr int kVLd = 40;    // transposed value tile: row stride in elements (32 keys + pad, 16-byte aligned rows)
HS_DEVICE float tanh_fast(float x) {  // 1 - 2 / (e^2x + 1); saturates cleanly at both ends
  return 1.f - 2.f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x * 2.88539008177792681f) + 1.f);
}

constexpr int kNW = 4, kRows = 16 * kNW /* x MT */, kThreads = 64 * kNW, kFT = kThreads / kKeys;

template <int KS> struct KLd { static constexpr int v = KS * 32 + 8; };

HS_DEVICE bool find_tile_rows(const int* __restrict__ seq_cu, int seq0, int seq1, int tq, int wg, int& s, int& tok0) {
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

// KS: 32-dim steps of a key head (dim <= 32 KS); NV: 16-dim tiles of a value head (vdim <= 16 NV); MT: 16-row
// tiles per wave (a workgroup owns 64 MT rows; every key / value operand read from LDS feeds MT MFMAs).
template <int KS, int NV, int MT, bool DIFF>
__global__ __launch_bounds__(kThreads, 2) void window_attention_mfma_kernel(
    unsigned short* __restrict__ out, long out_ld, const unsigned short* __restrict__ proj, long proj_ld,
    const unsigned short* __restrict__ cache, int block_size, const int* __restrict__ seq_cu,
    const int* __restrict__ seq_ctx, const int* __restrict__ seq_bt, int bt_width, int seq0, int seq1, int tq, int hc,
    int hchunks, int heads, int kv_heads, int dim, int vdim, int gate_off, float scale, int window, bool sink,
    float out_scale, int part_keys, float* __restrict__ ws_acc, float* __restrict__ ws_ml, int row_base, int ws_rows,
    float lam, float post, float eps, bool one_row_seqs, bool qvec, int keep, float softcap,
    const float* __restrict__ sink_w) {
  static_assert(!DIFF || MT % 2 == 0, "a wave's row tiles come in pairs: the two maps of the same 16 rows");
  constexpr int RT = DIFF ? MT / 2 : MT;   // distinct 16-row tiles per wave; tile mt is rows mt / kMaps, map mt % kMaps
  constexpr int kLd = KLd<KS>::v;
  constexpr int kMaps = DIFF ? 2 : 1;
  constexpr int kKF = (kMaps * KS * 4 + kFT - 1) / kFT, kVF = (NV * 2 + kFT - 1) / kFT;  // 16-byte chunks per thread and tile
  __shared__ __attribute__((aligned(16))) unsigned short kt[kMaps * kKeys * kLd];  // [map][key][dim]
  __shared__ __attribute__((aligned(16))) unsigned short vt[NV * 16 * kVLd];  // [value dim][permuted key]
  int s, tok0;
  if (one_row_seqs) {  // decode rows: sequence seq0 + x has the one row of workgroup x (no walk over the row counts)
    s = seq0 + blockIdx.x;
    tok0 = 0;
    if (s >= seq1) return;
  } else if (!find_tile_rows(seq_cu, seq0, seq1, tq, blockIdx.x, s, tok0)) {
    return;
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int group = heads / kv_heads;
  const int kvh = blockIdx.y / hchunks, h0 = (blockIdx.y % hchunks) * hc;
  const int nh = min(hc, group - h0);
  const int r0 = seq_cu[s], n = seq_cu[s + 1] - r0, ctx = seq_ctx[s];
  const int ntok = min(tq, n - tok0);
  const int p_first = ctx - n + tok0, p_last = p_first + ntok - 1;
  const int lo_all = window > 0 ? max(0, p_first - window + 1) : 0;
  const int nk = (window > 0 && keep > 0) ? min(keep, lo_all) : 0;   // kept keys below the workgroup's window
  const int total = nk + p_last - lo_all + 1;
  const int lo = blockIdx.z * part_keys;                              // compacted key indices from here on
  const int hi = gridDim.z > 1 ? min(total - 1, lo + part_keys - 1) : total - 1;
  auto key_of = [&](int u) { return u < nk ? u : u - nk + lo_all; };
  const float cap2 = softcap * 1.44269504088896341f, icap = softcap > 0.f ? scale / softcap : 0.f;
  const long Dc = (long)kv_heads * (kMaps * dim + vdim);
  const long koff = (long)kvh * kMaps * dim, voff = (long)kv_heads * kMaps * dim + (long)kvh * vdim;
  const bool first_part = blockIdx.z == 0;
  const float scale2 = scale * 1.44269504088896341f;
  // this lane's rows: row sr = token sr / hc, head sr % hc of the group
  bool sact[MT];
  int head[MT], spos[MT], s_lo[MT];
  long trow[MT];
  bf16x8 qf[MT][KS];   // Q operands of the rows: dims 32 ks + 8 g .. + 7
  f32x4 acc[MT][NV];
  float m_run[MT], l_run[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int sr = 16 * (wave * RT + (DIFF ? mt >> 1 : mt)) + c;
    const int srt = sr / hc, srh = sr % hc;
    sact[mt] = srt < ntok && srh < nh;
    head[mt] = kvh * group + h0 + (sact[mt] ? srh : 0);
    trow[mt] = r0 + tok0 + (sact[mt] ? srt : 0);
    spos[mt] = p_first + srt;
    s_lo[mt] = window > 0 ? max(0, spos[mt] - window + 1) : 0;
    const unsigned short* src = proj + trow[mt] * proj_ld + ((long)head[mt] * kMaps + (DIFF ? mt & 1 : 0)) * dim;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (qvec) {  // rows and heads start at multiples of 8 elements: one 16-byte load (dim % 8 == 0)
        if (sact[mt] && 32 * ks + 8 * g < dim) v = *reinterpret_cast<const u16x8*>(src + 32 * ks + 8 * g);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int d = 32 * ks + 8 * g + e;
          if (sact[mt] && d < dim) v[e] = src[d];
        }
      }
      qf[mt][ks] = __builtin_bit_cast(bf16x8, v);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) acc[mt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[mt] = (sink && first_part) ? (sink_w != nullptr ? sink_w[head[mt]] * 1.44269504088896341f : 0.f) : -INFINITY;
    l_run[mt] = (sink && first_part) ? 1.f : 0.f;
  }
  // tile fill: kFT threads per key; key 16 a + 4 gg + b of the tile sits in column 8 gg + 4 a + b of the value tile
  const int fkey = tid / kFT, fk = tid % kFT;
  const int vcol = 8 * ((fkey >> 2) & 3) + 4 * (fkey >> 4) + (fkey & 3);
  const int kchunks = dim / 8, vchunks = vdim / 8;
  u16x8 kf[kKF], vf[kVF];
  auto fetch = [&](int u0) {
    const int j = key_of(u0 + fkey);
    const bool in = u0 + fkey <= hi;
    const long kr = in ? ((long)seq_bt[(long)s * bt_width + j / block_size] * block_size + j % block_size) * Dc : 0;
#pragma unroll
    for (int i = 0; i < kKF; ++i) {
      const int ch = fk + kFT * i;          // chunk ch % (4 KS) of map ch / (4 KS)
      const int mp = ch / (KS * 4), cw = ch % (KS * 4);
      kf[i] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (in && mp < kMaps && cw < kchunks) kf[i] = *reinterpret_cast<const u16x8*>(cache + kr + koff + mp * dim + 8 * cw);
    }
#pragma unroll
    for (int i = 0; i < kVF; ++i) {
      const int ch = fk + kFT * i;
      vf[i] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (in && ch < vchunks) vf[i] = *reinterpret_cast<const u16x8*>(cache + kr + voff + 8 * ch);
    }
  };
  if (lo <= hi) fetch(lo);
  for (int j0 = lo; j0 <= hi; j0 += kKeys) {
    __syncthreads();  // the previous tile's reads are done
#pragma unroll
    for (int i = 0; i < kKF; ++i) {
      const int ch = fk + kFT * i;
      if (ch < kMaps * KS * 4)
        *reinterpret_cast<u16x8*>(kt + (ch / (KS * 4)) * kKeys * kLd + fkey * kLd + 8 * (ch % (KS * 4))) = kf[i];
    }
#pragma unroll
    for (int i = 0; i < kVF; ++i) {
      const int ch = fk + kFT * i;
      if (ch < NV * 2) {
#pragma unroll
        for (int e = 0; e < 8; ++e) vt[(8 * ch + e) * kVLd + (vcol ^ ((ch & 3) << 3))] = vf[i][e];
      }
    }
    __syncthreads();
    if (j0 + kKeys <= hi) fetch(j0 + kKeys);  // the next tile's loads fly during this tile's math
    // S^T tiles: a = keys (16 per tile), b = 16 rows
    f32x4 sc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) sc[mt][0] = sc[mt][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        if constexpr (DIFF) {
#pragma unroll
          for (int mp = 0; mp < 2; ++mp) {  // map mp: its own key tile, shared by the wave's row tiles
            const bf16x8 a = __builtin_bit_cast(
                bf16x8, *reinterpret_cast<const u16x8*>(kt + mp * kKeys * kLd + (16 * nt + c) * kLd + 32 * ks + 8 * g));
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              sc[2 * rt + mp][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[2 * rt + mp][ks], sc[2 * rt + mp][nt], 0, 0, 0);
          }
        } else {
          const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u16x8*>(kt + (16 * nt + c) * kLd + 32 * ks + 8 * g));
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            sc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[mt][ks], sc[mt][nt], 0, 0, 0);
        }
      }
    }
    bf16x8 pb8[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      // scores in the log2 domain (scale2 = scale * log2 e). A tile that every row of the wave sees whole
      // (most tiles of a long window) skips the per-key visibility tests.
      float v[8];
      float mx = -INFINITY;
      const int ja = key_of(j0), jb = key_of(j0 + kKeys - 1);   // j0: the tile's first compacted index
      const bool whole = sact[mt] && j0 + kKeys - 1 <= hi && jb - ja == kKeys - 1 && jb <= spos[mt] &&
                         (ja >= s_lo[mt] || jb < keep);
      if (__all(whole)) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float x = sc[mt][e >> 2][e & 3];
          v[e] = softcap > 0.f ? cap2 * tanh_fast(x * icap) : x * scale2;
          mx = fmaxf(mx, v[e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int u = j0 + 16 * (e >> 2) + 4 * g + (e & 3);
          const int j = key_of(u);
          const bool vis = sact[mt] && u <= hi && j <= spos[mt] && (j >= s_lo[mt] || j < keep);
          const float x = sc[mt][e >> 2][e & 3];
          v[e] = vis ? (softcap > 0.f ? cap2 * tanh_fast(x * icap) : x * scale2) : -INFINITY;
          mx = fmaxf(mx, v[e]);
        }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mn = fmaxf(m_run[mt], mx);
      float sum = 0.f;
      u16x8 pk;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(v[e] - mn);  // -inf - mn: 0 (mn is finite whenever a key is seen)
        const unsigned short pb = f32_to_bf16(mn > -INFINITY ? p : 0.f);  // rounded to bf16: what is multiplied
        pk[e] = pb;
        sum += bf16_to_f32(pb);  // the sum of the weights that are actually multiplied
      }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      const float al = (mn > -INFINITY) ? __builtin_amdgcn_exp2f(m_run[mt] - mn) : 1.f;  // m_run = -inf: 0
      l_run[mt] = l_run[mt] * al + sum;
      m_run[mt] = mn;
      if (__any(al != 1.f)) {  // the running maxima settle after a few tiles: most tiles skip this
#pragma unroll
        for (int j = 0; j < NV; ++j) acc[mt][j] *= al;
      }
      pb8[mt] = __builtin_bit_cast(bf16x8, pk);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const bf16x8 a = __builtin_bit_cast(
          bf16x8, *reinterpret_cast<const u16x8*>(vt + (16 * j + c) * kVLd + 8 * (g ^ ((2 * j + (c >> 3)) & 3))));
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb8[mt], acc[mt][j], 0, 0, 0);
    }
  }
  // lane (c, g) holds value dims 16 j + 4 g .. + 3 of its rows
  if constexpr (DIFF) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int m0 = 2 * rt, m1 = 2 * rt + 1;   // the two maps of row tile rt
      if (!sact[m0]) continue;
      if (gridDim.z > 1) {
#pragma unroll
        for (int mp = 0; mp < 2; ++mp) {  // the runs of map mp live under "head" 2 head + mp
          const long wrow = ((long)blockIdx.z * heads * 2 + head[m0] * 2 + mp) * ws_rows + (trow[m0] - row_base);
          if (g == 0) { ws_ml[2 * wrow] = m_run[m0 + mp]; ws_ml[2 * wrow + 1] = l_run[m0 + mp]; }
#pragma unroll
          for (int j = 0; j < NV; ++j) {
            const int d = 16 * j + 4 * g;
            if (d < vdim) *reinterpret_cast<f32x4*>(ws_acc + wrow * vdim + d) = acc[m0 + mp][j];
          }
        }
        continue;
      }
      const float i0 = l_run[m0] > 0.f ? 1.f / l_run[m0] : 0.f, i1 = l_run[m1] > 0.f ? lam / l_run[m1] : 0.f;
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float o = acc[m0][j][e] * i0 - acc[m1][j][e] * i1;  // dims past vdim are zero (zero value rows)
          acc[m0][j][e] = o;
          ss += o * o;
        }
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      float f = out_scale * post / sqrtf(ss / (float)vdim + eps);
      if (gate_off >= 0) f *= sigmoid_f(bf16_to_f32(proj[trow[m0] * proj_ld + gate_off + head[m0]]));
      unsigned short* dst = out + trow[m0] * out_ld + (long)head[m0] * vdim;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int d = 16 * j + 4 * g;
        if (d >= vdim) continue;
        u16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = f32_to_bf16(acc[m0][j][e] * f);
        *reinterpret_cast<u16x4*>(dst + d) = o;
      }
    }
    return;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (!sact[mt]) continue;
    if (gridDim.z > 1) {
      const long wrow = ((long)blockIdx.z * heads + head[mt]) * ws_rows + (trow[mt] - row_base);
      if (g == 0) { ws_ml[2 * wrow] = m_run[mt]; ws_ml[2 * wrow + 1] = l_run[mt]; }
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int d = 16 * j + 4 * g;
        if (d < vdim) *reinterpret_cast<f32x4*>(ws_acc + wrow * vdim + d) = acc[mt][j];
      }
      continue;
    }
    float f = out_scale;
    if (gate_off >= 0) f *= sigmoid_f(bf16_to_f32(proj[trow[mt] * proj_ld + gate_off + head[mt]]));
    f = l_run[mt] > 0.f ? f / l_run[mt] : 0.f;
    unsigned short* dst = out + trow[mt] * out_ld + (long)head[mt] * vdim;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int d = 16 * j + 4 * g;
      if (d >= vdim) continue;  // vdim % 8 == 0: the four dims are inside together
      u16x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = f32_to_bf16(acc[mt][j][e] * f);
      *reinterpret_cast<u16x4*>(dst + d) = o;
    }
  }
}

// out[row_base + r, head] = sum_p acc_p e^(m_p - M) / sum_p l_p e^(m_p - M) * sigmoid(gate) * out_scale
constexpr int kMaxRuns = 64;
__global__ __launch_bounds__(128) void window_attention_reduce_kernel(
    unsigned short* __restrict__ out, long out_ld, const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
    const unsigned short* __restrict__ proj, long proj_ld, int gate_off, int nparts, int heads, int ws_rows,
    int row_base, int vdim, float out_scale) {
  __shared__ float sc[kMaxRuns];  // each run's weight e^(m_p - M) / L * gate * scale, 0 for empty runs
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  if (tid < 64) {  // one wave: run p on lane p
    const long w = ((long)min(tid, nparts - 1) * heads + h) * ws_rows + r;
    const float m = tid < nparts ? ws_ml[2 * w] : -INFINITY;
    const float l = tid < nparts ? ws_ml[2 * w + 1] : 0.f;
    const float M = wave_max(m);
    const float e = m > -INFINITY ? __builtin_amdgcn_exp2f(m - M) : 0.f;  // the runs' maxima are in the log2 domain
    const float L = wave_sum(l * e);
    float f = out_scale;
    if (gate_off >= 0) f *= sigmoid_f(bf16_to_f32(proj[(long)(row_base + r) * proj_ld + gate_off + h]));
    sc[tid] = L > 0.f ? e * f / L : 0.f;
  }
  __syncthreads();
  const long trow = row_base + r;
  for (int d = tid; d < vdim; d += 128) {
    float o = 0.f;
    for (int p = 0; p < nparts; ++p) o += ws_acc[(((long)p * heads + h) * ws_rows + r) * vdim + d] * sc[p];
    out[trow * out_ld + (long)h * vdim + d] = f32_to_bf16(o);
  }
}

// Two maps per head: the runs of map m of head h sit under workspace head 2 h + m (of 2 heads). Each map's runs
// are merged as above, then o = a1 - lam a2 and out = o / sqrt(mean(o^2) + eps) * post * gate * out_scale.
__global__ __launch_bounds__(128) void window_attention_diff_reduce_kernel(
    unsigned short* __restrict__ out, long out_ld, const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
    const unsigned short* __restrict__ proj, long proj_ld, int gate_off, int nparts, int heads, int ws_rows,
    int row_base, int vdim, float out_scale, float lam, float post, float eps) {
  __shared__ float sc[2][kMaxRuns];
  __shared__ float red[16];
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  {  // wave m: map m, run p on lane p
    const long w = ((long)min(lane, nparts - 1) * heads * 2 + 2 * h + wave) * ws_rows + r;
    const float m = lane < nparts ? ws_ml[2 * w] : -INFINITY;
    const float l = lane < nparts ? ws_ml[2 * w + 1] : 0.f;
    const float M = wave_max(m);
    const float e = m > -INFINITY ? __builtin_amdgcn_exp2f(m - M) : 0.f;
    const float L = wave_sum(l * e);
    sc[wave][lane] = L > 0.f ? e * (wave == 1 ? lam : 1.f) / L : 0.f;
  }
  __syncthreads();
  float o[2] = {0.f, 0.f};  // vdim <= 256: dims tid, tid + 128
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int d = tid + 128 * i;
    if (d < vdim) {
      for (int p = 0; p < nparts; ++p) {
        const long w0 = ((long)p * heads * 2 + 2 * h) * ws_rows + r;
        o[i] += ws_acc[w0 * vdim + d] * sc[0][p] - ws_acc[(w0 + ws_rows) * vdim + d] * sc[1][p];
      }
      ss += o[i] * o[i];
    }
  }
  ss = block_sum(ss, red);
  float f = out_scale * post / sqrtf(ss / (float)vdim + eps);
  const long trow = row_base + r;
  if (gate_off >= 0) f *= sigmoid_f(bf16_to_f32(proj[trow * proj_ld + gate_off + h]));
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int d = tid + 128 * i;
    if (d < vdim) out[trow * out_ld + (long)h * vdim + d] = f32_to_bf16(o[i] * f);
  }
}

template <int KS, int NV, int MT, bool DIFF>
void launch_mfma(unsigned short* out, long out_ld, const unsigned short* proj, long proj_ld, const unsigned short* cache,
                 int block_size, const int* seq_cu, const int* seq_ctx, const int* seq_bt, int bt_width, int seq0,
                 int seq1, int rows_bound, int heads, int kv_heads, int dim, int vdim, int gate_off, float scale,
                 int window, bool sink, float out_scale, int nparts, int part_keys, float* ws_acc, float* ws_ml,
                 int row_base, float lam, float post, float eps, int keep, float softcap, const float* sink_w,
                 hipStream_t s) {
  const int group = heads / kv_heads;
  const int rows = kRows * (DIFF ? MT / 2 : MT);
  const int hc = min(group, rows);
  const int hchunks = (group + hc - 1) / hc;
  // split rows (decode): one token per workgroup; else as many consecutive tokens as fit the rows
  const int tq = nparts > 1 ? 1 : rows / hc;
  // split rows are decode rows, one per sequence: workgroup x serves sequence seq0 + x
  const bool one_row_seqs = nparts > 1 && rows_bound == seq1 - seq0;
  const bool qvec = proj_ld % 8 == 0 && reinterpret_cast<uintptr_t>(proj) % 16 == 0;
  dim3 grid(one_row_seqs ? rows_bound : rows_bound / tq + (seq1 - seq0), kv_heads * hchunks, nparts);
  window_attention_mfma_kernel<KS, NV, MT, DIFF><<<grid, kThreads, 0, s>>>(
      out, out_ld, proj, proj_ld, cache, block_size, seq_cu, seq_ctx, seq_bt, bt_width, seq0, seq1, tq, hc, hchunks,
      heads, kv_heads, dim, vdim, gate_off, scale, window, sink, out_scale, part_keys, ws_acc, ws_ml, row_base,
      rows_bound, lam, post, eps, one_row_seqs, qvec, keep, softcap, sink_w);
  if (nparts > 1 && DIFF)
    window_attention_diff_reduce_kernel<<<dim3(rows_bound, heads), 128, 0, s>>>(
        out, out_ld, ws_acc, ws_ml, proj, proj_ld, gate_off, nparts, heads, rows_bound, row_base, vdim, out_scale, lam,
        post, eps);
  else if (nparts > 1)
    window_attention_reduce_kernel<<<dim3(rows_bound, heads), 128, 0, s>>>(out, out_ld, ws_acc, ws_ml, proj, proj_ld,
                                                                         gate_off, nparts, heads, rows_bound, row_base,
                                                                         vdim, out_scale);
}

}  // namespace

bool window_attention_mfma_ok(int dim, int vdim, long out_ld, long out_off, int maps) {
  const int cap = maps == 2 ? 128 : 256;  // two maps: the kernel variants with two row tiles per wave
  return dim % 8 == 0 && vdim % 8 == 0 && dim <= cap && vdim <= cap && out_ld % 4 == 0 && out_off % 4 == 0 &&
         (maps == 1 || maps == 2);
}

void launch_window_attention_mfma(void* out, long out_ld, const void* proj, long proj_ld, const void* cache,
                                  int block_size, const int* seq_cu, const int* seq_ctx, const int* seq_bt,
                                  int bt_width, int seq0, int seq1, int rows_bound, int heads, int kv_heads, int dim,
                                  int vdim, int gate_off, float scale, int window, bool sink, float out_scale,
                                  int nparts, int part_keys, float* ws_acc, float* ws_ml, int row_base, int maps,
                                  float lam, float post, float eps, int keep, float softcap, const float* sink_w,
                                  hipStream_t s) {
  if (seq1 <= seq0 || rows_bound <= 0) return;
#define HS_WA(KS, NV, MT, DIFF)                                                                                     \
  launch_mfma<KS, NV, MT, DIFF>((unsigned short*)out, out_ld, (const unsigned short*)proj, proj_ld,                  \
                                (const unsigned short*)cache, block_size, seq_cu, seq_ctx, seq_bt, bt_width, seq0,    \
                                seq1, rows_bound, heads, kv_heads, dim, vdim, gate_off, scale, window, sink,          \
                                out_scale, nparts, part_keys, ws_acc, ws_ml, row_base, lam, post, eps, keep, softcap,  \
                                sink_w, s)
  // two row tiles per wave where a prompt portion brings enough rows and the accumulators fit the registers
  const int ks = (dim + 31) / 32, nv = (vdim + 15) / 16;
  const bool wide = nparts == 1 && (long)rows_bound * (heads / kv_heads) >= 128 * (long)(seq1 - seq0);
  if (maps == 2) {
    // row tiles come in pairs (the two maps): 64 rows per workgroup. Four tiles per wave (128 rows) measured
    // slower on 4 x 2048-row prompts (532 against 396 us with 64-dim maps and 128-dim values): too many registers.
    if (ks <= 2 && nv <= 4) HS_WA(2, 4, 2, true);
    else if (ks <= 2) HS_WA(2, 8, 2, true);   // 64-dim maps over 128-dim values: no score products on padding
    else HS_WA(4, 8, 2, true);
    return;
  }
  if (ks <= 2 && nv <= 4) { if (wide) HS_WA(2, 4, 2, false); else HS_WA(2, 4, 1, false); }
  else if (ks <= 4 && nv <= 8) { if (wide) HS_WA(4, 8, 2, false); else HS_WA(4, 8, 1, false); }
  else HS_WA(8, 16, 1, false);
#undef HS_WA
}

}  // namespace hipserve
