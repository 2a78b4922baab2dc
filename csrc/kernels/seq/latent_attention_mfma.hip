// Latent attention for prompt portions on the matrix cores (bf16 activations and cache).
//
// latent_q_cat: the query rows the attention multiplies with the cached rows,
//   qc[h, t, :] = [ q_abs[h, t, :kv_rank] | RoPE(q[t, h, dim:]) ]  (bf16, Dk = kv_rank + rot_dim).
//
// latent_attention_mfma: a workgroup (4 waves) owns 64 (token, head) rows of one sequence, tokens
// consecutive, so all rows share one run of keys. Per 32-key tile:
//   1. the tile's cache rows [32][Dk] go to LDS row-major; wave w computes S = K . Q^T for its 16 rows
//      (mfma_f32_16x16x32_bf16, the Q operands stay in registers);
//   2. the same wave does the masked online softmax in fp32 on the scores in its registers (a row's 32
//      scores sit in four lanes) and writes P as bf16 to LDS for all waves;
//   3. every wave owns a slice of the latent dims for ALL 64 rows: acc = acc * alpha + V^T . P^T. The
//      contraction index is the key, so the V operand is read column-wise from the same row-major K
//      tile (eight 2-byte LDS reads per operand); the MFMA's k slots are dealt to the keys in the order the
//      score registers hold them, so P needs no shuffle.
// Decode rows (one token, many keys) split their keys over grid.z; latent_attention_reduce merges the
// runs' (max, sum, output).
// The output (latent space, times the head's sigmoid gate, over the softmax sum) is written as bf16.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

__global__ __launch_bounds__(256) void latent_q_cat_kernel(unsigned short* __restrict__ qc,
                                                           const float* __restrict__ q_abs,
                                                           const unsigned short* __restrict__ q,
                                                           const long* __restrict__ positions,
                                                           const float* __restrict__ inv_freq, int nfreq, int T,
                                                           int heads, int dim, int rot_dim, int kv_rank) {
  const int t = blockIdx.x, h = blockIdx.y;
  const int Dk = kv_rank + rot_dim;
  unsigned short* dst = qc + ((long)h * T + t) * Dk;
  const float* qa = q_abs + ((long)h * T + t) * kv_rank;
  if (q_abs != nullptr)  // else the absorbed part is already in qc (written by the absorption GEMM)
    for (int e = threadIdx.x; e < kv_rank; e += 256) dst[e] = f32_to_bf16(qa[e]);
  const unsigned short* qr = q + (long)t * heads * (dim + rot_dim) + (long)h * (dim + rot_dim) + dim;
  const float pos = (float)positions[t];
  for (int e = threadIdx.x; e < rot_dim; e += 256) {
    float v;
    if (e < 2 * nfreq) {
      const int i = e < nfreq ? e : e - nfreq;
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      const float u = bf16_to_f32(qr[i]), w = bf16_to_f32(qr[i + nfreq]);
      v = e < nfreq ? u * cs - w * sn : w * cs + u * sn;
    } else {
      v = bf16_to_f32(qr[e]);
    }
    dst[kv_rank + e] = f32_to_bf16(v);
  }
}

// (token, head) rows per workgroup = 16 x its waves NW (4: 64 rows)
constexpr int kKeys = 32;   // keys per tile
constexpr int kPLd = 40;    // P tile row stride (elements): 16-byte aligned rows, padded

HS_DEVICE bool find_tile64(const int* __restrict__ seq_cu, int seq0, int seq1, int tq, int wg, int& s, int& tok0) {
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

// K tile row stride: 32 KS + 8 elements (16-byte aligned rows; stride / 2 = 4 (mod 16) dwords keeps both the
// row-wise 16-byte operand reads of S and the column-wise 2-byte reads of P . V at two-way bank conflicts).
template <int KS> struct KtLd { static constexpr int v = KS * 32 + 8; };

// KS: 32-dim steps of a cache row (Dk <= 32 KS); NPW: 16-dim output tiles per wave (kv_rank <= 64 NPW).
// grid.z > 1 splits the keys of a row into runs of part_keys; the runs' unnormalised outputs and
// (max, sum) go to ws_acc / ws_ml for latent_attention_reduce (decode rows: many keys, few rows).
template <int KS, int NPW, int NW>
__global__ __launch_bounds__(64 * NW, 2) void latent_attention_mfma_kernel(
    unsigned short* __restrict__ o_lat, const unsigned short* __restrict__ qc, const unsigned short* __restrict__ proj,
    long proj_ld, const unsigned short* __restrict__ cache, int block_size, const int* __restrict__ seq_cu,
    const int* __restrict__ seq_ctx, const int* __restrict__ seq_bt, int bt_width, int seq0, int seq1, int tq, int hc,
    int T_rows, int heads, int rot_dim, int kv_rank, int gate_off, float scale, int window, int part_keys,
    float* __restrict__ ws_acc, float* __restrict__ ws_ml, int row_base, int ws_rows) {
  constexpr int kLd = KtLd<KS>::v;
  constexpr int kRows = 16 * NW, kThreads = 64 * NW, kFT = kThreads / kKeys;  // kFT threads fill one key's row
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned short* kt = reinterpret_cast<unsigned short*>(smem);                    // [32][kLd] bf16 cache rows
  unsigned short* p_lds = kt + kKeys * kLd;                                        // [rows][kPLd] bf16, MFMA k order
  float* alpha = reinterpret_cast<float*>(p_lds + kRows * kPLd);                   // [rows]
  float* m_lds = alpha + kRows;                                                    // [rows] (epilogue)
  float* l_lds = m_lds + kRows;                                                    // [rows] (epilogue)
  int s, tok0;
  // (workgroups are dealt to the XCDs round-robin; giving each XCD a contiguous run of token tiles was
  // measured slower, 1188 vs 1013 us at 8192 tokens x 16 heads: the causal start makes the runs unequal)
  if (!find_tile64(seq_cu, seq0, seq1, tq, blockIdx.x, s, tok0)) return;
  const int Dk = kv_rank + rot_dim;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int r0 = seq_cu[s], n = seq_cu[s + 1] - r0, ctx = seq_ctx[s];
  const int ntok = min(tq, n - tok0);
  const int h0 = blockIdx.y * hc, nh = min(hc, heads - h0);
  const int p_first = ctx - n + tok0, p_last = p_first + ntok - 1;
  const int lo_all = window > 0 ? max(0, p_first - window + 1) : 0;
  const int lo = lo_all + blockIdx.z * part_keys;
  const int hi = gridDim.z > 1 ? min(p_last, lo + part_keys - 1) : p_last;
  // Q operands of this wave's 16 rows (row = 16 wave + c): dims 32 ks + 8 g .. + 7
  bf16x8 qf[KS];
  {
    const int r = 16 * wave + c;
    const int rt = r / hc, rh = r % hc;
    const bool act = rt < ntok && rh < nh;
    const unsigned short* src = qc + ((long)(h0 + (act ? rh : 0)) * T_rows + r0 + tok0 + (act ? rt : 0)) * Dk;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 32 * ks + 8 * g;
      u16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (act && d < Dk) v = *reinterpret_cast<const u16x8*>(src + d);
      qf[ks] = __builtin_bit_cast(bf16x8, v);
    }
  }
  f32x4 acc[NW][NPW];
#pragma unroll
  for (int mt = 0; mt < NW; ++mt)
#pragma unroll
    for (int j = 0; j < NPW; ++j) acc[mt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int ntiles_dv = (kv_rank + 15) / 16;
  const int chunks = Dk / 8;  // 16-byte chunks of a cache row
  // tile fill: kFT threads per key, each its key's chunks fk, fk + kFT, ...
  const int fkey = tid / kFT, fk = tid % kFT;
  // softmax: the wave that computed a row's scores keeps them; lane (c, g) owns row 16 wave + c and the keys
  // 16 nt + 4 g + i of a tile (nt = 0, 1; i = 0..3) = the MFMA k slot (g, e = 4 nt + i) of P . V below
  const int sr = 16 * wave + c;
  const int srt = sr / hc, srh = sr % hc;
  const bool sact = srt < ntok && srh < nh;
  const int spos = p_first + srt;
  const int s_lo = window > 0 ? max(0, spos - window + 1) : 0;
  float m_run = -INFINITY, l_run = 0.f;
  constexpr int kFill = (KS * 4 + kFT - 1) / kFT;
  u16x8 fv[kFill];
  // the thread's part of a tile, all loads in flight together; zero past Dk and past the last key
  auto fetch = [&](int j0) {
    const int j = j0 + fkey;
    const bool in = j <= hi;
    const long kr = in ? ((long)seq_bt[(long)s * bt_width + j / block_size] * block_size + j % block_size) * Dk : 0;
#pragma unroll
    for (int i = 0; i < kFill; ++i) {
      const int ch = fk + kFT * i;
      fv[i] = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (in && ch < chunks) fv[i] = *reinterpret_cast<const u16x8*>(cache + kr + 8 * ch);
    }
  };
  for (int j0 = lo; j0 <= hi; j0 += kKeys) {
    fetch(j0);        // (prefetching a tile ahead costs 40 registers and the second workgroup per CU)
    __syncthreads();  // the previous tile's reads of the K tile (P . V) are done
#pragma unroll
    for (int i = 0; i < kFill; ++i) {
      const int ch = fk + kFT * i;
      if (ch < KS * 4) *reinterpret_cast<u16x8*>(kt + fkey * kLd + 8 * ch) = fv[i];
    }
    __syncthreads();
    // 1. S^T tiles: a = keys (16 per tile), b = this wave's 16 query rows
    f32x4 sc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const u16x8 a = *reinterpret_cast<const u16x8*>(kt + (16 * nt + c) * kLd + 32 * ks + 8 * g);
        sc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), qf[ks], sc[nt], 0, 0, 0);
      }
    }
    // 2. online softmax in fp32 on the scores in registers (lane (c, g): keys 16 nt + 4 g + i of row sr; the
    //    row's four lanes meet through two shuffles); P as bf16 in the k order of the MFMA below
    {
      float v[8];
      float mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = j0 + 16 * (e >> 2) + 4 * g + (e & 3);
        const bool vis = sact && j <= hi && j <= spos && j >= s_lo;
        v[e] = vis ? sc[e >> 2][e & 3] * scale : -INFINITY;
        mx = fmaxf(mx, v[e]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mn = fmaxf(m_run, mx);
      float sum = 0.f;
      u16x8 pk;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = (v[e] > -INFINITY) ? __expf(v[e] - mn) : 0.f;  // rounded to bf16 right below
        const unsigned short pb = f32_to_bf16(p);
        pk[e] = pb;
        sum += bf16_to_f32(pb);  // the sum of the weights that are actually multiplied
      }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      *reinterpret_cast<u16x8*>(p_lds + sr * kPLd + 8 * g) = pk;
      const float al = (mn > -INFINITY) ? __expf(m_run - mn) : 1.f;  // m_run = -inf: 0
      if (g == 0) alpha[sr] = al;
      l_run = l_run * al + sum;
      m_run = mn;
    }
    __syncthreads();
    // 3. acc[rows][dims] = acc * alpha + V^T . P^T: a = 16 latent dims, b = 16 rows; the MFMA's k slot
    //    (g, e) is key 16 (e / 4) + 4 g + e % 4, read column-wise from the row-major K tile
    bf16x8 pb[NW];
    float al[NW];
    bool rescale = false;
#pragma unroll
    for (int mt = 0; mt < NW; ++mt) {
      pb[mt] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u16x8*>(p_lds + (16 * mt + c) * kPLd + 8 * g));
      al[mt] = alpha[16 * mt + c];
      rescale |= al[mt] != 1.f;
    }
    if (__any(rescale)) {  // the running maxima settle after a few tiles: most tiles skip this
#pragma unroll
      for (int j = 0; j < NPW; ++j)
#pragma unroll
        for (int mt = 0; mt < NW; ++mt) acc[mt][j] *= al[mt];
    }
#pragma unroll
    for (int j = 0; j < NPW; ++j) {
      const int nt = wave + NW * j;
      if (nt < ntiles_dv) {
        u16x8 a;
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] = kt[(16 * (e >> 2) + 4 * g + (e & 3)) * kLd + 16 * nt + c];
#pragma unroll
        for (int mt = 0; mt < NW; ++mt)
          acc[mt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), pb[mt], acc[mt][j], 0, 0, 0);
      }
    }
  }
  if (g == 0) { m_lds[sr] = m_run; l_lds[sr] = l_run; }
  __syncthreads();
  const bool partial = gridDim.z > 1;
  if (tid < kRows) {  // alpha <- gate / softmax sum of the row (1 for partial results)
    const int rt = tid / hc, rh = tid % hc;
    const bool act = rt < ntok && rh < nh;
    float f = 0.f;
    if (act && partial) {
      f = 1.f;
      const long wrow = (long)blockIdx.z * heads * ws_rows + (long)(h0 + rh) * ws_rows + (r0 + tok0 + rt - row_base);
      ws_ml[2 * wrow] = m_lds[tid];
      ws_ml[2 * wrow + 1] = l_lds[tid];
    } else if (act && l_lds[tid] > 0.f) {
      f = 1.f / l_lds[tid];
      if (gate_off >= 0) f *= sigmoid_f(bf16_to_f32(proj[(long)(r0 + tok0 + rt) * proj_ld + gate_off + h0 + rh]));
    }
    alpha[tid] = f;
  }
  __syncthreads();
  // lane (c, g) holds latent dims 16 nt + 4 g .. + 3 of row 16 mt + c
#pragma unroll
  for (int mt = 0; mt < NW; ++mt) {
    const int r = 16 * mt + c;
    const int rt = r / hc, rh = r % hc;
    if (!(rt < ntok && rh < nh)) continue;
    const float f = alpha[r];
    const long trow = r0 + tok0 + rt;
#pragma unroll
    for (int j = 0; j < NPW; ++j) {
      const int d = 16 * (wave + NW * j) + 4 * g;
      if (d >= kv_rank) continue;  // kv_rank % 8 == 0: the four dims are inside together
      if (partial) {
        float* dst = ws_acc + (((long)blockIdx.z * heads + h0 + rh) * ws_rows + (trow - row_base)) * kv_rank + d;
        *reinterpret_cast<f32x4*>(dst) = acc[mt][j];
      } else {
        u16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = f32_to_bf16(acc[mt][j][e] * f);
        *reinterpret_cast<u16x4*>(o_lat + ((long)(h0 + rh) * T_rows + trow) * kv_rank + d) = o;
      }
    }
  }
}

// o_lat[h, row_base + r, :] = sum_p acc_p e^(m_p - M) / sum_p l_p e^(m_p - M) * sigmoid(gate)
constexpr int kMaxRuns = 64;
__global__ __launch_bounds__(128) void latent_attention_reduce_kernel(
    unsigned short* __restrict__ o_lat, const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
    const unsigned short* __restrict__ proj, long proj_ld, int gate_off, int nparts, int heads, int ws_rows,
    int row_base, int T_rows, int kv_rank) {
  __shared__ float sc[kMaxRuns];  // each run's weight e^(m_p - M) / L * gate, 0 for empty runs
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  if (tid < 64) {  // one wave: run p on lane p
    const long w = ((long)min(tid, nparts - 1) * heads + h) * ws_rows + r;
    const float m = tid < nparts ? ws_ml[2 * w] : -INFINITY;
    const float l = tid < nparts ? ws_ml[2 * w + 1] : 0.f;
    const float M = wave_max(m);
    const float e = m > -INFINITY ? __expf(m - M) : 0.f;
    const float L = wave_sum(l * e);
    const float gate = gate_off >= 0 ? sigmoid_f(bf16_to_f32(proj[(long)(row_base + r) * proj_ld + gate_off + h])) : 1.f;
    sc[tid] = L > 0.f ? e * gate / L : 0.f;
  }
  __syncthreads();
  const long trow = row_base + r;
  for (int d = tid; d < kv_rank; d += 128) {
    float o = 0.f;
    for (int p = 0; p < nparts; ++p) o += ws_acc[(((long)p * heads + h) * ws_rows + r) * kv_rank + d] * sc[p];
    o_lat[((long)h * T_rows + trow) * kv_rank + d] = f32_to_bf16(o);
  }
}

template <int KS, int NPW, int NW>
bool launch_mfma(unsigned short* o_lat, const unsigned short* qc, const unsigned short* proj, long proj_ld,
                 const unsigned short* cache, int block_size, const int* seq_cu, const int* seq_ctx, const int* seq_bt,
                 int bt_width, int seq0, int seq1, int rows_bound, int T, int heads, int rot_dim, int kv_rank,
                 int gate_off, float scale, int window, int nparts, int part_keys, float* ws_acc, float* ws_ml,
                 int row_base, hipStream_t s) {
  constexpr int kLd = KtLd<KS>::v, kRows = 16 * NW;
  constexpr size_t smem = kKeys * kLd * 2 + kRows * kPLd * 2 + 3 * kRows * 4;
  static_assert(smem <= 160 * 1024, "LDS");
  auto* fn = &latent_attention_mfma_kernel<KS, NPW, NW>;
  if (smem > 64 * 1024) {  // once per kernel: more dynamic LDS than the default limit
    static const bool ok = hipFuncSetAttribute(reinterpret_cast<const void*>(fn),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) == hipSuccess;
    if (!ok) return false;
  }
  const int hc = min(heads, kRows);
  // split rows (decode): one token per workgroup; else as many consecutive tokens as fit the rows
  const int tq = nparts > 1 ? 1 : kRows / hc;
  dim3 grid(rows_bound / tq + (seq1 - seq0), (heads + hc - 1) / hc, nparts);
  fn<<<grid, 64 * NW, smem, s>>>(o_lat, qc, proj, proj_ld, cache, block_size, seq_cu, seq_ctx, seq_bt, bt_width, seq0, seq1,
                                tq, hc, T, heads, rot_dim, kv_rank, gate_off, scale, window, part_keys, ws_acc, ws_ml,
                                row_base, rows_bound);
  if (nparts > 1)
    latent_attention_reduce_kernel<<<dim3(rows_bound, heads), 128, 0, s>>>(o_lat, ws_acc, ws_ml, proj, proj_ld, gate_off,
                                                                         nparts, heads, rows_bound, row_base, T,
                                                                         kv_rank);
  return true;
}

}  // namespace

void launch_latent_q_cat(void* qc, const float* q_abs, const void* q, const long* positions, const float* inv_freq,
                         int nfreq, int T, int heads, int dim, int rot_dim, int kv_rank, hipStream_t s) {
  if (T <= 0) return;
  latent_q_cat_kernel<<<dim3(T, heads), 256, 0, s>>>((unsigned short*)qc, q_abs, (const unsigned short*)q, positions,
                                                     inv_freq, nfreq, T, heads, dim, rot_dim, kv_rank);
}

bool latent_attention_mfma_ok(int kv_rank, int rot_dim) {
  const int Dk = kv_rank + rot_dim;
  return kv_rank % 8 == 0 && rot_dim % 8 == 0 && kv_rank <= 512 && Dk <= 640;
}

void launch_latent_attention_mfma(void* o_lat, const void* qc, const void* proj, long proj_ld, const void* cache,
                                  int block_size, const int* seq_cu, const int* seq_ctx, const int* seq_bt,
                                  int bt_width, int seq0, int seq1, int rows_bound, int T, int heads, int rot_dim,
                                  int kv_rank, int gate_off, float scale, int window, int nparts, int part_keys,
                                  float* ws_acc, float* ws_ml, int row_base, hipStream_t s) {
  if (seq1 <= seq0 || rows_bound <= 0) return;
  const int Dk = kv_rank + rot_dim;
#define HS_LA(KS, NPW, NW)                                                                                          \
  launch_mfma<KS, NPW, NW>((unsigned short*)o_lat, (const unsigned short*)qc, (const unsigned short*)proj, proj_ld,  \
                           (const unsigned short*)cache, block_size, seq_cu, seq_ctx, seq_bt, bt_width, seq0, seq1,   \
                           rows_bound, T, heads, rot_dim, kv_rank, gate_off, scale, window, nparts, part_keys, ws_acc, \
                           ws_ml, row_base, s)
  // (an 8-wave / 128-row variant, NW = 8, halves the tile fetches per row but was not faster: 1107 vs 1019 us
  // at 8192 tokens x 16 heads, its 512-thread launch bound caps it at 128 registers and it spills)
  if (kv_rank <= 128 && Dk <= 192) HS_LA(6, 2, 4);
  else if (kv_rank <= 256 && Dk <= 320) HS_LA(10, 4, 4);
  else HS_LA(20, 8, 4);
#undef HS_LA
}

}  // namespace hipserve
