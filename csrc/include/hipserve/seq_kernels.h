// Launchers of the layer-list decoders' kernels (csrc/kernels/seq/*.hip): grouped RMSNorm
// fused with the scaled residual update, latent attention on a paged latent cache, the
// minGRU scan over state slots, and the table-routed experts' GEMMs. Every launcher has a
// bf16 and a true fp32 build (``f32``): the activations' element type; norms, scores,
// softmax, recurrences and the residual stream are fp32 in both.
#pragma once
#include <hip/hip_runtime.h>

namespace hipserve {

// residual[T, H] (fp32, in place) += ls1 * mix + ls2 * (1/top) * sum_j y[pair_slot[t*top+j]] + extra;
// out = residual normalised in `groups` consecutive parts, times w (fp32 [H]). Null inputs are skipped.
void launch_scaled_add_group_rmsnorm(void* out, float* residual, const float* w, int T, int H, int groups, float eps,
                                     const void* mix, const float* ls1, const void* y, const int* pair_slot, int top,
                                     const float* ls2, const void* extra, bool f32, hipStream_t s);

// proj[T, ld] rows = [q latent (q_rank) | kv latent (kv_rank) | rotary key (rot_dim) | ...]:
// cq[T, q_rank] = RMSNorm(q latent) * q_norm; cache row slots[t] (>= 0) = [RMSNorm(kv latent) * kv_norm |
// RoPE(rotary key)], rotate-half over the first 2 * nfreq dims with angle pos * inv_freq[i].
void launch_latent_prepare(void* cq, void* cache, const void* proj, long ld, const long* positions, const long* slots,
                           const float* q_norm, const float* kv_norm, const float* inv_freq, int nfreq, int T,
                           int q_rank, int kv_rank, int rot_dim, float eps, bool f32, hipStream_t s);

// Attention of every (token, head) row on the cached latents of its sequence; sequences
// seq0 .. seq1-1 of the step, `tq` tokens per workgroup. o_lat[heads, T, kv_rank] gets the
// latent-space output times sigmoid(proj[t, gate_off + h]).
void launch_latent_attention(void* o_lat, const float* q_abs, const void* q, const void* proj, long proj_ld,
                             const void* cache, int block_size, const int* seq_cu, const int* seq_ctx,
                             const int* seq_bt, int bt_width, int seq0, int seq1, int rows_bound, int tq,
                             const float* inv_freq, int nfreq, int T, int heads, int dim, int rot_dim, int kv_rank,
                             int gate_off, float scale, int window, bool f32, hipStream_t s);

// bf16 prompt portions on the matrix cores (latent_attention_mfma.hip): qc[heads, T, kv_rank + rot_dim] =
// [q_abs | RoPE(q rotary part)] as bf16, then the attention on 64-row x 32-key MFMA tiles. nparts > 1
// (rows of one token each, rows_bound of them from batch row row_base on): the keys are split into runs of
// part_keys (a multiple of 32) over ws_acc [nparts, heads, rows_bound, kv_rank] / ws_ml [.., 2] and merged.
void launch_latent_q_cat(void* qc, const float* q_abs, const void* q, const long* positions, const float* inv_freq,
                         int nfreq, int T, int heads, int dim, int rot_dim, int kv_rank, hipStream_t s);
bool latent_attention_mfma_ok(int kv_rank, int rot_dim);
void launch_latent_attention_mfma(void* o_lat, const void* qc, const void* proj, long proj_ld, const void* cache,
                                  int block_size, const int* seq_cu, const int* seq_ctx, const int* seq_bt,
                                  int bt_width, int seq0, int seq1, int rows_bound, int T, int heads, int rot_dim,
                                  int kv_rank, int gate_off, float scale, int window, int nparts, int part_keys,
                                  float* ws_acc, float* ws_ml, int row_base, hipStream_t s);

// minGRU over the step's rows of every sequence, from / to its fp32 state slot.
void launch_mingru_scan(void* y, float* state, const void* proj, const float* b_z, const float* b_x,
                        const int* seq_cu, const int* seq_ctx, const int* seq_state, int nseq, int width, int max_q,
                        bool f32, hipStream_t s);

// out[slot, N] = act(W[e(tile)] [N, K] . x[row(slot)]) over moe_align tiles of `tile` slots; tiles whose
// expert is < 0 or >= E (no weights) are skipped. act 0: none, 1: squared ReLU, 2: W[e] = [gate rows; up rows]
// and out[slot, N / 2] = silu(gate) * up.
void launch_expert_gemm(void* out, const void* x, long x_ld, const void* w, const int* slots, const int* tile_expert,
                        int ntiles_cap, int tile, int gather_k, int N, int K, int act, int E, bool f32,
                        hipStream_t s);

// Residual update with the norm on the sublayer's output (group_norm.hip): residual[T, H] (fp32, in place) +=
// y / sqrt(mean(y^2) + eps) * w; out = residual in the activation type. y null: the addend is a mixture's output,
// shared (or 0) + sum_j wts[t, j] * (ids[t, j] < E ? ye[pair_slot[t * top + j]] : h[t]).
void launch_add_normed(void* out, float* residual, const float* w, int T, int H, float eps, const void* y,
                       const void* ye, const int* pair_slot, const int* ids, const float* wts, int top, int E,
                       const void* h, const void* shared, bool f32, hipStream_t s);

// Softmax router (router.hip): s = softmax(logits[T, n]); the `top` largest s + correction are chosen (ties: the
// lower index); ids[T, top] = min(index, E), wts[T, top] = s * scale. groups > 1: only outputs of the `keep`
// groups (of n / groups neighbours) with the largest s + correction can be chosen; renorm: the chosen s are
// divided by their sum + 1e-20 first.
int route_topk_max_outputs();
void launch_route_topk(int* ids, float* wts, const float* logits, const float* correction, int T, int n, int top,
                       float scale, int E, int groups, int keep, bool renorm, hipStream_t s);

// Window attention on a paged cache [blocks, block_size, kv_heads * dim | kv_heads * vdim] (window_attention.hip).
// attn_prepare: per row of proj = [q | k | v | ...]: optional RMS norm of q and k (norm_mode 0: none; 1: over the
// whole projection, weights per element; 2: per head - and map - of `dim` elements, one weight of `dim` elements),
// rotate-half rotation of the first 2 * nfreq dims per head, optional per-head unit-rms values; q in place, k / v
// into cache row slots[t] (>= 0). `maps` query / key maps per head (rows hold heads * maps * dim query and
// kv_heads * maps * dim key elements). cache null: the rows are [q | ...] and only q is prepared.
void launch_attn_prepare(void* proj, long ld, void* cache, const long* positions, const long* slots,
                         const float* inv_freq, int nfreq, int T, int heads, int kv_heads, int maps, int dim, int vdim,
                         const float* q_norm, const float* k_norm, int norm_mode, bool v_norm, float eps, bool f32,
                         hipStream_t s);
// Sequences seq0 .. seq1-1 of the step, `tq` tokens per workgroup: keys 0 <= pos - j < window (0: all) or
// j < keep, scores q . k * scale, through softcap * tanh(. / softcap) when softcap > 0,
// weights exp(s_j) / (sink + sum exp) with sink = exp(sink_w[h]) (1 when sink_w is null),
// head output times sigmoid(proj[t, gate_off + h]) (gate_off >= 0) and
// out_scale into out[t * out_ld + h * vdim ..]. maps = 2 (differential attention): queries and keys hold
// [map 1 | map 2] per head; the head output is o = a1 - lam a2, o / sqrt(mean(o^2) + eps) * post.
int window_attention_max_vdim();
void launch_window_attention(void* out, long out_ld, const void* proj, long proj_ld, const void* cache, int block_size,
                             const int* seq_cu, const int* seq_ctx, const int* seq_bt, int bt_width, int seq0, int seq1,
                             int rows_bound, int tq, int heads, int kv_heads, int dim, int vdim, int gate_off,
                             float scale, int window, bool sink, float out_scale, int maps, float lam, float post,
                             float eps, int keep, float softcap, const float* sink_w, bool f32, hipStream_t s);

// bf16 on the matrix cores (window_attention_mfma.hip): 64 (token, head) rows of one key/value head per
// workgroup, 32-key tiles. nparts > 1 (rows of one token each, rows_bound of them from batch row row_base on):
// the keys are split into runs of part_keys (a multiple of 32) over ws_acc [nparts, heads, rows_bound, vdim] /
// ws_ml [.., 2] and merged (two maps: the workspaces hold 2 * heads "heads"). out_off: element offset of `out`
// in its allocation (alignment of the stores).
bool window_attention_mfma_ok(int dim, int vdim, long out_ld, long out_off, int maps);
void launch_window_attention_mfma(void* out, long out_ld, const void* proj, long proj_ld, const void* cache,
                                  int block_size, const int* seq_cu, const int* seq_ctx, const int* seq_bt,
                                  int bt_width, int seq0, int seq1, int rows_bound, int heads, int kv_heads, int dim,
                                  int vdim, int gate_off, float scale, int window, bool sink, float out_scale,
                                  int nparts, int part_keys, float* ws_acc, float* ws_ml, int row_base, int maps,
                                  float lam, float post, float eps, int keep, float softcap, const float* sink_w,
                                  hipStream_t s);

// Delta-rule recurrences over state slots (delta_scan.hip). scratch: fp32, T * (2 * kv_heads * dim +
// 2 * heads * vdim + 2 * heads) floats for the gated rule, T * 7 * heads * dim for the generalized one.
int delta_max_dim();
int delta_max_taps();
void launch_gated_delta(void* y, float* S, float* conv_state, const void* proj, long ld, const float* conv_w,
                        const float* a_log, const float* dt_bias, const float* norm_w, const int* seq_cu,
                        const int* seq_ctx, const int* seq_state, int nseq, int T, float* scratch, int heads,
                        int kv_heads, int dim, int vdim, int taps, float eps, bool f32, hipStream_t s);
void launch_delta_rule(void* out, long out_ld, float* S, const void* proj, long ld, const float* wl, const float* a_b,
                       const float* w0, const float* norm_w, const int* seq_cu, const int* seq_ctx,
                       const int* seq_state, int nseq, int T, float* scratch, int heads, int dim, float eps,
                       float out_scale, bool f32, hipStream_t s);
// Token shift: out[nb, T, H] (activation type) = x + (previous row - x) * mu[b] from the 32-bit rows x; a
// sequence's row before the step comes from state[slot] (zeros at position 0), which then gets the step's last row.
void launch_token_shift(void* out, const float* x, float* state, const float* mu, const int* seq_cu,
                        const int* seq_ctx, const int* seq_state, int nseq, int T, int H, int nb, bool f32,
                        hipStream_t s);
// Linear attention with per-channel decays: proj [4, T, heads * dim] = r, k, v, gate; wl fp32 [T, heads * dim];
// scratch: T * (5 * heads * dim + heads) floats.
void launch_wkv(void* out, float* S, const void* proj, const float* wl, const float* w0, const float* u,
                const float* norm_w, const int* seq_cu, const int* seq_ctx, const int* seq_state, int nseq, int T,
                float* scratch, int heads, int dim, float eps, bool f32, hipStream_t s);
// The same for steps in which every sequence has ONE row, in one launch: low [T, rank] is the decay bottleneck's
// output BEFORE its tanh, w2 [heads * dim, rank] its up-projection; dim <= 256.
void launch_wkv_step(void* out, float* S, const void* proj, long T, const void* low, const void* w2, int rank,
                     const float* w0, const float* u, const float* norm_w, const int* seq_cu, const int* seq_ctx,
                     const int* seq_state, int nseq, int heads, int dim, float eps, bool f32, hipStream_t s);
// kind 0: tanh; 1: c0 z^2 + z/2 (z > 0), c1 (exp(z) - 1 - z) + z/2 (z <= 0); 2: max(z, 0)^2;
// 3: x rows = [gate | up] of `cols` each, out = silu(gate) * up.
void launch_activation(void* out, long out_ld, const void* x, long x_ld, int rows, int cols, int kind, float c0,
                       float c1, bool f32, hipStream_t s);

// Per row z of x: out = a N(z) + b N(z^2) + c N(z^3) + e, N(u) = u / sqrt(mean(u^2) + eps), coef = [a, b, c, e].
void launch_polynorm(void* out, long out_ld, const void* x, long x_ld, int rows, int cols, const float* coef,
                     float eps, bool f32, hipStream_t s);
// out[t, h * d + j] = x[h, t, j] * sigmoid(gate[t * gate_ld + h * d + j]) for x [heads, rows, d].
void launch_gate_mul(void* out, const void* x, const void* gate, long gate_ld, int rows, int heads, int d, bool f32,
                     hipStream_t s);

// Parallel block with gated sublayer results and the next norms (gated_block.hip): residual[T, H] (fp32, in place)
// += sigmoid(g1 + b1) * y1 + sigmoid(g2 + b2) * y2, y2 a row or (y2 null) shared + sum_j wts[t, j] ye[pair_slot[t top + j]];
// out1 = residual / rms * w1, out2 (may be null) = residual / rms * w2; w1n / w2n: 1 or H weights.
void launch_gated_add_norms(void* out1, void* out2, float* residual, const float* w1, int w1n, const float* w2, int w2n,
                            int T, int H, float eps, const void* y1, const void* g1, long g1_ld, const float* b1,
                            const void* y2, const void* g2, long g2_ld, const float* b2, const void* ye,
                            const int* pair_slot, const float* wts, int top, const void* shared, bool f32,
                            hipStream_t s);

// mLSTM matrix memory over state slots (mlstm.hip): proj rows = [q | k | v | gate | ...], gates fp32 [T, 2 heads] =
// [input | forget] pre-activations, b_if their biases, S [slots, heads, dim, vdim], N [slots, heads, dim],
// M [slots, heads]; scratch: T * heads * (2 dim + 2 vdim + 6) floats. one_row_seqs: every sequence brings one row.
int mlstm_max_dim();
void launch_mlstm(void* out, float* S, float* N, float* M, const void* proj, long ld, const float* gates,
                  const float* b_if, const float* norm_w, const int* seq_cu, const int* seq_ctx, const int* seq_state,
                  int nseq, int T, float* scratch, int heads, int dim, int vdim, float cap, float eps,
                  bool one_row_seqs, bool f32, hipStream_t s);

}  // namespace hipserve
