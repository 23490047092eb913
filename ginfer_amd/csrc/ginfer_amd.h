// Entry points of the kernel libraries of ginfer_amd (gfx950), for callers outside Python.
//
// Every source under this folder is built into a shared library of its own (lib<source>.so; the matrix-core
// attention once per head size, libattention_mfma_HEAD_DIM<n>.so).  All entry points are `extern "C"`, take raw
// device pointers and the stream to launch on, check what can be checked on the host, and return 0 or a
// negative number without launching anything.  Sizes are in elements unless bytes are named.  bfloat16 values
// are raw 16-bit patterns.  Nothing here allocates device memory: scratch memory is the caller's (or, for
// ga_sample_rows_static, a static array of the library).
//
// Every source includes this header, so the compiler checks each definition against its declaration.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// ---- embedding.hip: out float [tokens, hidden] = table[ids] (table bfloat16 or float, ids int32)
int ga_embedding_gather(void* out, const void* table, const void* ids, int tokens, int hidden, int is_bf16,
                        hipStream_t stream);

// ---- norm.hip: residual float [num_tokens, hidden] += delta (null, [num_tokens, hidden], or float partial sums
// [delta_parts, num_tokens, hidden] added in order); out = rmsnorm(residual) * gain for all rows, or for the
// int32 `rows` alone (then the residual is left as it is)
int ga_add_rmsnorm(void* out, void* residual, const void* delta, int delta_parts, int num_tokens, const void* gain,
                   const void* rows, int num_rows, int hidden, float eps, int is_bf16, int gain_is_f32,
                   hipStream_t stream);

// ---- rope_kv.hip: NeoX rotation of q and k inside the fused projection [tokens, (nh + 2 nkv) hd], k and v
// written to the pages (keys [page][kv head][slot][dim], values [page][kv head][dim][slot]); slot_mapping int64,
// -1: no write
int ga_rope_kv_write(void* qkv, const void* positions, const void* cos_t, const void* sin_t, const void* slot_mapping,
                     void* k_pages, void* v_pages, int tokens, int nh, int nkv, int hd, int rotary_dim, int page_size,
                     int write_kv, int is_bf16, hipStream_t stream);
// the same on 32-bit partial sums of the projection, parts [n_parts][tokens][(nh + 2 nkv) hd] added in order, then the bias
// (bfloat16 or null): q to q_out [tokens][nh hd] in bfloat16, k and v into the pages
int ga_rope_kv_from_parts(void* q_out, const void* parts, int n_parts, const void* bias, const void* positions,
                          const void* cos_t, const void* sin_t, const void* slot_mapping, void* k_pages, void* v_pages,
                          int tokens, int nh, int nkv, int hd, int rotary_dim, int page_size, int write_kv,
                          hipStream_t stream);

// ---- gemm.hip: C [M, N] = A [M, K] . W [N, K]^T + bias in true 32-bit: the matrix cores' 32-bit instructions (and plain FMA
// for 33 to 64 rows of very wide products), every element one accumulator over ascending k: the same bits whichever
// kernel runs (the 32-bit path; also bfloat16 in)
int ga_gemm_nt(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias, int M, int N, int K,
               int in_bf16, int out_bf16, hipStream_t stream);

// ---- gemm_skinny.hip: bfloat16 products for at most 64 rows on the matrix cores
// What ga_gemm_skinny and ga_qkv_rope_skinny take beside the product itself: a norm folded into the products
// around it.  All null or zero for a plain product.
struct GaSkinnyNorm {
  const float* in_sumsq;   // [M][in_parts]: the rows of A are (h * gain) of a norm whose sums of squares these are
  int in_parts;
  float inv_width, eps;
  float* residual;         // [M][N], row stride ldr: the product is added to it (C is not written)
  int64_t ldr;
  const void* gain;        // [N] of the norm that follows
  int gain_f32;
  void* scaled;            // bfloat16 [M][N], row stride lds
  int64_t lds;
  float* out_sumsq;        // [M][ga_skinny_norm_parts(M, N)]
};
int ga_skinny_norm_parts(int M, int N);
int ga_gemm_skinny(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias, int M, int N, int K,
                   int out_f32, int nt, int ks, int grid_splits, int gated, int pack, const struct GaSkinnyNorm* norm,
                   hipStream_t stream);
// the gated product (W [2N, K], gate over up) with a bounded gate: C = g * sigmoid(alpha g) * (u + shift), g = min(gate, limit),
// u = clamp(up, -limit, limit)
int ga_gemm_skinny_bounded_gate(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, int M, int N, int K,
                                int out_f32, int ks, int pack, float limit, float alpha, float shift,
                                const struct GaSkinnyNorm* norm, hipStream_t stream);
int ga_qkv_rope_skinny(void* q_out, const void* A, int64_t lda, const void* W, const void* bias, const void* positions,
                       const void* cos_t, const void* sin_t, const void* slot_mapping, void* k_pages, void* v_pages,
                       int M, int K, int nh, int nkv, int hd, int page_size, int write_kv, int pack,
                       const struct GaSkinnyNorm* norm, hipStream_t stream);

// ---- activation.hip: out [tokens, inter] = silu(gu[:, :inter]) * gu[:, inter:]
int ga_silu_mul(void* out, const void* gu, int tokens, int inter, int is_bf16, hipStream_t stream);
// the same on a product that lies transposed, gu_t [2 inter, tokens] bfloat16; tokens and inter multiples of 8
int ga_silu_mul_transposed(void* out, const void* gu_t, int tokens, int inter, hipStream_t stream);

// a gated activation with bounded factors: out = g * sigmoid(alpha g) * (u + shift), g = min(gu[:, :inter], limit),
// u = clamp(gu[:, inter:], -limit, limit)
int ga_clamped_glu(void* out, const void* gu, int tokens, int inter, float limit, float alpha, float shift, int is_bf16,
                   hipStream_t stream);

// ---- scalar_norm.hip: RMS norm with ONE gain for all coordinates (gain: one float or bfloat16).  rows: out [num_rows,
// hidden] = norm of the rows x[rows[r]] of the float stream (rows null: all rows in order).  add: residual float
// [tokens, hidden] += norm(y); copy (or null): the new residual in y's dtype
int ga_scalar_rmsnorm_rows(void* out, const void* x, const void* gain, const void* rows, int num_rows, int hidden, float eps,
                           int out_bf16, int gain_bf16, hipStream_t stream);
int ga_add_scalar_rmsnorm(void* residual, const void* y, const void* gain, void* copy, int tokens, int hidden, float eps,
                          int y_bf16, int gain_bf16, hipStream_t stream);

// ---- embedding_sinusoid.hip: out float [tokens, hidden] = table[ids] + (sin | cos)(position * freq[i / 2]), then the norm
// with one gain (gain null: no norm); freq float [(hidden + 1) / 2]
int ga_embedding_sinusoid_norm(void* out, const void* table, const void* ids, const void* positions, const void* freq,
                               const void* gain, int tokens, int hidden, float eps, int table_bf16, int gain_bf16,
                               hipStream_t stream);

// ---- short_conv.hip: causal convolution of `taps` taps over time on each channel of the float stream x [tokens, width],
// w float [width, taps]; the inputs before a step's tokens come from state float [slots, taps - 1, width].  apply: out
// (compute dtype) = (add_input ? x : 0) + conv(x); update (after apply): the state moves on by the step's tokens.
// slots int64 [entries], token_entry int32 [tokens], cu int32 [entries + 1], q_start int32 [entries]
int ga_short_conv_apply(void* out, const void* x, const void* w, const void* state, const void* slots,
                        const void* token_entry, const void* cu, const void* q_start, int tokens, int width, int taps,
                        int add_input, int out_bf16, int64_t x_stride, const void* bias, hipStream_t stream);
int ga_short_conv_update(void* state, const void* x, const void* slots, const void* cu, const void* q_start, int entries,
                         int width, int taps, int64_t x_stride, hipStream_t stream);

// ---- gated_recurrence.hip: the HGRN2 recurrence.  proj float [tokens, 2 heads dim + heads vdim] (row stride given) holds
// (q before its SiLU | forget-gate logits | v); state float [slots, heads, dim, vdim]; out float [tokens, heads, vdim]
int ga_hgrn2_scan(void* out, const void* proj, int64_t proj_stride, const void* f_bias, const void* lower, void* state,
                  const void* slots, const void* cu, const void* q_start, int entries, int heads, int dim, int vdim,
                  hipStream_t stream);
// out [rows, vdim] (compute dtype) = x / sqrt(mean(x^2) + eps) * weight, x float [rows, vdim], weight float [vdim]
int ga_headwise_rmsnorm(void* out, const void* x, const void* weight, int64_t rows, int vdim, float eps, int out_bf16,
                        hipStream_t stream);

// ---- latent_attention.hip: attention over a cached latent (one row c of `rank` numbers per token, in pages
// [pages, page_size * rank]) that serves every head as key and as value; queries qa float, already in the latent space
// (element strides per token and per head); window 0: all earlier keys; sink float [heads] or null; gate float
// [tokens, heads] or null; out in the compute dtype (element strides per token and per head)
int ga_latent_attention_max_rank();
// ct_pages (or null): a second copy of the latent, transposed inside the page ([pages][rank][page_size])
int ga_latent_prepare(void* cq, void* c_pages, void* ct_pages, int page_size, void* gate, const void* proj,
                      int64_t proj_stride, const void* wq, const void* wkv, const void* slot_mapping, int tokens, int q_rank,
                      int kv_rank, int heads, float eps, int write_c, int is_bf16, hipStream_t stream);
int ga_latent_attention(void* out, int64_t out_t, int64_t out_h, const void* qa, int64_t qa_t, int64_t qa_h,
                        const void* c_pages, const void* block_table, int table_width, const void* token_entry,
                        const void* positions, const void* sink, const void* gate, int tokens, int heads, int rank,
                        int page_size, int window, float scale, int is_bf16, hipStream_t stream);

// the same on the matrix cores, bfloat16, with both copies of the latent: rows = prompt portions, 16 neighbouring tokens as
// columns (skip_singles: requests that bring one token are left to the other entry point; cu int32 [entries + 1]);
// heads = single tokens, 16 heads as columns, info int32 [n][4] = (row, position, entry, -), the keys dealt to `splits`
// workgroups of tiles_per_split tiles of 32 (ws_o: n * heads * splits * ga_latent_attention_mfma_padded_rank(rank)
// floats, ws_ml: n * heads * splits * 2 floats; null for one split)
int ga_latent_attention_mfma_padded_rank(int rank);
int ga_latent_attention_rows(void* out, int64_t out_t, int64_t out_h, const void* qa, int64_t qa_t, int64_t qa_h,
                             const void* c_pages, const void* ct_pages, const void* block_table, int table_width,
                             const void* token_entry, const void* positions, const void* cu, const void* sink,
                             const void* gate, int tokens, int heads, int rank, int page_size, int window, float scale,
                             int skip_singles, hipStream_t stream);
int ga_latent_attention_heads(void* out, int64_t out_t, int64_t out_h, void* ws_o, void* ws_ml, const void* qa, int64_t qa_t,
                              int64_t qa_h, const void* c_pages, const void* ct_pages, const void* block_table,
                              int table_width, const void* info, int n, const void* sink, const void* gate, int heads,
                              int rank, int page_size, int window, float scale, int splits, int tiles_per_split,
                              hipStream_t stream);

// ---- attention_generic.hip: every token attends to its request's pages; any head size up to 256, window or 0;
// tokens_per_workgroup neighbouring tokens share a workgroup's tiles of keys and values (0: the library chooses; -1: the
// same, and every request of the step has at least 8 tokens in it); few_tokens_workgroups, fill_workgroups: the two
// thresholds by which the launcher chooses among its kernels (speed only); sink_scores: null, or one float per head: a
// score that every query of the head sees beside its keys' and that has no value (it only enters the denominator)
int ga_paged_attention_generic(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                               const void* v_pages, const void* block_table, int table_width, const void* token_entry,
                               const void* positions, int tokens, int nh, int nkv, int hd, int page_size, int window,
                               float scale, int is_bf16, int tokens_per_workgroup, int few_tokens_workgroups,
                               int fill_workgroups, const void* sink_scores, hipStream_t stream);

// ---- attention_mfma.hip (one library per head size): bfloat16 on the matrix cores
int ga_attn_head_dim();
int ga_attn_prefill_max_tile_rows();
// sinks (both entry points): null, or one float per head, a score that enters every denominator of the head
// single new tokens; workspace_o: n_tokens * nh * num_splits * head_dim floats, workspace_ml: n_tokens * nh *
// num_splits * 2 floats
int ga_attn_decode(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                   const void* v_pages, const void* block_table, int table_width, const void* decode_info, int n_tokens,
                   int nh, int nkv, int page_size, int window, float scale, int split_keys, int num_splits,
                   void* workspace_o, void* workspace_ml, const void* sinks, hipStream_t stream);
// rows of prompt portions, in tiles of int32 x 4 = (entry, first row of the step, rows, first position).  parts (or
// null): per tile int32 x 4 = (first key, end of keys, index of the tile's first row among the rows that come in parts,
// part + (number of parts << 16)): the keys of such a tile are dealt to several workgroups, whose partial results
// (part_o: n_part_rows * nh * num_parts * head_dim floats, part_ml: ... * 2) a second kernel merges; part_rows: int32 x 4
// per row in parts, its row of the step first
int ga_attn_prefill(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_pages,
                    const void* v_pages, const void* block_table, int table_width, const void* tiles, int n_tiles,
                    int tile_rows, int nh, int nkv, int page_size, int window, float scale, int fill_workgroups,
                    int prefer_workgroups, const void* parts, const void* part_rows, int n_part_rows, int num_parts, void* part_o,
                    void* part_ml, const void* sinks, hipStream_t stream);

// ---- conv_rope_kv.hip: behind a fused q|k|v projection proj [tokens, (nh + nkv) hd + nkv vd] whose channels pass a
// causal convolution of `taps` taps over time (w float [channels, taps], or null with taps 1: none; state float [slots,
// taps - 1, channels]: a request's last projected rows): convolution, rotation of the first rotary_dim coordinates of
// q's and k's heads (cos_t, sin_t float [positions, rotary_dim / 2], or null with rotary_dim 0), q into q_out [tokens, nh
// * padded], k and v into their pages (k [pages, nkv, page_size, padded], v [pages, nkv, padded, page_size]), heads
// padded with zeros; then (update_state) a second launch moves the state on by the step's tokens; proj may be float
// beside a bfloat16 compute dtype (proj_bf16 0, is_bf16 1)
int ga_conv_rope_kv(void* q_out, const void* proj, const void* w, void* state, const void* slots, const void* token_entry,
                    const void* cu, const void* q_start, const void* positions, const void* cos_t, const void* sin_t,
                    const void* slot_mapping, void* k_pages, void* v_pages, int tokens, int entries, int nh, int nkv, int hd,
                    int vd, int padded, int rotary_dim, int taps, int page_size, int write_kv, int update_state, int is_bf16,
                    int proj_bf16, void* row_scale, const void* gain, float norm_eps, hipStream_t stream);

// ---- output_norm.hip: residual[t] += scale * gain * y[t] / sqrt(mean(y[t]^2) + eps) (a norm on a sublayer's output, a
// factor per channel behind it; gain and scale float [hidden], scale may be null); with `next` also next[t] = next_gain *
// residual[t] / sqrt(mean(residual[t]^2) + next_eps), the rows that the following sublayer reads, in the compute dtype;
// parts > 1: y is float [parts, tokens, hidden], partial sums that are added in order first
int ga_output_norm_add(void* residual, const void* y, const void* gain, const void* scale, float eps,
                       const void* next_gain, float next_eps, void* next, int tokens, int hidden, int y_bf16,
                       int next_bf16, int parts, hipStream_t stream);

// ---- routing.hip: the `top` largest of every row of scores float [tokens, experts] (lowest index among equals) as
// ids int32 [tokens, top], their softmax weights float [tokens, top], and the same weights as rows float [tokens,
// experts] with zeros elsewhere; and the gated activation of experts laid side by side, gate_up [tokens, 2 * width]
// (every expert's ff gate columns followed by its ff up columns; behind the experts a shared one's) -> out [tokens,
// width], column c weighted by dense[t, c / ff] (columns behind experts * ff by 1)
int ga_route_topk(void* ids, void* weights, void* dense, const void* scores, int tokens, int experts, int top,
                  hipStream_t stream);
// the same outputs from sigmoid scores: choice by s + correction inside the `keep` best of `groups` groups (a group's score:
// its group_top largest choice scores added), weights s (/ (their sum + floor) where normalise) * scale
int ga_route_sigmoid_groups(void* ids, void* weights, void* dense, const void* logits, const void* correction, int tokens,
                            int experts, int top, int groups, int keep, int group_top, int normalise, float floor, float scale,
                            hipStream_t stream);
int ga_weighted_silu_mul(void* out, const void* gate_up, const void* dense, int tokens, int width, int experts, int ff,
                         int is_bf16, hipStream_t stream);
// router scores: scores float [tokens, experts] = w . x + b, 32-bit sums, x in the compute dtype or float
int ga_router_max_experts();
int ga_router_scores(void* scores, const void* x, const void* w, const void* b, int tokens, int hidden, int experts, int x_bf16,
                     hipStream_t stream);
// the token-expert pairs grouped by expert (offsets int32 [experts + 1], pair_of_row and row_of_pair int32 [pairs]), the
// rows an expert reads gathered side by side, and the chosen experts' results added up per token with their weights
int ga_route_sort(const void* ids, void* offsets, void* pair_of_row, void* row_of_pair, int pairs, int experts, hipStream_t stream);
// (every expert's group lies `capacity` rows long in `sorted` and in `y`: row r of the grouped order at ids[pair] *
// capacity + r - offsets[ids[pair]])
int ga_gather_pair_rows(void* sorted, const void* x, const void* pair_of_row, const void* ids, const void* offsets, int capacity,
                        int pairs, int hidden, int top, int is_bf16, hipStream_t stream);
int ga_combine_pairs(void* out, const void* y, const void* shared, const void* weights, const void* row_of_pair, const void* ids,
                     const void* offsets, int capacity, int tokens, int hidden, int top, int is_bf16, hipStream_t stream);

// ---- activation.hip: out[i] = max(x[i], 0)^2 over `total` elements (out may be x)
int ga_relu_square(void* out, const void* x, int64_t total, int is_bf16, hipStream_t stream);
// out[i] = sa * a[i] + sb * b[i] in 32-bit (two sublayers' results side by side).  a_parts / b_parts 0: the operand comes in
// the output's dtype (out may be that operand); >= 1: float partial sums [parts, total], added in order first
int ga_scaled_sum(void* out, const void* a, int a_parts, const void* b, int b_parts, float sa, float sb, int64_t total,
                  int is_bf16, hipStream_t stream);

// ---- decay_scan.hip: linear attention with a decay as a recurrence, S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per
// head.  q, k, v: 32-bit rows with a common stride; a from `decay` float [tokens, heads dim] or from `head_decay` float
// [heads] (exactly one of them); q and k turned on their first rot_dims coordinates (pairs i, i + rot_dims / 2; tables float
// [positions, rot_dims / 2]) and multiplied by q_scale, k_scale; state float [slots, heads, dim, vdim], zeros for a request
// whose q_start is 0; out float [tokens, heads, vdim]
int ga_decay_scan(void* out, const void* q, const void* k, const void* v, int64_t stride, const void* decay,
                  const void* head_decay, const void* cos_t, const void* sin_t, int rot_dims, float q_scale, float k_scale,
                  void* state, const void* slots, const void* cu, const void* q_start, int entries, int heads, int dim,
                  int vdim, int silu_inputs, hipStream_t stream);
// decay float [tokens, channels] = sigmoid(a2 low + bias)^(1 / tau); low: 32-bit rows of `rank` numbers with a stride; a2t:
// a2 transposed, float [rank, channels]
int ga_gla_decay(void* decay, const void* low, int64_t low_stride, const void* a2t, const void* bias, int tokens,
                 int channels, int rank, float tau, hipStream_t stream);
// out [tokens, heads, vdim] = x / rms(x over vdim) (* weight [vdim], or null) (* silu(gate), or sigmoid(gate) where sigmoid_gate;
// 32-bit rows with a stride, or null); heads == 1 with a wide vdim: a norm over all heads together
// (decay_scan's silu_inputs: the recurrence reads silu(q), silu(k), silu(v))
int ga_head_norm_gate(void* out, const void* x, const void* weight, const void* gate, int64_t gate_stride, int64_t tokens,
                      int heads, int vdim, float eps, int out_bf16, int sigmoid_gate, hipStream_t stream);

// ---- pooled_attention.hip: attention over a window of tokens and the means of the blocks before it, sigmoid weights.
// prepare: q and k of a 32-bit projection [q heads | k heads | v heads ...] turned by position (pairs 2i, 2i + 1), divided by
// their root mean square per head where `unit`; q out float [tokens, nh dim]; k into rows [slot][nkv][dim], v transposed inside
// its page [page][nkv][vdim][slot]
int ga_pwa_prepare(void* q_out, const void* proj, int64_t stride, const void* positions, const void* cos_t, const void* sin_t,
                   const void* slot_mapping, void* k_rows, void* v_rows, int tokens, int nh, int nkv, int dim, int vdim,
                   int rot_dims, int unit, float eps, int write, int page_size, int cache_bf16, hipStream_t stream);
// for every token that ends a block of `pool` positions: the block's mean key and value (float rows at pool_slots[token])
int ga_pwa_pool(void* pk_rows, void* pv_rows, const void* k_rows, const void* v_rows, const void* positions,
                const void* token_entry, const void* table, int width, const void* pool_slots, int tokens, int nkv, int dim,
                int vdim, int pool, int page_size, int cache_bf16, hipStream_t stream);
// out [tokens, nh vdim] = sum over the visible blocks and tokens of sigmoid(scale q . k + head_bias) v (* sigmoid(gate))
int ga_pwa_attend(void* out, const void* q, const void* k_rows, const void* v_rows, const void* pk_rows, const void* pv_rows,
                  const void* positions, const void* token_entry, const void* table, int width, const void* pool_table,
                  int pool_width, const void* head_bias, const void* gate, int64_t gate_stride, int tokens, int nh, int nkv,
                  int dim, int vdim, int size, int pool, int page_size, float scale, int cache_bf16, int out_bf16,
                  hipStream_t stream);

// the same on the matrix cores (bfloat16 cache and output): prompt portions by the step's tiles int32 [n_tiles][4] = (entry,
// first row, rows, first position), single tokens by info int32 [n_single][4] = (row, position, entry, -), their keys dealt to
// `splits` workgroups (partial: float [splits][n_single][nh vdim] where splits > 1); dim a multiple of 8, page_size too
int ga_pwa_attend_mfma(void* out, void* partial, const void* q, const void* k_rows, const void* v_pages, const void* pk_rows,
                       const void* pv_pages, const void* tiles, int n_tiles, const void* info, int n_single, int splits,
                       const void* table, int width, const void* pool_table, int pool_width, const void* head_bias,
                       const void* gate, int64_t gate_stride, int nh, int nkv, int dim, int vdim, int size, int pool,
                       int page_size, float scale, hipStream_t stream);

// ---- gated_residual.hip: residual float [tokens, hidden] += sigmoid(z[:, :hidden]) * y1 (+ sigmoid(z[:, hidden:]) * y2, y2
// may be null; z: float rows with the stride z_stride); with next: next = rmsnorm(residual) * next_gain (float [hidden])
int ga_gated_residual_add(void* residual, const void* z, int64_t z_stride, const void* y1, const void* y2, int tokens, int hidden,
                          int y_bf16,
                          const void* next_gain, float next_eps, void* next, int next_bf16, hipStream_t stream);

// ---- hyper_connection.hip: the residual stream as S streams side by side, X float [tokens, S, width].  open: every stream
// = x; read: rows = gain * u / rms(u), u = sum_s in[s] X_s; write: X_j <- sum_s mix[s, j] X_s + out[j] * y for all j at once (y
// in the compute dtype, or float partial sums [parts, tokens, width]) and, where next_in / next_gain / rows are given, the
// read of the new streams; sum_rows: the streams' sum at the listed rows (rows null: at every row)
int ga_hc_max_streams();
int ga_hc_open(void* X, const void* x, int tokens, int width, int streams, hipStream_t stream);
int ga_hc_read(void* rows, const void* X, const void* in_w, const void* gain, float eps, int tokens, int width, int streams,
               int rows_bf16, hipStream_t stream);
int ga_hc_write(void* X, const void* mix, const void* out_w, const void* y, int y_bf16, int parts, int64_t part_stride,
                const void* next_in, const void* next_gain, float next_eps, void* rows, int rows_bf16, int tokens, int width,
                int streams, hipStream_t stream);
int ga_hc_sum_rows(void* out, const void* X, const void* rows, int n_rows, int width, int streams, hipStream_t stream);

// ---- rglru.hip: the real-gated linear recurrent unit.  gates: a = exp(-rate * sigmoid(Ra u + ra) * softplus(lam)), b =
// sqrt(1 - a^2) * sigmoid(Ri u + ri) * u, the matrices block-diagonal and handed over transposed [block][in][out]; all float
// [tokens, channels]; and g = gelu_tanh(y), y float rows with a stride.  scan: S_t = a_t S_(t-1) + b_t per channel over float
// state [slots, channels] (zeros where an entry's q_start is 0), out = S * g
int ga_rglru_gates(void* a_out, void* b_out, const void* u, const void* ra_t, const void* ra_b, const void* ri_t,
                   const void* ri_b, const void* lam, const void* y, int64_t y_stride, void* g_out, int tokens, int channels,
                   int blocks, float rate, hipStream_t stream);
int ga_rglru_scan(void* out, const void* a, const void* b, const void* g, void* state, const void* slots, const void* cu,
                  const void* q_start, int entries, int tokens, int channels, int out_bf16, hipStream_t stream);

// ---- random_fill.hip: out[i] = mean + std * normal(key, i) for n elements, float or bfloat16: the counter-based
// generator of random_normal.h, which gives the host library (host/random_fill_host.cpp) the same bits
int ga_random_normal_fill(void* out, int64_t n, uint64_t key, float mean, float std, int is_bf16, hipStream_t stream);

// ---- sampling.hip: out int32 [rows]: argmax (lowest index among equals) where temperature is null or 0, else one
// draw from softmax(logits / temperature) by the given uniform number; scratch: ga_sample_scratch_floats floats
int64_t ga_sample_scratch_floats(int rows, int vocab);
int ga_sample_rows(void* out, const void* logits, int64_t row_stride, int rows, int vocab, const void* temperature,
                   const void* uniform, void* scratch, hipStream_t stream);

// ---- sampling.hip, for callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid allocation).  This entry point has no counterpart in the reference, whose argmax takes
// its buffers from the caller's allocator.  ga_sample_rows_static is ga_sample_rows with its scratch in a static
// device array of 196,608 bytes that each GPU holds until the process ends: at most
// ga_sample_rows_static_max_rows() (256) rows a call, more are refused with -2 and nothing is launched
// (ga_sample_rows_static_error(code) says what a negative code means).  It allocates nothing and calls nothing that
// does.  Calls on one GPU share the array: calls that overlap there (other streams, other threads) race.
// ga_sample_rows_static_init() looks the array up on the current device ahead of the first call (optional).
int ga_sample_rows_static_max_rows();
int ga_sample_rows_static_init();
const char* ga_sample_rows_static_error(int code);
int ga_sample_rows_static(void* out, const void* logits, int64_t row_stride, int rows, int vocab,
                          const void* temperature, const void* uniform, hipStream_t stream);

#ifdef __cplusplus
}
#endif
