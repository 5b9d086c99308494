// C entry points of the gfx950 kernel library.  Every function launches on `stream`
// and returns 0, or one of the EGPT_* error codes without launching anything.
// dtype: 0 = float32, 1 = bfloat16 (activations, weights and caches of one call share it).
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* egpt_error_string(int code);
int egpt_abi_version(void);

// The residual stream (`out` here, `h` below) is float32 [rows][hidden], or with fixed != 0 64-bit fixed point in
// units of 2^-32 (see common.h), which the products of steps of few tokens add their partial results into.
int egpt_embed(const int32_t* ids, const void* table, void* out, int fixed, int n_tokens, int hidden, int vocab,
               int dtype, void* stream);
// h += delta (delta may be null); out = rmsnorm(h) * weight.  rows == null: every row, h written back.
// rows != null: only the listed rows, gathered into out[n_rows], h untouched.
// A product may arrive as float32 partial sums of a split-k product, [n_splits][rows][cols]: then the
// *_splits argument is > 0 and the consumer adds the splits up; 0 means one tensor of the activation type.
int egpt_add_rmsnorm(void* h, int fixed, const void* delta, int delta_splits, int delta_rows, const int32_t* rows,
                     const void* weight, float eps, void* out, int n_rows, int hidden, int dtype, void* stream);
// row_ss (may be null) float32 [ss_splits, n_tokens]: gate_up are float32 partial sums that still lack each row's factor
// 1/sqrt(sum_s row_ss[s][t] / hidden + eps)
int egpt_swiglu(const void* gate_up, int n_splits, const float* row_ss, int ss_splits, int hidden, float eps, void* out,
                int n_tokens, int inter, int dtype, void* stream);
// qkv_out [n_tokens, (nq + 2 nkv) hd] of the activation type; may be qkv_in itself when n_splits == 0.
// row_ss != null: the product still lacks each row's factor 1 / sqrt(sum_s row_ss[s][row] / hidden + eps).
// cos_sin != null: the angles' cosines and sines from egpt_rope_table ([n_tokens][rotary_dim / 2][2]) instead of
// computing them from positions and inv_freq.
int egpt_qkv_rope_store(const void* qkv_in, int n_splits, const float* row_ss, int ss_splits, int hidden, float eps,
                        void* qkv_out, const void* bias, const int32_t* positions, const float* inv_freq,
                        const float* cos_sin, int rotary_dim, const int32_t* slots, void* k_cache, void* v_cache,
                        int n_tokens, int nq, int nkv, int hd, int page_size, int dtype, void* stream);
// cos_sin [n_tokens][half][2] = (cos, sin)(float(positions[t]) * inv_freq[i]) in float32: once per step for all layers.
int egpt_rope_table(const int32_t* positions, const float* inv_freq, float* cos_sin, int n_tokens, int half, void* stream);
// bfloat16 product for m <= 64 rows on the matrix cores, optionally split over k (see gemm_skinny.hip).
// waves: wavefronts (of 16 columns of the result each) per workgroup, 4, 8 or 16; here and below.
// acc_fixed != null (here and in the products below): instead of writing partial sums, every workgroup adds its
// part of the product into acc_fixed [m][n], a residual stream in fixed point, with integer atomics.
int egpt_gemm_skinny(const void* x, const void* w, const void* bias, float* out_f32, void* out_bf16, void* acc_fixed,
                     int m, int n, int k, int n_splits, int waves, void* stream);
// float32 product on the matrix cores (float32 operands and accumulation): out [n_splits][m][n] are partial sums over
// n_splits ranges of k (bias only with one).  k % 4 == 0.  A row's values do not depend on m or on the other rows.
int egpt_gemm_f32(const float* x, const float* w, const float* bias, float* out, int m, int n, int k, int n_splits,
                  void* stream);
// out = x w^T + bias; x [m,k], w [n,k], out [m,n]; out_f32 != 0 writes float32 whatever dtype is.
int egpt_linear(const void* x, const void* w, const void* bias, void* out, int m, int n, int k, int dtype,
                int out_f32, void* stream);
int egpt_paged_attention(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                         const int32_t* block_table, int table_width, const int32_t* q_start, const int32_t* q_len,
                         const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int hd, int page_size,
                         float scale, int window, int dtype, void* stream);
// The same on the matrix cores: bfloat16, head size 64 or 128, page size a multiple of 16.  With n_splits > 1
// the key range of every request is split and part_o [n_splits][n_tokens][nq][hd], part_ml
// [n_splits][n_tokens][nq][2] (float32) hold the partial results that a second kernel combines.
int egpt_paged_attention_mfma(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                              const void* v_cache, const int32_t* block_table, int table_width,
                              const int32_t* q_start, const int32_t* q_len, const int32_t* kv_len, int n_seqs,
                              int n_tokens, int nq, int nkv, int hd, int page_size, float scale, int window,
                              int n_splits, int rows_per_wave, int combine, void* stream);
// Prompt portions: the wavefronts of a workgroup share key/value tiles through LDS (n_splits == 1 semantics);
// page sizes that are powers of two; shape = 10 * row tiles + key splits per workgroup (41, 42, 44, 22, 24), or
// 100 + 10 * blocks of 32 rows + key splits (121, 122, 124, 141, 142; page sizes up to 64).
// key_splits > 1 (shapes from 100 on): the tiles of keys that a block of rows walks are dealt over as many workgroups,
// whose results part_o [key_splits][n_tokens][nq][hd] and part_ml [key_splits][n_tokens][nq][2] (float32) hold until a
// second kernel has combined them.
// single_waves > 0 (needs nq / nkv <= 16): the requests of the step that bring one token are left out here and taken
// by the decode kernel in a launch behind, which spreads a request's keys over the single_waves (1..8) wavefronts of a
// workgroup and over single_splits key ranges; with single_splits > 1, part_o [single_splits][n_seqs][nq][hd] and
// part_ml [single_splits][n_seqs][nq][2] hold those ranges' results until they are combined (the same memory as
// above, used after it: it must hold the larger of the two).
int egpt_paged_attention_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                               const int32_t* block_table, int table_width, const int32_t* q_start,
                               const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv,
                               int hd, int page_size, float scale, int window, int shape, int key_splits,
                               float* part_o, float* part_ml, int single_splits, int single_waves, int single_lean,
                               void* stream);
// One decoded token per request: workgroups of n_waves wavefronts per (request, kv head, key split); lean != 0: the
// variant with half the loads in flight per round and fewer registers.
int egpt_paged_attention_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                                const void* v_cache, const int32_t* block_table, int table_width,
                                const int32_t* q_start, const int32_t* kv_len, int n_seqs, int nq, int nkv, int hd,
                                int page_size, float scale, int window, int n_splits, int n_waves, int combine,
                                int lean, void* stream);
// The same with the QKV epilogue (partial sums, 1/rms, bias, rotation, store of the new key and value) folded in;
// token t belongs to request t; rotation over the whole head.
int egpt_attention_decode_fused(const float* qkv_prod, int in_splits, const float* row_ss, int ss_splits, int hidden,
                                float eps, const void* bias, const float* cos_sin, const int32_t* slots, void* out,
                                float* part_o, float* part_ml, void* k_cache,
                                void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                                const int32_t* kv_len, int n_seqs, int nq, int nkv, int hd, int page_size, float scale,
                                int window, int n_splits, int n_waves, int combine, int lean, void* stream);
// Paged attention on the matrix cores for every head size that is a multiple of 16 up to 256 and page sizes that are
// multiples of 16, bfloat16 or float32 (true float32: v_mfma_f32_16x16x4_f32); see attention_any.hip.  The tiled entry
// takes prompt portions and mixed batches (operands as egpt_paged_attention).  The decode entry takes one token per
// request (token q_start[b] belongs to request b): part_o [n_segments][n_seqs][nq][hd] and part_ml
// [n_segments][n_seqs][nq][2] (float32) take the results of the segments of 64 keys, n_segments >= ceil(longest
// context / 64), which a second kernel folds into out.  In float32 a row's result is the same bits from either.
int egpt_attention_any_tiled(const void* qkv, void* out, const void* k_cache, const void* v_cache,
                             const int32_t* block_table, int table_width, const int32_t* q_start, const int32_t* q_len,
                             const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv, int hd, int page_size,
                             float scale, int window, int dtype, void* stream);
int egpt_attention_any_decode(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                              const void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                              const int32_t* kv_len, int n_seqs, int nq, int nkv, int hd, int page_size, float scale,
                              int window, int n_segments, int dtype, void* stream);
int egpt_attention_combine(const float* part_o, const float* part_ml, void* out, int n_rows, int hd, int n_splits,
                           void* stream);
// Products for m <= 16 rows whose x operand is computed while it is staged (see gemm_skinny.hip).
// h_fixed != 0: h_in is a fixed-point residual stream that is complete as it is (no delta, h_out unused).
int egpt_gemm_skinny_norm(const void* h_in, int h_fixed, float* h_out, const float* delta, int delta_splits,
                          const void* norm_w, const void* w, float* out, float* ss_out, int m, int n, int k,
                          int n_splits, int waves, void* stream);
int egpt_gemm_skinny_swiglu(const float* gate_up, int gu_splits, const float* ss_in, int ss_splits, int hidden,
                            float eps, const void* w, float* out, void* acc_fixed, int m, int n, int k, int n_splits,
                            int waves, void* stream);
int egpt_gemm_skinny_attn(const float* part_o, const float* part_ml, int a_splits, int nq, int hd, const void* w,
                          float* out, void* acc_fixed, int m, int n, int n_splits, int waves, void* stream);
// Gate/up product with SwiGLU for up to 64 rows (see gemm_gate_up.hip): out bfloat16 [m][inter] from x bfloat16 [m][k]
// and w bfloat16 [2 * inter][k] (gate rows, then up rows); k % 8 == 0.
int egpt_gemm_gate_up_swiglu(const void* x, const void* w, void* out, int m, int inter, int k, int groups, void* stream);
// ---- mixers that norm or rotate single heads (head_prep.hip), and their attention (attention_window.hip)
// out [n_tokens][hidden] = table[id] / sqrt(mean(table[id]^2) + eps) * weight: an embedding with its norm, as the
// residual stream (float32, or fixed point with fixed != 0).  In the three functions below row_ss (may be null)
// float32 [ss_splits][n_tokens] says that the product (float32 partial sums) still lacks each row's factor
// 1 / sqrt(sum_s row_ss[s][t] / hidden + norm_eps), as a product with the norm folded in leaves it.
int egpt_embed_rmsnorm(const int32_t* ids, const void* table, const void* weight, float eps, void* out, int fixed,
                       int n_tokens, int hidden, int vocab, int dtype, void* stream);
// proj rows [nq heads of dk | nkv heads of dk | nkv heads of dv] (n_splits > 0: float32 partial sums).  Query and key
// heads are divided by their root mean square and multiplied by q_weight / k_weight [dk] (null: the heads pass as they
// are), value heads are divided by theirs if norm_values != 0.  Queries to q_out [n_tokens][nq * dk]; keys
// [pages][nkv][page_size][dk] and values [pages][nkv][dv][page_size] to slots[t] (null: not stored).
// Rows are row_width values wide.  flags: 1 the value heads are normed (the norm_values of the text above), 2 query and
// key heads are divided by their root mean square also without weights, 4 the norm comes behind the rotation, 8 there
// are no value columns and value head g is key head g as projected (dv == dk), 16 the rotation pairs place 2i with
// 2i + 1 instead of i with i + rot_dims / 2.  rot_dims > 0: the first rot_dims places of query and key heads turn by
// the angles in cos_sin float32 [n_tokens][rot_dims / 2][2] (cos, sin; both times mag).
int egpt_head_norm_store(const void* proj, int n_splits, const float* row_ss, int ss_splits, int hidden, float norm_eps,
                         int row_width, void* q_out, const void* q_weight, const void* k_weight, float eps, int flags,
                         const float* cos_sin, int rot_dims, float mag, const int32_t* slots, void* k_cache, void* v_cache,
                         int n_tokens, int nq, int nkv, int dk, int dv, int page_size, int dtype, void* stream);
// proj rows of row_width values: [nq heads of (dim | rot) | rank | rot | ...].  q_plain [n_tokens][nq][dim] takes the
// heads' unrotated parts; q_full [n_tokens][nq][rank + rot] their rotated parts behind the first rank places.  The
// latent (normed with c_weight [rank]) and the rotated shared key are stored as key [pages][1][page_size][rank + rot],
// the latent also as value [pages][1][rank][page_size].  cos_sin float32 [n_tokens][rot_dims / 2][2], multiplied by
// mag; pairs (2i, 2i + 1) of the first rot_dims places of a rotated part are rotated.
// queries (may be null): the query heads as a product of their own, rows [nq heads of (dim | rot)] (q_splits > 0: float32
// partial sums); the latent then begins at place `lead` of proj's rows.
int egpt_latent_prep(const void* proj, int n_splits, const float* row_ss, int ss_splits, int hidden, float norm_eps,
                     int row_width, const void* queries, int q_splits, int lead, void* q_plain, void* q_full,
                     const void* c_weight, float eps, const float* cos_sin, float mag, int rot_dims, const int32_t* slots,
                     void* k_cache, void* v_cache, int n_tokens, int nq, int dim, int rot, int rank, int page_size, int dtype,
                     void* stream);
// out [n_tokens][n] = x * sigmoid(gate[:, gate_off : gate_off + n]); x [n_tokens][n], or with heads > 0
// [heads][n_tokens][n / heads]; gate: rows of gate_width values (gate_splits > 0: float32 partial sums).
int egpt_sigmoid_gate(const void* x, int heads, const void* gate, int gate_splits, const float* row_ss, int ss_splits,
                      int hidden, float norm_eps, int gate_width, int gate_off, void* out,
                      int n_tokens, int n, int dtype, void* stream);
// Attention with key size dk and value size dv, a window that keeps the first keep_first tokens visible, and an
// optional sink per query head (float32 [nq], null: none) in the softmax's denominator, and an optional bias by
// head and distance (dist_bias float32 [nq][dist_far + 1], null: none): key j of a query at position p gets
// dist_bias[head][min(p - j, dist_far)] added to its scaled score.  block > 0: key j is seen only if it lies in the
// query's block of positions, floor(j / block) == floor(p / block).  slopes float32 [nq] (null: none): the scaled score
// of key j loses slopes[head] * (p - j) (the matrix-core kernel takes a bias table or slopes, not both).  q [n_tokens][nq][dk],
// out [n_tokens][nq][dv]; the other operands as egpt_paged_attention.
int egpt_window_attention(const void* q, void* out, const void* k_cache, const void* v_cache, const int32_t* block_table,
                          int table_width, const int32_t* q_start, const int32_t* q_len, const int32_t* kv_len,
                          int n_seqs, int n_tokens, int nq, int nkv, int dk, int dv, int page_size, float scale,
                          int window, int keep_first, const float* sink, const float* dist_bias, int dist_far, int block,
                          const float* slopes, int dtype, void* stream);
// The same on the matrix cores: dk a multiple of 4 (float32) or 8 (bfloat16) up to 256, dv a multiple of 16 up to 256,
// page_size a multiple of 16.  row_tiles: tiles of 16 rows to a workgroup of four wavefronts: 8 (32 rows to a wavefront)
// or 4 (16).  With
// n_splits > 1 the chunks of keys of a workgroup's rows are dealt over as many workgroups, whose results part_o
// [n_splits][n_tokens][nq][dv] and part_ml [n_splits][n_tokens][nq][2] (float32) a second kernel folds.
int egpt_window_attention_tiled(const void* q, void* out, float* part_o, float* part_ml, const void* k_cache,
                                const void* v_cache, const int32_t* block_table, int table_width, const int32_t* q_start,
                                const int32_t* q_len, const int32_t* kv_len, int n_seqs, int n_tokens, int nq, int nkv,
                                int dk, int dv, int page_size, float scale, int window, int keep_first, const float* sink,
                                const float* dist_bias, int dist_far, int block, const float* slopes, int n_splits,
                                int row_tiles, int dtype, void* stream);
// ---- residual stream and logits (stream_ops.hip)
// out[t] = table[ids[t]] * factor as the float32 residual stream.
int egpt_embed_scaled(const int32_t* ids, const void* table, float factor, float* out, int n_tokens, int hidden, int vocab,
                      int dtype, void* stream);
// h += delta; out = (h - mean) / sqrt(var + eps) * weight + bias (bias may be null); rows and delta as egpt_add_rmsnorm.
int egpt_add_layernorm(float* h, const void* delta, int delta_splits, int delta_rows, const int32_t* rows,
                       const void* weight, const void* bias, float eps, void* out, int n_rows, int hidden, int dtype,
                       void* stream);
// out = factor * (rmsnorm(a + bias_a) * wa + rmsnorm(b + bias_b) * wb) in float32 [n_rows][hidden]; a and b are products
// (one tensor or float32 partial sums), the biases may be null.
// (factor weighs a, factor_b weighs b; wa and wb both null: the branches are not normed, out = factor * a + factor_b * b)
int egpt_normed_pair_mean(const void* a, int a_splits, const void* b, int b_splits, const void* bias_a, const void* bias_b,
                          const void* wa, const void* wb, float eps, float factor, float factor_b, float* out, int n_rows,
                          int hidden, int dtype, void* stream);
// out[t] = table[ids[t]] + pos_table[positions[t]] as the float32 residual stream.
int egpt_embed_positions(const int32_t* ids, const int32_t* positions, const void* table, const void* pos_table, float* out,
                         int n_tokens, int hidden, int vocab, int max_pos, int dtype, void* stream);
// x = h + mult * LN(y) * post_w (LN without bias; y a product: one tensor or float32 partial sums).  With hist (float32
// [n_hist + 1][n_rows][hidden]) x is stored as hist[n_hist] and v = sum_(j <= n_hist) mix[j] * hist[j], else v = x.
// h_out = v (h_out may be h).  With next_w, out = LN(v) * next_w in the activation type.
// (y2, may be null: a second product; the branch is then fy * y + fy2 * y2)
int egpt_post_norm_add(const float* h, const void* y, int y_splits, const void* y2, int y2_splits, float fy, float fy2,
                       const void* post_w, float eps, float mult, float* hist, int n_hist, const float* mix, float* h_out,
                       const void* next_w, void* out, int n_rows, int hidden, int dtype, void* stream);
// x = cap * tanh(x / cap) in place.
// x <- x * scale; then, with cap > 0, x <- cap * tanh(x / cap)
int egpt_tanh_cap(float* x, float scale, float cap, long long n, void* stream);
// ---- head_prep.hip: norms over a whole projection, a position factor on the queries, the store into pages
int egpt_whole_norm_store(const void* proj, int n_splits, int row_width, const void* bias, void* q_out,
                          const void* q_weight, const void* k_weight, float eps, const int32_t* positions, float coef,
                          int every, const int32_t* slots, void* k_cache, void* v_cache, int n_tokens, int nq, int nkv,
                          int dk, int dv, int page_size, int dtype, void* stream);
// out = per-head rmsnorm(x) * weight[dv] * silu(gate columns gate_off.. of a product row); x float32 [n_tokens][heads][dv]
// (x_splits 0) or partial sums [x_splits][n_tokens][heads][dv]; gate null: no gate
// (x rows are x_width values wide, the heads from place 0; x_is_act: x is one tensor of the activation type; gate_act: 0
// silu, 1 sigmoid, 2 the gate's columns are the factor itself)
int egpt_head_norm_gate(const void* x, int x_splits, int x_is_act, int x_width, const void* weight, float eps, const void* gate,
                        int gate_splits, int gate_width, int gate_off, int gate_act, void* out, int n_tokens, int heads, int dv,
                        int dtype, void* stream);
// ---- linear_recurrence.hip: a matrix state per head that decays per key channel
// decay[t][c] = sigmoid(z)^(1 / tau), z = bias[c] + sum_r w[c][r] * low[t][r]; low: columns low_off.. of a product row.
// (rates float32 [channels], may be null: the exponent per channel in place of 1 / tau; negate: z changes its sign first)
int egpt_channel_decay(const void* low, int low_splits, int low_width, int low_off, int rank, const void* w, const void* bias,
                       float tau, const float* rates, int negate, float* decay, int n_tokens, int channels, int dtype, void* stream);
// gate[t][c] = lower[c] + (1 - lower[c]) * sigmoid(z[t][z_off + c] + bias[c]), float32 (bias, lower may be null: 0).
int egpt_bounded_gate(const void* z, int z_splits, int z_width, int z_off, const void* bias, const void* lower, float* gate,
                      int n_tokens, int channels, int dtype, void* stream);
// S <- diag(decay_t) S + k_t v_t^T, o_t = S^T (q_t * q_scale), token by token for every request of the step; the state
// float32 [slots][heads][dk][dv] is read from and written to states[slot[b]] (fresh[b] != 0: it starts at zero).
// q, k, v: columns q_off, k_off, v_off of a product row of proj_width values.  out float32 [egpt_scan_key_splits(dk)][n_tokens][heads][dv]:
// partial sums over ranges of the key channels, for the consumer to add.  q_silu: q_t is silu of its columns;
// tied_keys: k_t = 1 - decay_t (k_off is not read).
int egpt_scan_key_splits(int dk);
int egpt_decayed_state_scan(const void* proj, int n_splits, int proj_width, int q_off, int k_off, int v_off, float q_scale,
                            const float* decay, float* states, const int32_t* slots, const unsigned char* fresh,
                            const int32_t* q_start, const int32_t* q_len, int n_seqs, int n_tokens, float* out, int heads,
                            int dk, int dv, int q_silu, int tied_keys, int k_silu, int v_silu, const float* head_decay,
                            int dtype, void* stream);
// The columns col0.. of a product row as inputs of `channels` short causal convolutions over time (weights [channels][taps],
// the last tap the current token's; the taps - 1 inputs before a step's first token come from the request's record and
// the record is brought up to date behind), SiLU, unit vectors head by head over the first unit_heads * unit_dim channels
// (the first scaled_heads of them times scale), and the sigmoid of n_sig further columns: float32 [n_tokens][channels + n_sig].
int egpt_short_conv(const void* proj, int n_splits, int proj_width, int col0, const void* conv_w, int taps, int channels,
                    int unit_heads, int unit_dim, int scaled_heads, float scale, float unit_eps, int sig_off, int n_sig,
                    float* states, long long state_stride, const int32_t* slots, const unsigned char* fresh,
                    const int32_t* q_start, const int32_t* q_len, int n_seqs, int max_q_len, int n_tokens, float* out, int dtype,
                    void* stream);
// S <- diag(g_t) S; u = beta_t (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t, token by token for every request of the step.
// ops float32 rows hold queries and keys [kv_heads][dk], values [heads][dv] and beta [heads] at their offsets; decay float32
// [n_tokens][heads * dk]; value head h reads query/key head h / (heads / kv_heads); out float32 [n_tokens][heads * dv].
int egpt_delta_rule_scan(const float* ops, int ops_width, int q_off, int k_off, int v_off, int beta_off, const float* decay,
                         float* states, long long state_stride, const int32_t* slots, const unsigned char* fresh,
                         const int32_t* q_start, const int32_t* q_len, int n_seqs, int n_tokens, float* out, int heads,
                         int kv_heads, int dk, int dv, void* stream);
// ---- moe.hip: a mixture of gated experts
// logits = x router^T + bias in float32; the `top` largest per token (lowest index among equals) to chosen[t][top], the
// softmax over the chosen logits to weight[t][top].
// score_all: scores = softmax over all experts; the `top` experts with the largest score + correction (float32 [experts],
// null: none) are chosen, and weigh score / (sum of the chosen scores + 1e-20) * weight_scale.
int egpt_moe_route(const void* x, const void* router, const void* bias, int32_t* chosen, float* weight, int n_tokens,
                   int hidden, int experts, int top, int score_all, const float* correction, float weight_scale, int dtype,
                   void* stream);
// Rows (token, choice) grouped by expert: row_token[n_tokens * top] the token of every grouped row, place[t][top] the
// grouped row of every (token, choice), tiles[0] the number of row tiles, then per tile (expert, first row, rows).
// tile_rows: rows to a tile.  tiles holds 1 + 3 * (n_tokens * top / tile_rows + experts + 1) int32.
int egpt_moe_group(const int32_t* chosen, int32_t* row_token, int32_t* place, int32_t* tiles, int32_t* counts, int n_tokens,
                   int top, int experts, int tile_rows, void* stream);
// act[row] = silu(x[row_token[row]] Wg_e^T) * (x[row_token[row]] Wu_e^T) for every grouped row; w_gate_up [experts][2 ff][hidden]
// (an expert's gate rows, then its up rows).  act [n_tokens * top][ff] of the activation type.
int egpt_moe_gate_up(const void* x, const void* w_gate_up, const int32_t* row_token, const int32_t* tiles, void* act,
                     int n_rows, int hidden, int ff, int experts, int tile_rows, int dtype, void* stream);
// act[row] = relu(x[row_token[row]] Wu_e^T)^2 for every grouped row; w_up [experts][ff][hidden].
int egpt_moe_up(const void* x, const void* w_up, const int32_t* row_token, const int32_t* tiles, void* act, int n_rows,
                int hidden, int ff, int experts, int tile_rows, int dtype, void* stream);
// y[row] = act[row] Wd_e^T, float32 [n_tokens * top][hidden]; w_down [experts][hidden][ff].
int egpt_moe_down(const void* act, const void* w_down, const int32_t* tiles, float* y, int n_rows, int hidden, int ff,
                  int experts, int tile_rows, int dtype, void* stream);
// out[t] = sum_c weight[t][c] * y[place[t][c]] in the order of the choices, float32 [n_tokens][hidden].
int egpt_moe_combine(const float* y, const int32_t* place, const float* weight, float* out, int n_tokens, int top, int hidden,
                     void* stream);
// ---- activations.hip: what stands between the two products of a feed-forward without a gate
// out[t][j] = f(z[t][j]) for the first `cols` columns of a product row of z_width values (one tensor or float32 partial sums):
// mode 0: relu(z)^2; mode 1: the normed polynomial c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with N(u) = u / sqrt(mean_j(u_j^2) + eps)
// over the row's cols values (coef float32 [4]).  gate_col >= 0: times sigmoid(z[t][gate_col]), one number per row.
int egpt_ff_activation(const void* z, int z_splits, int z_width, int cols, int mode, const float* coef, float eps, int gate_col,
                       void* out, int n_tokens, int dtype, void* stream);
// scratch: n_rows * 32 floats followed by n_rows * 32 int32 (two-stage search for wide vocabularies), or null.
int egpt_argmax(const float* logits, int32_t* out, void* scratch, int n_rows, int vocab, void* stream);
// egpt_argmax for callers that cannot allocate device memory and have no workspace to pass (code under graph
// capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The pieces
// of the two-stage search live in a buffer inside the library's device image (256 KiB per GPU, held until the process
// ends) instead of a workspace argument; the call allocates nothing and launches the same kernels as egpt_argmax.
// At most EGPT_ARGMAX_STATIC_MAX_ROWS rows (more: EGPT_STATIC_SCRATCH_TOO_SMALL, nothing is launched).  The buffer needs
// no clearing: every entry that the second stage reads is written by the first stage of the same call.  All calls on
// one GPU share that GPU's buffer, so calls that overlap there (on different streams, or from different threads)
// race; calls on one stream are ordered by the stream.  The stream must belong to the current device.
// egpt_argmax_static_init resolves the buffer's address on the current device (once per device; the entry point
// does it at its first call on a device otherwise): call it before a capture begins.
#define EGPT_ARGMAX_STATIC_MAX_ROWS 1024
int egpt_argmax_static_init(void);
int egpt_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, void* stream);
// weights: scratch for n_rows * vocab floats.
int egpt_sample(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
                const float* uniform, int32_t* out, float* weights, int n_rows, int vocab, void* stream);
// The same in stages for wide vocabularies (several workgroups per row, then the selection on the tokens that can still
// be kept); workspace: egpt_sample_workspace(n_rows, vocab) bytes of device memory.
size_t egpt_sample_workspace(int n_rows, int vocab);
int egpt_sample_wide(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
                     const float* uniform, int32_t* out, void* workspace, int n_rows, int vocab, void* stream);

#ifdef __cplusplus
}
#endif
