// C interface of the HIP library (gfx950).  Every function takes raw device pointers and a HIP
// stream, checks its arguments on the host before it launches anything, and returns 0 on success;
// otherwise alice_last_error() describes the problem.  dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

#define ALICE_ABI_VERSION 12

#define ALICE_EPI_NONE 0
#define ALICE_EPI_GEGLU 1     // W = [gate; up] stacked; epi_param 0: y = gelu_tanh(gate x) * (up x); epi_param = limit > 0:
                              // g = min(gate x, limit), u = clamp(up x, -limit, limit), y = g * sigmoid(1.702 g) * (u + 1);
                              // ALICE_GATED_SILU: y = (gate x) * sigmoid(gate x) * (up x)
#define ALICE_GATED_SILU (-1.0f)
#define ALICE_EPI_SOFTCAP 2   // one function of each output element, its form picked by epi_param: cap > 0: y = cap * tanh(y / cap);
                              // ALICE_UNARY_RELU2: y = max(y, 0)^2
#define ALICE_UNARY_RELU2 (-1.0f)
#define ALICE_EPI_ROPE 3      // internal: rotation and cache write (alice_linear_rope_cache)

#define ALICE_LAYOUT_ROW 0     // row-major [N, K]
#define ALICE_LAYOUT_FRAG16 1  // bfloat16 in 16x32 MFMA fragments, see linear_mfma.hip

#define ALICE_PREFILL_AUTO 0    // prompt attention: chosen by the grid's size
#define ALICE_PREFILL_TILES 1   // a wave takes whole tiles of 16 queries (two heads where the group is even)
#define ALICE_PREFILL_SPLIT 2   // the four waves of a block split one tile's keys
#define ALICE_PREFILL_SHARED4 3 // the four waves of a block share each block of keys and values through LDS
#define ALICE_PREFILL_SHARED8 4 // the same with eight waves
#define ALICE_PREFILL_SHARED4X2 5 // two sets of four waves, each with half of the block's keys

#define ALICE_LINEAR_AUTO 0
#define ALICE_LINEAR_GENERIC 1
#define ALICE_LINEAR_SKINNY 2
#define ALICE_LINEAR_MFMA 3
#define ALICE_LINEAR_TILED_W16 4   // the tiled kernel with a wave tile of 16 output features (activations in fragment order)
#define ALICE_LINEAR_TILED_W32 5   // the same with 32

#ifdef __cplusplus
extern "C" {
#endif

const char* alice_last_error();
int alice_abi_version();
// Digest of the sources and flags this library was built from; the bindings compare it with the sources beside them.
const char* alice_source_digest();
int alice_device_arch(char* out, int cap);

int alice_embed(const int* tokens, const void* table, int table_dtype, int table_layout, float* out,
                int T, int H, int V, float scale, hipStream_t stream);

int alice_add_norm(float* resid, const float* branch, int n_partials, long partial_stride,
                   const void* w_post, const void* w_pre, int w_dtype, void* out, int out_dtype,
                   const int* rows, int T, int H, float eps_post, float eps_pre, float off_post,
                   float off_pre, int full_precision, int out_layout, hipStream_t stream);

// resid += sum over n branches of norm_j(sum of the branch's partial results), norm_j(b) = b / sqrt(mean(b^2) +
// eps_j) * (offsets_j + weights_j) where weights_j is given and b itself where it is null; out (optional): the new
// rows in out_dtype.  The arrays are read on the host.
#define ALICE_MAX_BRANCHES 4
int alice_add_branches(float* resid, int n, const float* const* branches, const int* n_partials,
                       const long* partial_strides, const void* const* weights, int w_dtype, const float* eps,
                       const float* offsets, void* out, int out_dtype, int T, int H, int full_precision,
                       hipStream_t stream);

int alice_softcap(float* x, long n, float cap, int full_precision, hipStream_t stream);

// y[M, N] = x[M, K] . W^T with an optional epilogue.  `variant` forces a kernel (tests); AUTO picks.
// For GEGLU, W has 2N rows.  `split_k` > 1 asks for partial sums y[split_k][M][N] in float32
// (no epilogue), to be added up by the consumer (alice_add_norm's n_partials).
// x_layout / y_layout: ALICE_LAYOUT_ROW, or ALICE_LAYOUT_FRAG16 for activations stored in fragment order
// ([M/16][K/32][64][8], bfloat16, rows padded to 16), which the producers of a decode step write.
int alice_linear(const void* x, int x_dtype, const void* w, int w_dtype, int w_layout, void* y, int y_dtype,
                 int M, int N, int K, int epilogue, float epi_param, int split_k, int variant,
                 int full_precision, int x_layout, int y_layout, hipStream_t stream);
// How many partial sums AUTO would like for this shape (1 = none).
int alice_linear_split_hint(int M, int N, int K, int w_layout);

// Rearranges a row-major bfloat16 [N, K] matrix into the fragment layout ([Np/16][Kp/32][64][8],
// zero padded); dst holds Np * Kp elements with Np = ceil16(N), Kp = ceil32(K).
int alice_to_frag16(const void* src, void* dst, int N, int K, hipStream_t stream);
int alice_frag16_supported(int rows, int K, int epilogue);

// dv: the size of a value head (the v part of a row holds nKV * dv elements, the value pool's rows dv); 0: d.
int alice_rope_cache_write(const void* qkv, int dtype, void* q_out, void* k_pool, void* v_pool,
                           const float* cos_t, const float* sin_t, const int* positions,
                           const int* seq_of_token, const int* block_table, int bt_stride, int T,
                           int row_width, int nH, int nKV, int d, int rotary_dim, int page_size, int n_pages,
                           int kv_layout, int interleaved, int dv, hipStream_t stream);

// The fused q|k|v projection with the rotation and the cache write as its epilogue (single tokens: the
// streaming kernel; more than 64 tokens: the tiled one): x [M, K] (row-major or fragment order), W in the fragment layout with the rows of every q and k
// head in pair order (rows j and j + d/2 of a head at 2j and 2j + 1).  Writes what alice_linear followed by
// alice_rope_cache_write (interleaved) would: q_out [M, nH * d] and the token's keys and values in the cache.
int alice_linear_rope_cache(const void* x, int x_layout, const void* w, int M, int K, void* q_out, void* k_pool,
                            void* v_pool, const float* cos_t, const float* sin_t, const int* positions,
                            const int* seq_of_token, const int* block_table, int bt_stride, int nH, int nKV, int d,
                            int page_size, int n_pages, int kv_layout, hipStream_t stream);

// bias_slopes: null, or nH floats: head h's capped score of key k for the query at position p gets
// bias_slopes[h] * (k - p) added before the softmax (a linear distance bias at the score stage).
// dv: the size of a value head (0: d); out is [T, nH * dv].  gate: null, or the tokens' rows of gate_stride
// elements (the dtype of q) whose first nH hold one number a head: head h's output is multiplied by
// sigmoid(gate[t * gate_stride + h]).
int alice_attention_generic(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out,
                            const int* positions, const int* seq_of_token, const int* block_table,
                            int bt_stride, int T, int nH, int nKV, int d, int page_size, float scale,
                            float softcap, int window, const float* bias_slopes, int full_precision,
                            int dv, const void* gate, int gate_stride, hipStream_t stream);

// bfloat16 attention on the matrix cores over a cache in the fragment layout (kv_layout 1 of
// alice_rope_cache_write): prompts, and single tokens with the keys split over `splits` blocks.
int alice_attention_mfma_supported(int d);
int alice_attention_prefill(const void* q, const void* k_pool, const void* v_pool, void* out,
                            const int* cu_seqlens, const int* context_lens, const int* block_table,
                            int bt_stride, int B, int max_new, int nH, int nKV, int d, int page_size,
                            float scale, float softcap, int window, int variant, int out_layout, hipStream_t stream);
// out[t, h, :] *= sigmoid(gate[t * gate_stride + h]) in place on a bfloat16 attention output in either layout.
// alice_attention_generic with further parameters of the mask and the softmax (0 / null: off): gate: float32 rows,
// gate_mode 1: a number a head, 2: a number an output element ([T, nH dv]); out_scale: a constant factor of the
// gated output; chunk: keys of the query's own chunk of that many
// positions only; keep_first: the first positions stay visible beside the window; sink [nH]: a term of the
// softmax's denominator without a value; vrot_cos / vrot_sin [positions, dv / 2]: the head's output is turned back
// by the query's position; out32 [T, nH, nKV, dv]: every head's weights applied to each kv head's values, float32,
// nothing written to out (alice_mix_heads follows).
int alice_attention_masked(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out,
                           const int* positions, const int* seq_of_token, const int* block_table,
                           int bt_stride, int T, int nH, int nKV, int d, int page_size, float scale,
                           float softcap, int window, const float* bias_slopes, int full_precision,
                           int dv, const float* gate, int gate_stride, int gate_mode, float out_scale, int chunk,
                           int keep_first, const float* sink, const float* vrot_cos, const float* vrot_sin,
                           float* out32, hipStream_t stream);
// alice_attention_masked's result for bfloat16 prompts on the matrix cores (attention_tiled.hip): the step's tokens are
// those of n_seqs sequences in order (cu_seqlens), each at consecutive positions; head sizes multiples of 8 up to 256.
int alice_attention_tiled_supported(int d, int dv);
int alice_attention_tiled(const void* q, const void* k_pool, const void* v_pool, void* out, float* out32,
                          const int* positions, const int* cu_seqlens, const int* block_table, int bt_stride,
                          int T, int n_seqs, int nH, int nKV, int d, int dv, int page_size, float scale, int window,
                          int chunk, int keep_first, const float* bias_slopes, const float* sink,
                          const float* vrot_cos, const float* vrot_sin, const float* gate, int gate_stride,
                          int gate_mode, float out_scale, int heads_per_wave, hipStream_t stream);
// alice_attention_masked's result for single tokens with the keys split over blocks (attention_split.hip), either
// dtype, 32-bit arithmetic; max_keys: the most keys any token of the step sees; work: alice_attention_split_workspace
// floats (runs = alice_attention_split_runs(max_keys)).
int alice_attention_split_supported(int dtype, int nH, int nKV, int d, int dv);
int alice_attention_split_runs(int max_keys);
long alice_attention_split_workspace(int T, int nH, int nKV, int dv, int runs, int per_value_head);
int alice_attention_split(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out, float* out32,
                          const int* positions, const int* seq_of_token, const int* block_table, int bt_stride,
                          int T, int nH, int nKV, int d, int dv, int page_size, float scale, int window, int chunk,
                          int keep_first, int max_keys, const float* bias_slopes, const float* sink,
                          const float* vrot_cos, const float* vrot_sin, const float* gate, int gate_stride,
                          int gate_mode, float out_scale, float* work, hipStream_t stream);
// out[t, h, e] = out_scale * sigmoid(gate[t, h dv + e]) * sum_g talk[h, g] a[t, g, kv head of h, e] (gate optional)
int alice_mix_heads(const float* a, const float* talk, const float* gate, int gate_stride, float out_scale, void* out,
                    int dtype, int T, int nH, int nKV, int dv, int full_precision, hipStream_t stream);
// Bias, rotation in pairs (of q, k and optionally v) and the cache write for a fused projection's rows, see qkv_prepare.hip.
int alice_qkv_prepare(const void* rows, int rows_dtype, int row_width, const float* bias, void* q_out, void* k_pool,
                      void* v_pool, int out_dtype, const float* cos_t, const float* sin_t, int rotary_dim,
                      int interleaved, const float* vcos, const float* vsin, const int* positions,
                      const int* seq_of_token, const int* block_table, int bt_stride, int T, int nH, int nKV,
                      int d, int dv, int page_size, int n_pages, const float* norm_w, float norm_eps, float* inv_rms,
                      hipStream_t stream);
// (norm_w: float32 [nH d + nKV d] or null: the q columns and the k columns are each RMS-normed over the whole
// projection, after the bias and before the rotation; inv_rms: float32 [T, 2] workspace.)
// x[t, c] += a[t, c] + v[c] (either may be null)
int alice_add_rows(float* x, const float* a, const float* v, int T, int W, hipStream_t stream);
// Gated linear attention over a step's tokens, see gla.hip.
int alice_gla(const float* rows, int row_w, int q_col, int k_col, int v_col, int g_col, float* z,
              const float* z_bias, float tau, float q_scale, float out_scale, const void* norm_w, int w_dtype, float eps, void* out,
              int out_dtype, float* work, const int* cu_seqlens, const int* slots, float* S, int T, int n_seqs,
              int n_slots, int H, int d, int dv, int columns, hipStream_t stream);
// Short causal convolution per channel over each sequence's tokens, with the last taps - 1 inputs of earlier steps in
// state [slots, channels, taps - 1]; act 1: silu.  See recurrent.hip for this and the four entries below.
int alice_short_conv(const float* rows, int row_w, int col0, int channels, int taps, const float* w, const float* bias,
                     float* state, float* out, int act, const int* cu_seqlens, const int* seq_of_token, const int* slots,
                     int T, int n_seqs, hipStream_t stream);
// step = softplus(rows[:, dt_col + h] + dt_bias[h]), decay = exp(-exp(a_log[h]) step), both [T, H]
int alice_ssm_prepare(const float* rows, int row_w, int dt_col, const float* dt_bias, const float* a_log, float* step,
                      float* decay, int T, int H, hipStream_t stream);
// unit vectors of the q and k heads of qk [T, q (G d) | ... k at k_col (G d)] in place (q times q_scale); z [T, H d] turned
// into decays exp(-exp(a_log[h]) softplus(z + dt_bias)) in place; beta[t, h] = sigmoid(rows[t, b_col + h])
int alice_delta_prepare(float* qk, int qk_w, int k_col, int G, int d, float unit_eps, float q_scale, float* z,
                        const float* dt_bias, const float* a_log, const float* rows, int row_w, int b_col, float* beta,
                        int T, int H, hipStream_t stream);
// The matrix-state recurrence over a step's tokens (delta 0: S = diag(a) S + k (b v)^T; 1: the delta rule), o to out
// [T, H dv] float32; q and k are shared by groups of H / qk_heads heads; decay [T, H d] (decay_per_row) or [T, H].
int alice_matrix_recurrence(const float* q, int q_w, int q_col, const float* k, int k_w, int k_col, const float* v, int v_w,
                            int v_col, const float* decay, int decay_per_row, const float* b, const float* skip, float* out,
                            const int* cu_seqlens, const int* slots, float* S, int n_seqs, int n_slots, int H, int qk_heads,
                            int d, int dv, int delta, int columns, hipStream_t stream);
// (columns: value columns a wave, 4, 8 or 16; 0: by the step's size, the rule of alice_matrix_recurrence_columns)
int alice_matrix_recurrence_columns(int n_seqs, int H, int d, int dv);
// Rows of `width` in `parts` equal parts, each RMS-normed and multiplied by a weight (w_shared: of a part's length);
// gate_act 1: times silu(gate) before the norm, 2: times sigmoid(gate) after it, 0: no gate.
int alice_norm_gate(const float* x, int width, int parts, const float* gate, int gate_w, int gate_col, int gate_act,
                    const float* w, int w_shared, float eps, void* out, int out_dtype, int T, hipStream_t stream);
// Router of a mixture of experts: dense weights [T, E] from logits [T, E] (+ bias): softmax over the `top` largest,
// zero elsewhere; and y[t, e F + j] = x[t, e F + j] w[t, e].  See experts.hip.
int alice_route_topk(const float* z, const float* bias, float* w, int T, int E, int top, hipStream_t stream);
int alice_scale_columns(const void* x, int x_dtype, const float* w, void* y, int y_dtype, int T, int E, int F, hipStream_t stream);
// The routed feed-forward by grouped products over (token, expert) pairs in expert order (bfloat16, fragment layouts).
long alice_expert_rows(int T, int E, int top);
int alice_expert_products(const void* x, const float* weights, const void* gate_up, const void* down, float* y, int* ints,
                          void* mid, float* rows, int T, int W, int F, int E, int top, float epi, hipStream_t stream);
// Latent attention (latent.hip): the cache row of a token is [latent (kv_rank) | rotated key part (rot_dim)], one kv head,
// row-major pages; the first kv_rank dimensions of a row are also its value.
int alice_latent_prepare(const float* rows, int row_width, int q_rank, int kv_rank, int rot_dim, const float* w_q,
                         const float* w_kv, float eps, const float* cos_t, const float* sin_t, const int* positions,
                         const int* seq_of_token, const int* block_table, int bt_stride, int page_size, int n_pages,
                         void* q_latent, void* k_pool, int out_dtype, int T, hipStream_t stream);
// y[t, h, 0:n] = M_h x[t, h, 0:k], M transposed [H, k, n]; y[t, h, n:n+rot_dim] = x[t, h, k:k+rot_dim] rotated in pairs
// (2i, 2i + 1) by the token's position (tables [positions, rot_dim / 2]).  Rows and heads by their strides in elements.
int alice_heads_linear(const void* x, int x_dtype, long x_row, int x_head, const void* wt, int w_dtype, void* y,
                       int y_dtype, long y_row, int y_head, int T, int H, int n, int k, int rot_dim, const float* cos_t,
                       const float* sin_t, const int* positions, hipStream_t stream);
// q [T, nH, kv_rank + rot_dim] against the cached rows of the token's sequence: keys max(0, pos + 1 - window) .. pos
// (window 0: all), softmax of scale * q.k, out [T, nH, kv_rank] = weights times the rows' first kv_rank dimensions.
int alice_latent_attention(const void* q, int dtype, const void* k_pool, void* out, const int* positions,
                           const int* seq_of_token, const int* block_table, int bt_stride, int T, int nH, int kv_rank,
                           int rot_dim, int page_size, float scale, int window, int full_precision, hipStream_t stream);
// The same on the matrix cores (latent_tiled.hip): bfloat16, kv_rank and rot_dim multiples of 8, together at most 640.
// The step's tokens are those of n_seqs sequences in order (cu_seqlens).  splits > 1 spreads a row group's key blocks
// over that many blocks; part then holds splits * T * nH * (kv_rank + 2) floats.  single_tokens: every sequence brings
// exactly one token (T = n_seqs), which lets the kernel of such steps run where there are at most 16 heads.
int alice_latent_tiled_supported(int kv_rank, int rot_dim);
int alice_latent_tiled_max_splits();
int alice_latent_tiled(const void* q, const void* pool, void* out, float* part, const int* positions, const int* cu_seqlens,
                       const int* block_table, int bt_stride, int T, int n_seqs, int nH, int kv_rank, int rot_dim,
                       int page_size, float scale, int window, int splits, int single_tokens, hipStream_t stream);
// A matrix a head on the matrix cores: bfloat16, w as stored [H, n, k]; n a multiple of 4, k and rot_dim of 8.
int alice_heads_linear_mfma_supported(int n, int k, int rot_dim);
int alice_heads_linear_mfma(const void* x, long x_row, int x_head, const void* w, void* y, long y_row, int y_head, int T, int H,
                            int n, int k, int rot_dim, const float* cos_t, const float* sin_t, const int* positions,
                            hipStream_t stream);
int alice_head_gate(void* out, int out_layout, const void* gate, int gate_stride, int T, int nH, int d, hipStream_t stream);
long alice_attention_decode_workspace(int B, int nH, int d, int splits);
// out may be absent when splits > 1: the splits are then left in `parts`, [B][nH][splits][ALICE_ATTN_PARTS_HEAD + d]
// = (maximum as a base-2 exponent, sum, two unused, unnormalised output: the output starts at a multiple of 16
// bytes), for alice_linear_parts to combine.
#define ALICE_ATTN_PARTS_HEAD 4
// gate (optional, with splits > 1 and an output): bfloat16 rows of gate_stride elements whose first nH hold one
// number a head; head h's output is multiplied by sigmoid(gate[b * gate_stride + h]) where the splits are combined.
int alice_attention_decode(const void* q, const void* k_pool, const void* v_pool, void* out, float* parts,
                           const int* context_lens, const int* block_table, int bt_stride, int B, int nH,
                           int nKV, int d, int page_size, float scale, float softcap, int window, int splits,
                           int out_layout, const void* gate, int gate_stride, hipStream_t stream);

// The output projection straight from the parts of alice_attention_decode (at most 16 sequences and 16 splits, weights in the
// fragment layout, [N, nH d]): y[slices][M][N] float32 partial sums, slices = alice_linear_parts_split(...), which
// is 0 where the sizes are not covered.
int alice_linear_parts_split(int M, int N, int nH, int d, int splits);
int alice_linear_parts(const float* parts, int splits, int nH, int d, const void* w, float* y, int M, int N,
                       hipStream_t stream);

// The matrix memory (mLSTM), one step or several per sequence, with the head norm, its weight and the output
// gate behind it (see mlstm.hip).  proj: float32 rows [q: H*d | k: H*d | v: H*dv | g: H*dv | a: H | b: H] of
// row_w numbers; bias_i, bias_f: float32 [H]; norm_w: [H*dv]; out: [T, H*dv]; sequence s owns the rows
// cu_seqlens[s] .. cu_seqlens[s+1] and the state rows slots[s] of S [n_slots, H, d, dv], n [n_slots, H, d] and
// m [n_slots, H], all float32.
int alice_mlstm_step(const float* proj, int row_w, const float* bias_i, const float* bias_f,
                     const void* norm_w, int norm_dtype, void* out, int out_dtype,
                     const int* cu_seqlens, const int* slots, float* S, float* n, float* m,
                     int n_seqs, int n_slots, int H, int d, int dv, float cap, float eps, hipStream_t stream);

// alice_mlstm_cols: the same result for single tokens and pieces of a few, key sizes up to 256: a block per
// (sequence, head, 64 value columns), the state in registers, read and written once a step.
// The same for steps of many tokens a sequence, a chunk of tokens at a time on the 32-bit matrix instruction;
// work: alice_mlstm_chunks_workspace(...) float32 (alice_mlstm_cols: T * H * dv); max_new: the most tokens of one
// sequence in the step (steps that leave the chip unfilled run their chunks side by side).  alice_mlstm_chunks_supported says whether the head sizes are covered.
int alice_mlstm_cols(const float* proj, int row_w, const float* bias_i, const float* bias_f,
                     const void* norm_w, int norm_dtype, void* out, int out_dtype, float* work,
                     const int* cu_seqlens, const int* slots, float* S, float* n, float* m,
                     int T, int n_seqs, int n_slots, int H, int d, int dv, float cap, float eps, hipStream_t stream);
int alice_mlstm_chunks_supported(int n_seqs, int H, int d, int dv);
long alice_mlstm_chunks_workspace(int T, int n_seqs, int max_new, int H, int d, int dv);
int alice_mlstm_chunks(const float* proj, int row_w, const float* bias_i, const float* bias_f,
                       const void* norm_w, int norm_dtype, void* out, int out_dtype, float* work,
                       const int* cu_seqlens, const int* slots, float* S, float* n, float* m,
                       int T, int n_seqs, int n_slots, int H, int d, int dv, float cap, float eps, int max_new,
                       hipStream_t stream);

// out[t, j] = gelu_tanh(z[t, j]) * table[tokens[t], col0 + j], j < n: a gate on columns of a per-token table
// [V, table_w]; a token outside the table reads zeros.
int alice_gelu_mul_rows(const void* z, int z_dtype, const void* table, int table_dtype, int table_w, int col0,
                        const int* tokens, void* out, int out_dtype, int T, int n, int V,
                        int full_precision, hipStream_t stream);

// Lowest index among equal maxima.
int alice_argmax_chunks(int B, int V);
int alice_argmax(const float* logits, int* out, float* work_v, int* work_i, int B, int V, hipStream_t stream);
// The same argmax with no workspace argument and no allocation of any kind: the chunk maxima go to a device
// array inside the library (ALICE_ARGMAX_STATIC_MAX_PAIRS pairs of a float and an int, 4 KB, which every GPU
// that the library runs on holds until the process ends; it is the most that the chunk rule of
// alice_argmax_chunks ever asks for, ALICE_ARGMAX_MAX_PARTIALS, so no number of rows or vocabulary is too large).  It has no counterpart in the reference; it is for
// callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  It calls no hipMalloc, hipFree or allocating library routine; the caller passes logits and out
// as for alice_argmax.  Rows x chunks beyond the maximum are refused with an error (a check that the chunk rule
// keeps from firing; missing pointers and bad sizes are refused the same way).  All
// calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads) race;
// calls on one stream follow each other and are safe.  alice_argmax_static_init() resolves the array's address
// for the current device ahead of the first call (the first call on a device does it otherwise).
#define ALICE_ARGMAX_MAX_PARTIALS 512
#define ALICE_ARGMAX_STATIC_MAX_PAIRS ALICE_ARGMAX_MAX_PARTIALS
int alice_argmax_static_init();
int alice_argmax_static(const float* logits, int* out, int B, int V, hipStream_t stream);
// temperature -> top-k (0: off) -> top-p (>= 1: off) -> softmax -> first index whose cumulative
// probability exceeds uniform[row].  work: alice_sample_workspace(B, V) 32-bit words, 8-byte aligned.
long alice_sample_workspace(int B, int V);
int alice_sample(const float* logits, int* out, const float* uniform, void* work, int B, int V, float temperature,
                 int top_k, float top_p, hipStream_t stream);

#ifdef __cplusplus
}

// internal
int alice_linear_generic(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype,
                         int M, int N, int K, int epi, float epi_param, int full_precision,
                         hipStream_t stream);
#endif
