// C ABI of the gfx950 kernel library. Every function launches on the given HIP
// stream and returns 0, or non-zero after recording a message for
// he_last_error(). Pointers are device pointers unless named host_*. Shapes
// are validated on the host before any launch. dtype codes: 0 = float32,
// 1 = bfloat16 (2 = float16, as the input of he_cast only).
#pragma once
#include <stdint.h>

#define HE_ABI_VERSION 29

#ifdef __cplusplus
extern "C" {
#endif

const char* he_last_error(void);
int he_abi_version(void);

// ---- weight preparation ----------------------------------------------------
// out[i] = bf16(quantiles[16 bits of the counter-based word of (key, i)] * std + mean), stored as
// `dtype`; quantiles_f32: 65536 quantiles of the standard normal distribution (device pointer).
int he_fill_random(void* out, int64_t n, int dtype, uint64_t key, const void* quantiles_f32,
                   float mean, float std, void* stream);
// out[i] = uniform integer in [0, high) from the counter-based word of (key, i).
int he_fill_random_integers(void* out_i32, int64_t n, uint64_t key, int64_t high, void* stream);
// out = in converted (in: float32, bfloat16 or float16; out: float32 or bfloat16, nearest even).
int he_cast(void* out, const void* in, int64_t n, int in_dtype, int out_dtype, void* stream);

// ---- row-wise ------------------------------------------------------------
// out[t, :] = table[ids[t], :] * scale in fp32.
int he_embedding(void* out_f32, const void* table, const void* ids, int rows, int D, int V,
                 int table_dtype, float scale, void* stream);
int he_gather_rows_f32(void* out, const void* src, const void* rows, int n_out, int D, int n_src,
                       void* stream);
// resid += scale * delta.
int he_residual_add(void* resid_f32, const void* delta, int64_t n, int delta_dtype, float scale,
                    void* stream);
// splits > 0: gate_up is fp32 [splits][rows][2I], the K slices of the product.
int he_silu_mul(void* out, const void* gate_up, int rows, int I, int interleaved, int splits,
                int dtype, void* stream);
// The same columns through a gated activation with constants: gate' = min(gate, limit),
// up' = clamp(up, -limit, limit) (limit <= 0: unbounded), out = gate' * sigmoid(alpha * gate') *
// (up' + up_shift). alpha 1 without limit and shift is he_silu_mul.
int he_gated_act(void* out, const void* gate_up, int rows, int I, int interleaved, int splits,
                 int dtype, float alpha, float limit, float up_shift, void* stream);

// ---- norms ---------------------------------------------------------------
// resid (fp32, in place) += delta (may be null); out (may be null) = rmsnorm(resid) * weight.
int he_add_rmsnorm(void* resid_f32, const void* delta, const void* weight, void* out, int rows, int D,
                   float eps, int act_dtype, int w_dtype, void* stream);
// Dynamic Tanh where a norm would stand: resid (fp32, in place) += delta_scale * delta (may be null);
// out (may be null) = tanh(alpha * resid) * weight + bias, alpha a stored scalar (device pointer),
// weight and bias vectors [D], all three of w_dtype.
int he_add_dyt(void* resid_f32, const void* delta, float delta_scale, const void* weight,
               const void* bias, const void* alpha, void* out, int rows, int D, int act_dtype,
               int w_dtype, void* stream);
int he_rmsnorm_rows(void* out, const void* x, const void* weight, int rows, int D,
                    int64_t x_stride, int64_t out_stride, float eps, int dtype, int w_dtype,
                    void* stream);
// x[r, 0:D1] and x[r, col2:col2+D2] of rows `stride` elements apart, each divided by its own root mean square
// (eps inside the root) and multiplied by its gain (w1, w2; null: 1), in place, one launch.
int he_rmsnorm_row_pair(void* x, const void* w1, int D1, const void* w2, int D2, int col2, int rows, int64_t stride,
                        float eps, int dtype, int w_dtype, void* stream);

// ---- matrix products: C[M,N] = A[M,K] * W[N,K]^T (+ bias) -------------------
// he_gemm_plain: fp32 FMA sums in one fixed order per element (segments of 128 k, each a chain in
// ascending k, added in segment order). With a workspace of he_gemm_plain_workspace_floats(M, N, K)
// floats (0 for more than 8 rows) a product of few rows runs through kernels made for it; the
// result is the same bit for bit.
int64_t he_gemm_plain_workspace_floats(int M, int N, int K);
int he_gemm_plain(void* C, const void* A, const void* W, const void* bias, int M, int N, int K,
                  int64_t lda, int64_t ldw, int64_t ldc, int in_dtype, int out_dtype,
                  int bias_dtype, void* workspace_f32, int64_t workspace_floats, void* stream);
// bf16 MFMA product for M <= HE_BLOCKSPLIT_MAX_M with K cut inside the workgroup (NW
// wavefronts, one slice each, added in LDS): complete in one launch.
#define HE_BLOCKSPLIT_MAX_M 32
int he_gemm_blocksplit_bf16(void* C, const void* A, const void* W, const void* bias, int M, int N,
                            int K, int out_dtype, int bias_dtype, int gated, int R, int U, int NW,
                            void* stream);
// The same with an RMS norm carried across a pair of products. resid != null: the residual
// epilogue (resid[M,N] fp32 += result in place, xg[M,N] bf16 = resid * gain, sq_out[M, sq_count]
// = sums of resid^2 per workgroup, sq_count = he_gemm_blocksplit_blocks). scale_partials != null:
// the rows of A are such xg rows; the result is scaled by 1/sqrt(sum(partials)/K + eps) per row.
// x_pieces / out_pieces (M <= 16): A, or the bf16 output (C, or xg), lies piece-major: a [M, D] tensor as
// 16-byte pieces [D / 8][M][8], element (m, d) at ((d / 8) M + m) 8 + d % 8.
int he_gemm_blocksplit_blocks(int M, int N, int K);
int he_gemm_blocksplit_fused_bf16(void* C, const void* A, const void* W, const void* bias, int M,
                                  int N, int K, int out_dtype, int bias_dtype, int gated, int R,
                                  int U, int NW, const void* scale_partials, int scale_count,
                                  float scale_eps, void* resid, const void* gain, int gain_dtype,
                                  void* xg, void* sq_out, int sq_count, int x_pieces, int out_pieces,
                                  float act_alpha, float act_limit, float act_shift, float resid_scale,
                                  const void* dyt_bias, const void* dyt_alpha, void* stream);
// resid_scale: the residual epilogue adds resid_scale * result. dyt_alpha, dyt_bias (both null, or both
// of gain's dtype; alpha one stored number): the norm that follows is Dynamic Tanh, and the epilogue
// leaves it finished, xg = tanh(alpha * resid) * gain + dyt_bias, with sq_out = 0 (a reader that
// applies 1/sqrt(sum / K + eps) with eps = 1 applies 1). So for he_gemm_rows_bf16 and
// he_splitk_reduce_residual.
// act_alpha, act_limit, act_shift: the constants of the gated epilogue as he_gated_act takes them
// (1, 0, 0: SiLU(gate) * up); so for he_gemm_rows_bf16.
// out = x / sqrt(sum(partials of the row)/D + eps): such xg rows as a normalised tensor
// (row-major; x_pieces: x lies piece-major for exactly `rows` rows).
int he_scale_rows_bf16(void* out, const void* x, const void* partials, int count, int rows, int D,
                       float eps, int x_pieces, void* stream);
// C[M,N] = the slices of partial_f32 [splits][M][N] added in index order (+ bias).
int he_splitk_reduce(void* C, const void* partial_f32, const void* bias, int M, int N, int splits,
                     int out_dtype, int bias_dtype, void* stream);
// bf16 MFMA product for M <= HE_GEMM_ROWS_MAX_M rows whose activation rows are shared through LDS
// by the wavefronts of a workgroup (made for 17 to 64 rows), with the epilogues of
// he_gemm_blocksplit_fused_bf16 (x_pieces / out_pieces for any M here). R (1, 2), NWV (4, 8),
// splits <= 0: the heuristic. A product the plan cuts into several K slices (he_gemm_rows_plan
// says how many) writes fp32 [slices][M][N] into partial_f32 (each slice already scaled by the owed
// row scale) and takes no other epilogue; he_splitk_reduce or he_splitk_reduce_residual adds them.
// With one slice and resid != null, sq_count must be the plan's `groups`.
#define HE_GEMM_ROWS_MAX_M 64
int he_gemm_rows_plan(int M, int N, int K, int* groups, int* splits);
int he_gemm_rows_bf16(void* C, void* partial_f32, int64_t partial_floats, const void* A, const void* W,
                      const void* bias, int M, int N, int K, int out_dtype, int bias_dtype, int gated,
                      int R, int NWV, int splits, const void* scale_partials, int scale_count,
                      float scale_eps, void* resid, const void* gain, int gain_dtype, void* xg,
                      void* sq_out, int sq_count, int x_pieces, int out_pieces, int* splits_used,
                      float act_alpha, float act_limit, float act_shift, float resid_scale,
                      const void* dyt_bias, const void* dyt_alpha, void* stream);
// resid[M,N] (fp32, in place) += the slices of partial_f32 [splits][M][N] in index order (+ bias);
// xg = bf16(resid * gain) (piece-major with out_pieces); sq_out[M, sq_count] = sums of resid^2 per
// block of 1024 columns (sq_count = he_splitk_reduce_residual_blocks(N)): the rows a residual
// epilogue leaves for the next norm.
int he_splitk_reduce_residual_blocks(int N);
int he_splitk_reduce_residual(void* resid_f32, const void* partial_f32, const void* bias, int bias_dtype,
                              const void* gain, int gain_dtype, void* xg, void* sq_out, int sq_count,
                              int M, int N, int splits, int out_pieces, float resid_scale,
                              const void* dyt_bias, const void* dyt_alpha, void* stream);

// ---- position encoding + cache write -------------------------------------
int he_qkv_rope_cache(void* q_out, void* kpool, void* vpool, const void* q_in, const void* k_in,
                      const void* v_in, int64_t in_stride, const void* q_bias, const void* k_bias,
                      const void* v_bias, int bias_dtype, const void* positions,
                      const void* row_seq, const void* seq_slot, const void* page_table,
                      int max_blocks, int num_pages, const void* inv_freq, int rotary_dim, int rows,
                      int H, int KVH, int hd, int hd_in, int vd_in, int interleaved, float mscale,
                      float q_coef, int q_every, int dtype, void* stream);
// hd: head size of q_out and of the cache pages. hd_in, vd_in (0: hd): head sizes of the q/k rows and
// of the v rows that come in (at most hd; q_out is padded with zeros, the pages keep their zeros).
// interleaved: frequency i turns the pair (2i, 2i + 1), not (i, i + rotary_dim / 2). mscale multiplies
// cos and sin. q_every > 0: the q of a row at position p is multiplied by
// 1 + q_coef * ln(floor((p + 1) / q_every) + 1) (a query temperature that grows with the position).

// ---- attention over the paged cache ----------------------------------------
// he_attention_plain: fp32 sums in one fixed order per (query, head): page by page (64 positions),
// inside a page key by key with an online softmax begun afresh, the pages joined in ascending
// position. most_keys: no sequence holds more keys after the step. With a workspace of
// he_attention_plain_workspace_floats floats (0 for a step of many queries) the pages of a query
// run in parallel and a second kernel joins them; the result is the same bit for bit.
// chunk > 0: a query sees no key before the start of its own chunk of that many positions (counted
// from position 0). sinks (or null): one number a head that joins the softmax's denominator as
// exp(sink), without a value. gate (or null): gate[row * gate_stride + h], in the activation dtype;
// the head's output is multiplied by sigmoid(gate).
int64_t he_attention_plain_workspace_floats(int rows, int H, int hd, int most_keys, int window,
                                            int chunk);
int he_attention_plain(void* out, const void* q, const void* kpool, const void* vpool,
                       const void* positions, const void* row_seq, const void* seq_slot,
                       const void* page_table, int max_blocks, int num_pages, int rows, int H,
                       int KVH, int hd, int window, int chunk, float scale, const void* sinks,
                       int sinks_dtype, const void* gate, int64_t gate_stride, int dtype,
                       int most_keys, void* workspace_f32, int64_t workspace_floats, const void* slopes_f32,
                       void* stream);
// slopes_f32 (or null): one number a head; the score of key j for the query at p loses slope * (p - j).
// bf16, one query row per sequence (decode): split over the keys, then merged. chunk, sinks and
// gate (bf16 here) as he_attention_plain takes them; so does he_attention_prefill_bf16.
int he_attention_decode_bf16(void* out, const void* q, const void* kpool, const void* vpool,
                             const void* positions, const void* row_seq, const void* seq_slot,
                             const void* page_table, int max_blocks, int num_pages, int rows,
                             int H, int KVH, int hd, int window, float scale, int max_keys,
                             void* workspace_f32, int64_t workspace_floats, int chunk,
                             const void* sinks, int sinks_dtype, const void* gate, int64_t gate_stride,
                             const void* slopes_f32, void* stream);
int64_t he_attention_decode_workspace_floats(int rows, int H, int KVH, int hd, int max_keys);
// bf16, one query row per sequence, one launch for bias + rotary + cache write + attention +
// merge (a second launch joins the parts where few sequences are cut across workgroups).
// qkv: the un-biased projection rows [rows, (H + 2 KVH) hd]. he_attention_decode_fused_ok: 1
// when the sizes are taken (head_dim 64 or 128, rotated whole). out_pieces: out lies piece-major
// (as he_gemm_blocksplit_fused_bf16 reads it with x_pieces). spread: one sequence of the step has
// several times the keys of the others; every sequence's keys are then cut across more workgroups.
// seq_slot null: page_table has a row per row of the step ([rows, max_blocks], the page numbers of
// the row's sequence) instead of a row per slot. qkv null: the projection rows come as the fp32
// sums of their K slices, qkv_part [qkv_slices][.][qkv_stride] with qkv_slice_stride elements from
// slice to slice (what he_gemm_rows_bf16 leaves when it cuts a product along K); the kernel adds
// them in slice order and rounds to bfloat16, the bits he_splitk_reduce would have written.
int he_attention_decode_fused_ok(int H, int KVH, int hd, int rotary_dim);
int64_t he_attention_decode_fused_workspace_floats(int rows, int H, int KVH, int hd, int max_keys,
                                                   int spread);
int he_attention_decode_fused_bf16(void* out, const void* qkv, const void* qkv_part, int qkv_slices,
                                   int64_t qkv_slice_stride, int64_t qkv_stride, const void* bias,
                                   int bias_dtype, void* kpool, void* vpool, const void* positions,
                                   const void* row_seq, const void* seq_slot,
                                   const void* page_table, int max_blocks, int num_pages,
                                   const void* inv_freq, int rotary_dim, int rows, int H, int KVH,
                                   int hd, int window, float scale, int max_keys, int spread,
                                   int write_kv, int out_pieces, void* workspace_f32,
                                   int64_t workspace_floats,
                                   void* stream);
// bf16, prompt steps: tiles of queries of one sequence against its cache rows. kernel: 0 leaves
// the choice to the library; 1: 16 queries a wavefront, operands straight from global memory
// (any head size up to 256); 2: 32 queries a wavefront, pages shared through LDS, the softmax
// beside the matrix products (head sizes up to 128). parts > 1 (kernel 2 only): the keys of a
// block of queries are cut into that many parts that run side by side and are joined by a
// second launch; the workspace holds he_attention_prefill_workspace_floats() floats.
// he_attention_prefill_parts() is the number the library would take for a step.
int he_attention_prefill_parts(int num_seqs, int max_q_len, int H, int hd, int most_keys);
int64_t he_attention_prefill_workspace_floats(int total_rows, int H, int hd, int parts);
int he_attention_prefill_bf16(void* out, const void* q, const void* kpool, const void* vpool,
                              const void* cu_seqlens, const void* seq_slot, const void* seq_start,
                              const void* page_table, int max_blocks, int num_pages, int num_seqs,
                              int max_q_len, int H, int KVH, int hd, int window, float scale,
                              int kernel, int total_rows, int parts, void* workspace_f32,
                              int64_t workspace_floats, int chunk, const void* sinks, int sinks_dtype,
                              const void* gate, int64_t gate_stride, const void* slopes_f32, void* stream);

// ---- state-space mixer (state_space.hip) ------------------------------------
// A sequence's row of the state area holds, in fp32, the last K-1 inputs of the convolution [K-1][C] at
// its start, and the scan's state at state_offset, he_ssm_state_floats(R, P, N) floats.
// out[row, c] = silu(bias[c] + sum_j taps[c][j] * x[row - (K-1) + j, c]) within a sequence (inputs before the
// step come from the carried ones), then the carried inputs move on. x: [rows][>= C] at x_stride elements.
int he_conv_state(void* out, const void* x, int64_t x_stride, const void* taps, const void* bias,
                  int w_dtype, void* state, int64_t state_stride, const void* positions,
                  const void* row_seq, const void* seq_slot, const void* seq_start,
                  const void* cu_seqlens, int rows, int num_seqs, int C, int K, int all_single,
                  int act, int dtype, void* stream);
int64_t he_ssm_state_floats(int R, int P, int N);
// xbc [rows][R P + 2 Q N]: x, then the Q groups' B vectors, then their C vectors; dt_in[row * dt_stride + r].
// y [rows][R P] fp32 (rows without a sequence are not written). max_q_len: a bound on the rows a sequence brings (0: none).
int he_ssm_scan(void* y_f32, const void* xbc, const void* dt_in, int64_t dt_stride, const void* dt_bias,
                const void* a_log, const void* d_skip, int w_dtype, void* state, int64_t state_stride,
                int64_t state_offset, const void* cu_seqlens, const void* seq_slot, int rows, int num_seqs,
                int max_q_len, int R, int Q, int N, int P, int dtype, void* stream);
// out = rms over each of `parts` stretches of (y * silu(z)) * weight; z[row * z_stride + c]. gate_after 1: out =
// rms over each stretch of y, * weight * sigmoid(z) * out_scale (the gate behind the norm).
int he_gated_group_norm(void* out, const void* y_f32, const void* z, int64_t z_stride, const void* weight,
                        int w_dtype, int rows, int W, int parts, float eps, int gate_after, float out_scale, int dtype,
                        void* stream);

// ---- a matrix memory carried from token to token (matrix_memory.hip) ---------------------
// he_mlstm_gates: out_f32 [rows, 2 H] = the logarithms of the input gates (cap tanh((x + b) / cap)) and of the forget
// gates (logsigmoid of the same bounded number) from their fp32 pre-activations x [rows, 2 H]; cap <= 0: unbounded.
// he_mlstm_scan: y_f32 [rows, H dv] from q, k [rows, H dk] and v [rows, H dv] (views of rows in_stride elements
// apart) and the gates' logarithms (raw_gates: their pre-activations, with gate_bias and cap as he_mlstm_gates takes
// them, and the logarithms are formed inside); S, n and m of a sequence live at state_offset of its row of `state`,
// he_mlstm_state_floats(H, dk, dv) floats, zeros at a sequence's start. dk up to 512.
int64_t he_mlstm_state_floats(int H, int dk, int dv);
int he_mlstm_gates(void* out_f32, const void* x_f32, const void* bias, int bias_dtype, int rows, int H, float cap,
                   void* stream);
int he_mlstm_scan(void* y_f32, const void* q, const void* k, const void* v, int64_t in_stride, const void* gates_f32,
                  void* state, int64_t state_stride, int64_t state_offset, const void* cu_seqlens,
                  const void* seq_slot, int rows, int num_seqs, int H, int dk, int dv, float q_scale, int dtype,
                  int raw_gates, const void* gate_bias, int bias_dtype, float cap, void* stream);

// ---- routing and head combination (routing.hip) ---------------------------------
// logits_f32 [rows][E], or null and x [rows][D] (x_dtype) with router_f32 [E][D]: the kernel forms the logits itself.
int he_route_tokens(void* dense_f32, void* ids_i32, void* weights_f32, const void* logits_f32,
                    const void* x, int x_dtype, const void* router_f32, int D,
                    const void* correction, int c_dtype, int rows, int E, int real, int groups, int keep,
                    int top, float scale, int normalize, void* stream);
int he_routed_act(void* out, const void* gate_up, const void* dense_f32, const void* h, int rows, int real,
                  int I, int extra, int dtype, float alpha, float limit, float up_shift, void* stream);
// For a step of very few rows (bf16): out[rows][D] = the weighted sum of the chosen experts' results alone, from
// the same fused matrices the products over all experts use (gate_up [2 real I][D], rows alternating gate and up;
// down [D][ldw] with the experts' matrices side by side), plus dense[row][real] * x (the identity experts' share).
// ids / weights [rows][top] and dense [rows][real + 1] as he_route_tokens leaves them; h_scratch: rows * top * I
// elements. I, D and ldw in multiples of 8.
int he_chosen_experts(void* out, void* h_scratch, const void* x, const void* gate_up, const void* down,
                      int64_t ldw, const void* ids_i32, const void* weights_f32, const void* dense_f32,
                      int rows, int top, int real, int I, int D, float alpha, float limit, float up_shift,
                      void* stream);
int he_diff_heads(void* out, const void* attn, int rows, int H, int G, int hd, int vd, float lambda,
                  float post, float eps, int dtype, void* stream);

// ---- sampling ------------------------------------------------------------
int64_t he_argmax_workspace_bytes(int rows, int V);
int he_argmax_rows(void* out_i32, const void* logits_f32, int rows, int V, int64_t row_stride,
                   void* workspace, int64_t workspace_bytes, void* stream);
// Not in the reference: an argmax for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). The same kernels as
// he_argmax_rows, with the parts of the rows in a static device array of
// HE_ARGMAX_STATIC_SCRATCH_BYTES per GPU in place of a workspace; it calls no hipMalloc / hipFree
// and no allocating library routine. Inputs needing more scratch (rows * ceil(V / 8192) * 8
// bytes) are refused with an error. All calls on one GPU share that GPU's array: calls that
// overlap on one GPU (two streams, two threads) race; calls on one stream do not.
// he_argmax_rows_static_setup looks up the current device's copy of the array (once per device;
// the first call of he_argmax_rows_static on a device does the same), e.g. before a capture.
#define HE_ARGMAX_STATIC_SCRATCH_BYTES 65536
int he_argmax_rows_static_setup(void);
int he_argmax_rows_static(void* out_i32, const void* logits_f32, int rows, int V,
                          int64_t row_stride, void* stream);
int he_apply_penalties(void* logits_f32, int rows, int V, int64_t row_stride, const void* ids,
                       const void* counts, const void* offsets, float rep, float freq, float pres,
                       void* stream);
// The penalties of he_apply_penalties from a ring of recent tokens on the device: window [rows][W]
// (token number n at n % W), appended [rows] = tokens ever appended. last_ids (or null) are appended
// first, one a row. W up to 4096.
int he_apply_penalties_window(void* logits_f32, int rows, int V, int64_t row_stride, void* window_i32,
                              void* appended_i32, int W, const void* last_ids_i32, float rep, float freq,
                              float pres, void* stream);
int he_sample_rows(void* out_i32, const void* logits_f32, int rows, int V, int64_t row_stride,
                   const void* uniforms_u32, float temperature, int top_k, float top_p,
                   void* stream);


// ---- normed branch outputs, activations and gates (norm.hip, elementwise.hip) ---------------------
// resid += post_weight ? rmsnorm(delta) * post_weight : delta; then out (if given) = next_weight ?
// rmsnorm(resid) * next_weight : resid, in out_dtype. delta may be null (then only out is made).
int he_add_normed(void* resid_f32, const void* delta, int delta_dtype, const void* post_weight, float post_eps,
                  const void* next_weight, float next_eps, int w_dtype, void* out, int out_dtype, int rows, int D,
                  void* stream);
// kind: 0 relu^2, 1 gelu (tanh form), 2 silu, 3 relu
int he_unary_act(void* out, const void* x, int64_t n, int kind, int dtype, void* stream);
// out[r, j] = act(x[r, j]) * table[ids[r], offset + j], j < W
int he_token_gate(void* out, const void* x, const void* table, const void* ids, int rows, int W, int table_width,
                  int offset, int V, int kind, int dtype, int table_dtype, void* stream);
// x[r, h, d] *= sigmoid(gate[r * gate_stride + h * vd + d]) * scale for d < vd, heads hd apart
int he_sigmoid_gate(void* x, const void* gate, int64_t gate_stride, int rows, int H, int hd, int vd, float scale,
                    int dtype, void* stream);
int he_scaled_sum(void* out, const void* a, const void* b, int64_t n, float sa, float sb, int dtype, void* stream);

// ---- a gated delta rule carried from token to token (delta_rule.hip) -------------------------------
// y_f32 [rows, H e] from q, k [rows, G d] and v [rows, H e] (views of rows in_stride elements apart, head h reads the
// q and k of group h / (H / G)), ba_f32 [rows, 2 H] (write strengths b, then decay inputs a) and per head a_log, dt_bias:
// q, k to unit length (q times q_scale), beta = sigmoid(b), g = exp(-exp(a_log) softplus(a + dt_bias)); S <- g S;
// u = beta (v - S^T k); S <- S + k u^T; y = S^T q. S (fp32, he_delta_state_floats floats) lives at byte state_offset of the
// sequence's row of the state area and is carried on.
// workspace_f32: he_delta_workspace_floats floats (16-byte aligned) for what a first launch prepares row by row.
int64_t he_delta_state_floats(int H, int d, int e);
int64_t he_delta_workspace_floats(int rows, int H, int G, int d);
int he_delta_scan(void* y_f32, const void* q, const void* k, const void* v, int64_t in_stride, const void* ba_f32,
                  const void* a_log, const void* dt_bias, int w_dtype, void* state, int64_t state_stride,
                  int64_t state_offset, const void* cu_seqlens, const void* seq_slot, int rows, int num_seqs, int H, int G,
                  int d, int e, float q_scale, float unit_eps, void* workspace_f32, int64_t workspace_floats, int dtype,
                  void* stream);

// ---- norms over parts of a row (group_norm.hip) --------------------------------------------------------
// resid += delta_scale * gn(delta) with gn the RMS norm in `groups` equal consecutive parts times weight (delta null:
// nothing is added); then out (if given) = next_weight ? gn'(resid) : resid, in out_dtype.
int he_add_group_normed(void* resid_f32, const void* delta, int delta_dtype, const void* weight, int w_dtype, int groups,
                        float eps, float delta_scale, void* out, int out_dtype, const void* next_weight, int next_groups,
                        float next_eps, int rows, int D, void* stream);
// out = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e per row of W values; numbers = (a, b, c, e)
int he_polynorm(void* out, const void* x, const void* numbers, int n_dtype, int rows, int W, float eps, int dtype,
                void* stream);
// rows [H q heads | G k heads] of d from `in` to rows [H q heads | G k heads | G v heads] of out (which may be in):
// q and k heads RMS-normed with q_w / k_w [d]; copy_v: the k heads as they were become the v heads
int he_qk_head_norm(void* out, int64_t out_stride, const void* in, int64_t in_stride, const void* q_w, const void* k_w, int w_dtype, int H, int G, int d,
                    float eps, int copy_v, int rows, int dtype, void* stream);

// ---- whole rows of the stream (stream_ops.hip) ---------------------------------------------------------
// kept_f32 plane n - 1 = resid; resid = sum_{j < n} coeffs[j] * plane j
int he_depth_mix(void* resid_f32, void* kept_f32, int64_t plane, const void* coeffs, int c_dtype, int n, int64_t count,
                 void* stream);
// out = a + sigmoid(x . g) * b, row by row
int he_gated_add(void* out, const void* a, const void* b, const void* x, const void* g, int g_dtype, int rows, int D,
                 int Dx, int dtype, void* stream);

// ---- latent attention (latent.hip) ---------------------------------------------------------------------
// out[r, h, n] = sum_k x[r, h, k] w[h][k][n]
int he_head_product(void* out, int64_t o_row, int64_t o_head, const void* x, int64_t x_row, int64_t x_head, const void* w,
                    int w_dtype, int rows, int H, int K, int N, int dtype, void* stream);
int he_latent_pack(void* qkv, const void* q, const void* down, int64_t down_stride, int rows, int H, int d, int r,
                   int rank, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
