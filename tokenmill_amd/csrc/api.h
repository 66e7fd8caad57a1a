// C interface of the kernel library (libtokenmill_hip.so). Every function returns 0 on success,
// TM_ERR_ARG (1) for sizes or types the kernel does not run, TM_ERR_LAUNCH (2) if the launch failed.
// Pointers are device pointers; `stream` is a hipStream_t. dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

int tm_embed_gather(const void* table, int dtype, const int* ids, float* out, int T, int hidden, int vocab,
                    hipStream_t stream);

int tm_add_rmsnorm(float* resid, const void* delta, const int* rows, const void* weight, int w_dtype, void* out,
                   int dtype, int R, int hidden, float eps, hipStream_t stream);

// The same with what is to be added given as 32-bit partial sums parts[p * stride + i] (p < n_parts) of a product whose
// K was split over blocks: added in the order of p, rounded to `dtype`, then as above. tm_sum_parts: that rounded sum alone.
int tm_add_rmsnorm_parts(float* resid, const float* parts, int n_parts, size_t stride, const int* rows, const void* weight,
                         int w_dtype, void* out, int dtype, int R, int hidden, float eps, hipStream_t stream);
int tm_sum_parts(const float* parts, int n_parts, size_t stride, void* out, int dtype, size_t n, hipStream_t stream);

int tm_rope_kv_write(void* qkv, int dtype, int T, int H, int KVH, int D, int rot, const float* cos_t,
                     const float* sin_t, const int* positions, const int* slots, void* k_pool, void* v_pool,
                     int page, int write_kv, hipStream_t stream);

int tm_silu_mul(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream);

int tm_convert(const void* in, int in_dtype, void* out, int out_dtype, long long n, hipStream_t stream);

int tm_gemm_nt_tiled(const void* A, int lda, const void* W, const void* bias, int bias_dtype, void* C, int ldc,
                     int M, int N, int K, int in_dtype, int out_dtype, hipStream_t stream);

// The float32 product on the 32-bit matrix unit: all operands float32, K a multiple of 16, N and the row strides of 4,
// 16-byte aligned (tm_gemm_f32_mfma_fits says whether a product is taken).
int tm_gemm_f32_mfma_fits(const void* A, int lda, const void* W, const void* bias, const void* C, int ldc, int M, int N,
                          int K);
int tm_gemm_f32_mfma(const float* A, int lda, const float* W, const float* bias, float* C, int ldc, int M, int N, int K,
                     hipStream_t stream);

int tm_attn_paged_generic(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                          const void* v_pool, const int* block_tables, int table_width, const int* seq_of_token,
                          const int* positions, int T, int H, int KVH, int D, int page, float scale, int window,
                          int dtype, hipStream_t stream);

// The same with keys and values of different sizes (D, DV), scores capped smoothly at +-softcap (0: as they are) and a gate
// per (token, head) (float32, rows ldg apart; null: none) whose sigmoid multiplies the head's result.
int tm_attn_paged_generic_ext(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                              const int* block_tables, int table_width, const int* seq_of_token, const int* positions, int T, int H,
                              int KVH, int D, int DV, int page, float scale, int window, float softcap, const float* gate, int ldg,
                              int dtype, hipStream_t stream);

// The matrix-unit attention kernels with capped scores (softcap > 0: s <- softcap * tanh(s / softcap); 0: as the plain entries).
int tm_attn_prefill_mfma_cap(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                             const int* block_tables, int table_width, const int* tiles, int n_tiles, int H, int KVH, int D, int page,
                             float scale, int window, float softcap, hipStream_t stream);
int tm_attn_prefill_shared_cap(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                               const int* block_tables, int table_width, const int* tiles, int n_tiles, int H, int KVH, int D, int page,
                               float scale, int window, float softcap, hipStream_t stream);
int tm_attn_prefill_f32_cap(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                            const int* block_tables, int table_width, const int* tiles, int n_tiles, int H, int KVH, int D, int page,
                            float scale, int window, float softcap, hipStream_t stream);
int tm_attn_decode_mfma_cap(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                            const int* block_tables, int table_width, const int* context_lens, float* part_o, float* part_ml,
                            int max_chunks, int S, int H, int KVH, int D, int page, float scale, int window, float softcap,
                            hipStream_t stream);

// q and k normed over the whole projection, rotated and stored (attention_prepare.hip): see the head of that file.
int tm_whole_norm_rope_store(const float* proj, int ld, void* q_out, int dtype, int T, int H, int G, int D, int Dv, int rot,
                             int interleaved, const float* q_w, const float* k_w, float eps, const float* cos_t, const float* sin_t,
                             const int* positions, const int* slots, void* k_pool, void* v_pool, int page, int has_kv,
                             int per_head, hipStream_t stream);
int tm_head_gate(void* x, int dtype, const float* gate, int ldg, int T, int H, int Dv, hipStream_t stream);

int tm_gemm_skinny(const void* A, int lda, const void* W, const void* bias, int bias_dtype, void* C, int ldc, int M,
                   int N, int K, int out_dtype, int silu, float* accum, int ldacc, hipStream_t stream);

// Strip order of a bfloat16 matrix W [N, K] for the decode-step products ("packed", strips of R = 16, 8 or 4
// rows): with KS = ceil(K / 32) k-steps, packed[((s * KS + ks) * 4 + g) * R + r][i] = W[s * R + r][32 ks + 8 g + i]
// for i < 8, zero where the row or the k does not exist; ceil(N / R) strips in all. A wavefront's
// 16-byte loads of one k-step of one strip are then one run of R * 64 bytes. A stacked matrix whose
// parts meet in an epilogue (gate and up) is packed part by part, each part's strips behind the other's.
int tm_skinny_strip_rows(int N, int K);
int tm_fused_qkv_strip_rows(int H, int KVH, int D, int K);
int tm_gemm_skinny_packed(const void* A, int lda, const void* W, int rows, const void* bias, int bias_dtype, void* C,
                          int ldc, int M, int N, int K, int out_dtype, int silu, float* accum, int ldacc,
                          hipStream_t stream);

int tm_attn_decode_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                        const void* v_pool, const int* block_tables, int table_width, const int* context_lens,
                        float* part_o, float* part_ml, int max_chunks, int S, int H, int KVH, int D, int page,
                        float scale, int window, hipStream_t stream);

int tm_fused_norm_qkv_rope(const float* resid, const void* norm_w, int norm_w_dtype, float eps, int M, int K,
                           const void* W, const void* bias, int bias_dtype, void* q_out, int H, int KVH, int D,
                           const float* cos_t, const float* sin_t, const int* positions, const int* slots,
                           void* k_pool, void* v_pool, int page, hipStream_t stream);

int tm_fused_norm_gate_up_silu(const float* resid, const void* norm_w, int norm_w_dtype, float eps, int M, int K,
                               const void* W, void* act_out, int I, hipStream_t stream);

int tm_gemm_panel_fits(int M, int K);
int tm_panel_qkv_rope(const void* X, int ldx, int M, int K, const void* W, const void* bias, int bias_dtype, void* q_out,
                      int H, int KVH, int D, const float* cos_t, const float* sin_t, const int* positions,
                      const int* slots, void* k_pool, void* v_pool, int page, hipStream_t stream);

// The same products for up to 64 tokens at any width (K a multiple of 8), the matrix streamed once from its packed
// copy in strips of `rows` rows (16, 8 or 4), and the plain product with bias whose result is stored or, rounded to
// bfloat16, added into a 32-bit tensor (gemm_stream.hip).
int tm_gemm_stream_fits(int M, int K);
int tm_stream_qkv_rope(const void* X, int ldx, int M, int K, const void* W, int rows, const void* bias, int bias_dtype,
                       void* q_out, int H, int KVH, int D, const float* cos_t, const float* sin_t, const int* positions,
                       const int* slots, void* k_pool, void* v_pool, int page, hipStream_t stream);
int tm_stream_gate_up_silu(const void* X, int ldx, int M, int K, const void* W, void* act_out, int I, hipStream_t stream);
int tm_stream_linear(const void* X, int ldx, int M, int K, const void* W, int rows, int N, const void* bias, int bias_dtype,
                     void* C, int ldc, int out_f32, float* accum, int ldacc, hipStream_t stream);
// The plain product with K split over tm_stream_linear_parts(N, K) groups of blocks (a number from the matrix's shape
// alone; 1: not worth splitting): parts[p][M][N] (float32, M * N elements apart) receives the 32-bit partial sums,
// the bias in part 0, for tm_add_rmsnorm_parts or tm_sum_parts to add up.
int tm_stream_linear_parts(int N, int K);
int tm_stream_linear_split(const void* X, int ldx, int M, int K, const void* W, int rows, int N, const void* bias,
                           int bias_dtype, float* parts, hipStream_t stream);

int tm_attn_prefill_mfma(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                         const void* v_pool, const int* block_tables, int table_width, const int* tiles, int n_tiles,
                         int H, int KVH, int D, int page, float scale, int window, hipStream_t stream);

// The same attention with the keys and values of a tile staged through LDS once for all query heads of a kv
// head (attention_prefill_shared.hip); same operands, out rows 8-byte aligned.
int tm_attn_prefill_shared(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                           const void* v_pool, const int* block_tables, int table_width, const int* tiles, int n_tiles,
                           int H, int KVH, int D, int page, float scale, int window, hipStream_t stream);
int tm_attn_prefill_shared_takes(int H, int KVH, int D);

int tm_gemv_f32(const float* A, int lda, const float* W, const float* bias, float* C, int ldc, int M, int N, int K,
                hipStream_t stream);

// How a caller wants the library's algorithm for a product chosen (tm_gemm_library): see gemm_library.hip.
struct TmTune {
    int candidates;     // 0 or 1: the library's first choice, untimed; n: up to n candidates are timed, the fastest kept
    int after;          // the call of a shape (with the matrix of its first call) at which that happens; 1: at once
    int every;          // a shape timed at its first call also tries every algorithm the library holds for the types
};
int tm_gemm_library(const void* A, int lda, const void* W, int ldw, const void* bias, int bias_dtype, void* C, int ldc,
                    int out_f32, int M, int N, int K, void* workspace, size_t workspace_bytes, const TmTune* tune,
                    hipStream_t stream);

int tm_attn_prefill_f32(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                        const void* v_pool, const int* block_tables, int table_width, const int* tiles, int n_tiles,
                        int H, int KVH, int D, int page, float scale, int window, hipStream_t stream);

// out[t] = table[ids[t]] + places[positions[t]] as 32-bit rows (a learned position table beside the token table).
int tm_embed_gather_pos(const void* table, const void* places, int dtype, const int* ids, const int* positions,
                        float* out, int T, int hidden, int vocab, int max_pos, hipStream_t stream);

int tm_gelu_tanh(const void* in, void* out, int dtype, long long n, hipStream_t stream);
int tm_relu2(const void* in, void* out, int dtype, long long n, hipStream_t stream);

// RMS norm in `groups` equal consecutive parts of a row, around a sublayer (norm_groups.hip):
// resid[r] += norm(y[r]; post_w) (post_w null: y as it is; y null: nothing), out[r] = norm(resid[r]; pre_w) (out null: none).
int tm_group_norm(float* resid, const void* y, const void* post_w, const int* rows, const void* pre_w, int w_dtype,
                  void* out, int dtype, int R, int hidden, int groups, float eps, hipStream_t stream);

// Attention with sigmoid weights that are not normalized over the keys, keys of size D and values of size Dv, within
// chunks and / or a window (attention_sigmoid.hip). qkv rows = [H x D | G x D | G x Dv]; q_w, k_w: weights [D] of the
// per-head RMS norm of q and k (both null: none); head_bias [H] is added to the scaled score (null: none).
int tm_qk_norm_rope_store(void* qkv, int ld, int dtype, int T, int H, int G, int D, int Dv, int rot, const float* q_w,
                          const float* k_w, float eps, const float* cos_t, const float* sin_t, const int* positions,
                          const int* slots, void* k_pool, void* v_pool, int page, int write_kv, hipStream_t stream);
int tm_attn_sigmoid_paged(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                          const int* block_tables, int table_width, const int* seq_of_token, const int* positions,
                          const float* head_bias, int T, int H, int G, int D, int Dv, int page, float scale, int chunk,
                          int window, int dtype, int split_keys, int n_splits, float* parts, hipStream_t stream);

// The same attention for the prompt portions of a step on the matrix unit (attention_sigmoid_prefill.hip): bfloat16, the
// step's tiles of up to 16 tokens as for tm_attn_prefill_mfma; tm_attn_sigmoid_prefill_takes says which sizes it runs.
int tm_attn_sigmoid_prefill_takes(int D, int DV, int page, int q_stride);
int tm_attn_sigmoid_prefill(const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
                            const int* block_tables, int table_width, const int* tiles, int n_tiles, const float* head_bias,
                            int H, int G, int D, int DV, int page, float scale, int chunk, int window, hipStream_t stream);

// Gated linear attention (gla.hip): the decays from the gate projection, the recurrence over a step's rows request by
// request with the state [slots, H, D, Dv] in 32-bit, and the per-head norm of the result times silu(gate).
int tm_gla_decay(const float* z, float* a, float tau, long long n, hipStream_t stream);
int tm_gla_scan(const void* proj, int ld, int q_off, int k_off, int v_off, int dtype, const float* decay, float* o,
                float* state, const int* cu_q_lens, const int* state_slots, int S, int H, int D, int Dv, float q_scale,
                hipStream_t stream);
// Whether tm_gla_scan takes o == nullptr for these operands (only the states are advanced): rows in whole 16-byte pieces.
int tm_gla_scan_in_pieces(int dtype, const void* proj, int ld, int q_off, int k_off, const float* decay, int D);
int tm_gla_out_gate(const float* o, const void* gate, int ldg, int dtype, const float* w, void* y, int T, int H, int Dv,
                    float eps, hipStream_t stream);
// The decays straight from the narrow projection x [T, K] (rows ldx apart), W [N, K], bias [N] of the model's type:
// a = sigmoid(x W^T + b)^(1/tau), 32-bit. And a long portion in segments (see gla.hip): the product of each segment's
// decays, and the chain over a request's segments that turns the segments' local states into their true start states
// and the request's new state.
int tm_gla_gate_decay(const void* x, int ldx, const void* W, const void* bias, int dtype, float* a, int T, int N, int K,
                      float tau, hipStream_t stream);
int tm_gla_segment_decay(const float* decay, const int* cu_seg, float* P, int n_seg, int HD, hipStream_t stream);
int tm_gla_combine(float* state, const int* state_slots, const int* first_seg, const float* P, const float* local,
                   float* start, int S, int HD, int Dv, hipStream_t stream);

// Layer norm with weight and bias behind a gated, scaled residual add (layer_norm.hip):
// v = resid[r] + mult * y[r] * sigmoid(gate[r]) (gate null: no gate; y null: nothing added), written back to resid when
// every row runs (rows null); out[r] = layer_norm(v) * w + b (out null: the add alone). y, gate, out of type `dtype`.
int tm_layer_norm(float* resid, const void* y, const void* gate, float mult, const int* rows, const float* w, const float* b,
                  void* out, int dtype, int R, int hidden, float eps, hipStream_t stream);
// out[t] = h[t] + sum_j w[:, j] * h[t - taps + 1 + j] over a request's rows, the rows before the step's first from the
// request's state [taps - 1, width] (row state_slots[s] of `state`); then tm_short_conv_state makes the state the last
// taps - 1 rows the request has seen. h, out, w [width, taps] and state of type `dtype`; taps up to 16.
int tm_short_conv(const void* h, void* out, const void* w, const void* state, const int* cu_q_lens, const int* state_slots,
                  const int* seq_of_token, int T, int width, int taps, int dtype, hipStream_t stream);
int tm_short_conv_walk(const void* h, void* out, const void* w, void* state, const int* cu_q_lens, const int* state_slots, int S,
                       int width, int taps, int dtype, hipStream_t stream);
int tm_short_conv_state(const void* h, void* state, const int* cu_q_lens, const int* state_slots, int S, int width, int taps,
                        int dtype, hipStream_t stream);
// out = a N(z) + b N(z^2) + c N(z^3) + e with coef = (a, b, c, e) on the device, N(v) = v / sqrt(mean(v^2) + eps) per row.
int tm_poly_norm(const float* z, const float* coef, void* out, int dtype, int T, int F, float eps, hipStream_t stream);

// The gated delta rule and two sublayers side by side (delta_rule.hip): see the head of that file.
int tm_delta_prepare(const void* proj, int ld, const void* conv_w, const void* conv_state, const float* ba, int ldba,
                     const float* a_log, const float* dt_bias, const int* cu_q_lens, const int* state_slots, const int* seq_of_token,
                     float* out, int ldo, int T, int H, int G, int D, int Dv, int taps, float unit_eps, int dtype, hipStream_t stream);
int tm_delta_conv_state(const void* proj, int ld, void* state, const int* cu_q_lens, const int* state_slots, int S, int C, int taps,
                        int dtype, hipStream_t stream);
int tm_delta_scan(const float* rows, int ld, float* o, float* state, const int* cu_q_lens, const int* state_slots, int S, int H, int G,
                  int D, int Dv, int row_dv, int use_v, hipStream_t stream);
int tm_delta_combine(const float* trans, const float* local, float* start, float* state, const int* state_slots, const int* first_seg,
                     int S, int H, int D, int Dv, hipStream_t stream);
int tm_pair_norm_mean(const void* a, const void* b, const float* wa, const float* wb, void* out, int T, int W, float eps, int dtype,
                      hipStream_t stream);
int tm_gelu_mul(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream);
int tm_embed_gather_scaled(const void* table, int dtype, const int* ids, float* out, int T, int hidden, int vocab, float scale,
                           hipStream_t stream);

// Attention over a shared latent (latent.hip): see the head of that file.
int tm_latent_prepare(const float* low, int ld, int Lq, int Lk, int Dr, int rot, const float* wq, const float* wk, float eps,
                      const float* cos_t, const float* sin_t, const int* positions, const int* slots, void* cq, void* pool,
                      int dtype, int T, int half_pairs, hipStream_t stream);
int tm_heads_matmul(const void* A, int lda, int a_head, const void* B, void* C, int ldc, int c_head, const float* gate, int ldg,
                    int T, int H, int K, int N, int dtype, hipStream_t stream);
int tm_rotate_heads(const void* src, int ld_src, int src_head, void* dst, int ld_dst, int dst_head, int T, int H, int Dr, int rot,
                    const float* cos_t, const float* sin_t, const int* positions, int dtype, int half_pairs, hipStream_t stream);
int tm_attn_latent(const void* qa, int q_stride, void* out, int out_stride, const void* pool, const int* block_tables,
                   int table_width, const int* seq_of_token, const int* positions, int T, int H, int Lk, int Dk, int page,
                   float scale, int window, const float* sink, int dtype, hipStream_t stream);
// The same attention on the matrix unit (latent_mfma.hip), bfloat16: the prompt tiles of a step (tiles as for
// tm_attn_prefill_mfma) or its single tokens (rows first_single .. first_single + n_single - 1), one of the two per call.
int tm_attn_latent_mfma_takes(int Lk, int Dk, int q_stride, int out_stride);
// Single tokens have their visible rows dealt in chunks of chunk_runs = tm_attn_latent_chunk_runs(the most rows the model lets
// a token see) runs to blocks of their own: tm_attn_latent_chunks(most rows a token of the call sees, chunk_runs) chunks,
// part_o [n_single * H, chunks, Lk] and part_ml [n_single * H, chunks, 2] 32-bit scratch.
int tm_attn_latent_chunk_runs(int bound);
int tm_attn_latent_chunks(int most_rows, int chunk_runs);
int tm_attn_latent_mfma(const void* qa, int q_stride, void* out, int out_stride, const void* pool, const int* block_tables,
                        int table_width, const int* tiles, int n_tiles, const int* seq_of_token, const int* positions,
                        int first_single, int n_single, float* part_o, float* part_ml, int n_chunks, int chunk_runs, int H, int Lk,
                        int Dk, int page, float scale, int window, const float* sink, hipStream_t stream);

// Experts chosen by a table row of the token id (moe.hip): see the head of that file.
int tm_moe_route(const int* ids, const int* table, int T, int top, int E, int tile_rows, int* slot_pair, int* pair_slot,
                 int* tiles, int* n_tiles, hipStream_t stream);
int tm_moe_gate_up(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                   const int* n_tiles, int max_tiles, int K, int F, int dtype, hipStream_t stream);
int tm_moe_down(const void* act, const void* W, float* part, const int* tiles, const int* n_tiles, int max_tiles, int F, int N,
                int dtype, hipStream_t stream);
int tm_moe_combine(const float* part, const int* pair_slot, void* y, int T, int top, float weight, int N, int dtype,
                   hipStream_t stream);

// Experts chosen by a router, experts without a gate, experts that stand for the input itself, a shared expert (moe.hip).
int tm_moe_router(const float* z, int ldz, const float* correction, int T, int E, int top, int* chosen, float* weight,
                  int over_chosen, hipStream_t stream);
int tm_moe_route_chosen(const int* ids, const int* table, int T, int top, int E, int real, int tile_rows, int* slot_pair,
                        int* pair_slot, int* tiles, int* n_tiles, hipStream_t stream);
int tm_moe_up_act(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                  const int* n_tiles, int max_tiles, int K, int F, int dtype, hipStream_t stream);
int tm_moe_combine_weighted(const float* part, const int* pair_slot, const float* weight, const void* x, int ldx, const float* shared,
                            const float* shared_gate, int ldg, void* y, int T, int top, int N, int dtype, hipStream_t stream);
int tm_moe_up_act_mfma(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                       const int* n_tiles, int max_tiles, int tile_rows, int K, int F, hipStream_t stream);

// The per-head products and the experts' products on the matrix unit (grouped_mfma.hip), bfloat16; the matrices as
// [groups, N, K] with k contiguous. The *_takes functions say whether the operands come in whole 16-byte pieces.
int tm_heads_matmul_mfma_takes(const void* A, int lda, int a_off, const void* W, int K);
int tm_heads_matmul_mfma(const void* A, int lda, int a_off, const void* W, void* C, int ldc, int c_off, const float* gate, int ldg,
                         int T, int H, int K, int N, int tail, int rot, const float* cos_t, const float* sin_t, const int* positions,
                         int half_pairs, hipStream_t stream);
int tm_moe_mfma_takes(const void* x, int ldx, const void* Wgu, const void* Wd, const void* act, int K, int F);
int tm_moe_gate_up_mfma(const void* x, int ldx, const int* slot_pair, int top, const void* W, void* act, const int* tiles,
                        const int* n_tiles, int max_tiles, int tile_rows, int K, int F, hipStream_t stream);
int tm_moe_down_mfma(const void* act, const void* W, float* part, const int* tiles, const int* n_tiles, int max_tiles, int tile_rows,
                     int F, int N, hipStream_t stream);

int tm_argmax_work_chunks(int V);
int tm_argmax_rows(const float* logits, int R, int V, int* out, float* work_v, int* work_i, hipStream_t stream);

// The argmax again, for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc. (The reference has no counterpart: its argmax is a
// torch call that allocates as it likes.) Same result as tm_argmax_rows. The chunk candidates of the
// two-stage path go to a fixed array of 512 KiB that each GPU holds from the library's load to the
// process's end; the call allocates nothing and frees nothing. R * tm_argmax_work_chunks(V) may be at
// most tm_argmax_rows_static_max_pairs() (65,536: 256 rows of a 1M-entry vocabulary, 1,724 rows of
// 151,936 entries); more is refused with TM_ERR_ARG before anything is launched. All calls on one GPU
// share that GPU's array: two calls whose kernels can overlap there (different streams, or threads
// without an order between them) race; calls on one stream are ordered and safe. The device of
// `stream` must be the current device.
int tm_argmax_rows_static_max_pairs(void);
int tm_argmax_rows_static(const float* logits, int R, int V, int* out, hipStream_t stream);

size_t tm_sample_work_bytes(int R, int V);
int tm_sample_rows(const float* logits, int R, int V, const float* temperature, const int* top_k,
                   const float* top_p, const float* u, int* out, void* work, size_t work_bytes, int stages,
                   hipStream_t stream);

}  // extern "C"
