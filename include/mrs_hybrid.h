/* mrs_hybrid.h -- C ABI of libmrs_hybrid.so: the kernels of layer-list ("hybrid") decoders served in their checkpoint dtype (csrc/hyb_kernels.hip, csrc/hyb_gemm.hip) and
 * the host-side state slot pool (csrc/host/state_pool.cpp; the paged KV cache manager's mrs_kv_* of mrs_hip_ext.h is linked into this library as well).
 *
 * Conventions: every launcher runs on the stream handed in as its last argument and returns 0, or 1 after storing a message for mrs_hyb_last_error() /
 * mrs_hyb_gemm_last_error().  `dtype` is 1 = bf16, 2 = f32: the type of GEMM operands and of K / V pages; everything else is f32.  A step's rows form one flat range:
 * entry s owns rows [seq_start[s], seq_start[s + 1]) at positions seq_pos0[s] + i, holds state slot seq_slot[s] and the block table row s; an entry whose first position is 0
 * reads its state slot as zero.  The segment table cuts every entry's rows into pieces (seg_entry / seg_row0 / seg_len per segment, ent_seg0 per entry + the total). */
#ifndef MRS_HYBRID_H
#define MRS_HYBRID_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ---- hyb_kernels.hip */
const char *mrs_hyb_last_error();
int mrs_hyb_embed(const int *tokens, const void *table, float *x, int rows, int W, int vocab, int dtype, void *stream);
int mrs_hyb_rmsnorm(const float *x, int ldx, const float *w, void *out, float *out32, float *rstd, int rows, int width, int parts, float eps, int one_plus, int dtype, const float *gate, int ldg, int gate_after, void *stream);
int mrs_hyb_conv(const float *u, int ldu, const float *in_bias, const float *cw, const float *cb, float *state, const int *tok_seq, const int *seq_start, const int *seq_pos0, const int *seq_slot, float *out, int rows, int entries, int C, int taps, int act, void *stream);
int mrs_hyb_conv_silu(const float *u, int ldu, const float *cw, const float *cb, float *state, const int *tok_seq, const int *seq_start, const int *seq_pos0, const int *seq_slot, float *out, int rows, int entries, int C, int taps, void *stream);
int mrs_hyb_ssd_scan(const float *xbc, const float *u, const float *dt_bias, const float *A_log, const float *D, float *state, float *out, const int *seq_pos0, const int *seq_slot, const int *seg_entry, const int *seg_row0, const int *seg_len, const int *ent_seg0, float *steps, float *carry, float *decay, int rows, int entries, int segments, int C, int ldu, int dt_col, int heads, int P, int N, int G, void *stream);
int mrs_hyb_conv_qkv_cache(const float *u, int ldu, const float *in_bias, const float *cw, float *state, const int *tok_seq, const int *seq_start, const int *seq_pos0, const int *seq_slot, const int *tok_pos, const long long *slot_mapping, void *q_out, void *k_cache, void *v_cache, int rows, int entries, int H, int G, int D, int Dv, int block_size, int taps, float temp_coef, int temp_every, int dtype, void *stream);
int mrs_hyb_decay_scan(const float *xkq, int ld, const float *fixed_decay, float *state, float *out, const int *seq_pos0, const int *seq_slot, const int *seg_entry, const int *seg_row0, const int *seg_len, const int *ent_seg0, float *steps, float *carry, float *decay, int rows, int entries, int segments, int heads, int P, int N, int G, void *stream);
int mrs_hyb_qk_norm_rope_cache(const float *qkv, int ld, const float *qw, const float *kw, const float *freq, const int *tok_pos, const long long *slot_mapping, void *q_out, void *k_cache, void *v_cache, int rows, int H, int G, int D, int Dv, int rot, int block_size, float eps, int dtype, void *stream);
int mrs_hyb_paged_window_attn(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_seq, const int *tok_pos, void *out, int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int window, int keep_first, float scale, int dtype, const int *seg_entry, const int *seg_row0, const int *seg_len, int segments, int seg_rows, void *stream);
int mrs_hyb_paged_attn_opts(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_seq, const int *tok_pos, void *out, int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int window, int keep_first, float scale, int dtype, const int *seg_entry, const int *seg_row0, const int *seg_len, int segments, int seg_rows, float softcap, int sink, const float *gate, int ldg, float *scratch, int splits, int token_major, void *stream);
int mrs_hyb_route_sigmoid_topk(const float *h, const float *wr, int rows, int W, int E, int top, int has_gate, int *ids, float *wts, float *gate, void *stream);
int mrs_hyb_moe_dispatch(const int *ids, int R, int E, int *bounds, int *sorted_route, int *route_pos, int *sorted_expert, void *stream);
int mrs_hyb_moe_gather(const float *h32, const int *sorted_route, const float *wts, int top, void *out, int R, int W, int dtype, void *stream);
int mrs_hyb_glu_silu(const float *gu, void *out, int rows, int ff, int dtype, void *stream);
int mrs_hyb_moe_combine(float *x, const float *d, const int *route_pos, int top, const float *shared, const float *gate, int rows, int W, void *stream);
int mrs_hyb_gather_rows(const float *x, const int *idx, float *out, int n, int W, void *stream);
int mrs_hyb_route_softmax_topk(const float *h, const float *wr, int rows, int W, int E, int top, float scale, int *ids, float *wts, void *stream);
int mrs_hyb_moe_combine_weighted(float *out, const float *d, const int *route_pos, const float *wts, int top, const float *shared, int rows, int W, int accumulate, void *stream);
int mrs_hyb_glu_clamped(const float *gu, void *out, int rows, int ff, float limit, float alpha, int dtype, void *stream);
int mrs_hyb_bias_xielu(const float *u, int ldu, const float *bias, void *out, int rows, int ff, float ap, float an, int dtype, void *stream);
int mrs_hyb_layernorm(const float *x, int ldx, const float *in_bias, const float *w, const float *b, void *out, float *out32, float *resid, int ldr, int rows, int width, float eps, int dtype, void *stream);
int mrs_hyb_layernorm_pair(const float *y, int ldy, const float *in_bias, const float *w, const float *b, float *resid, int ldr, const float *w2, const float *b2, void *out, float *out32, int rows, int width, float eps, int dtype, void *stream);
int mrs_hyb_qkv_bias_temp_cache(const float *qkv, int ld, const float *qb, const float *kb, const float *vb, const int *tok_pos, const long long *slot_mapping, void *q_out, void *k_cache, void *v_cache, int rows, int H, int G, int D, int Dv, int block_size, float temp_coef, int temp_every, int dtype, void *stream);
int mrs_hyb_rotary_half(float *u, int ld, int q_col, int k_col, int heads, int D, int rot, const float *freq, const int *tok_pos, float k_mult, int rows, void *stream);
int mrs_hyb_latent_norm_cache(const float *u, int ld, int nq, int R, const float *w, const long long *slot_mapping, void *q_out, void *c_cache, float eps, int rows, int dtype, void *stream);
int mrs_hyb_hyper_step(float *x, const float *y, const float *mix, const float *outw, const float *inw, const float *norm_w, void *out, float *out32, int rows, int S, int W, float eps, int one_plus, int dtype, void *stream);
int mrs_hyb_gated_scan(const float *xkq, int ld, float *steps, float *state, float *out, const int *seq_pos0, const int *seq_slot, const int *seg_entry, const int *seg_row0, const int *seg_len, const int *ent_seg0, float *carry, float *decay, int rows, int entries, int segments, int heads, int P, int N, int G, int ones, float q_mult, void *stream);
int mrs_hyb_qk_headnorm_rope_cache(const float *qkv, int ld, const float *qw, const float *kw, const float *freq, const int *tok_pos, const long long *slot_mapping, void *q_out, void *k_cache, void *v_cache, int rows, int H, int G, int D, int Dv, int rot, int block_size, float eps, int dtype, void *stream);
int mrs_hyb_paged_attn_chunked(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_seq, const int *tok_pos, void *out, int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int chunk, float scale, int dtype, const int *seg_entry, const int *seg_row0, const int *seg_len, int segments, int seg_rows, float softcap, int sink, const float *sink_logit, const float *gate, int ldg, int gate_per_head, float *scratch, int splits, void *stream);
int mrs_hyb_route_topk_softmax(const float *h, const float *wr, const float *bias, int rows, int W, int E, int top, float scale, int *ids, float *wts, void *stream);
/* ---- hyb_recur.hip */
const char *mrs_hyb_recur_last_error();
int mrs_hyb_rmsnorm_pair(const float *x, int ldx, const float *w1, const float *w2, void *out1, void *out2, float *out2_32, int rows, int W, float eps, int one_plus, int dtype, void *stream);
int mrs_hyb_delta_prep(float *c, int ldc, const float *u, int ldu, int b_col, const float *a, int lda, const float *A_log, const float *dt_bias, float *beta, float *dec, int rows, int H, int G, int D, int per, void *stream);
int mrs_hyb_delta_step_prep(const float *u, int ldu, const float *cw, float *state, float *c, int ldc, int C, int taps, int b_col, const float *a, int lda, const float *A_log, const float *dt_bias, float *beta, float *dec, const int *seq_start, const int *seq_pos0, const int *seq_slot, int rows, int entries, int H, int G, int D, int per, void *stream);
int mrs_hyb_delta_scan(const float *c, int ldc, const float *beta, const float *dec, float *state, float *out, const int *seq_pos0, const int *seq_slot, const int *seg_entry, const int *seg_row0, const int *seg_len, const int *ent_seg0, float *carry, float *trans, int rows, int entries, int segments, int H, int G, int D, int Dv, int per, int lanes_per_column, void *stream);
int mrs_hyb_exp_gates(const float *u, int ldu, int i_col, int f_col, const float *bi, const float *bf, float cap, float *m_state, float *steps, float *mbuf, float *mexp, const int *tok_seq, const int *seq_start, const int *seq_pos0, const int *seq_slot, int rows, int entries, int H, void *stream);
int mrs_hyb_head_norm_gate(const float *y, int ldp, const float *mexp, const float *w, int w_full, const float *gate, int ldg, int gate_mode, void *out, int rows, int H, int Dv, float eps, int dtype, void *stream);
int mrs_hyb_norm_pair_add(float *x, int ldx, const float *y1, const float *w1, const float *y2, const float *w2, int rows, int W, float eps, float c, int accumulate, void *stream);
int mrs_hyb_round_cols(const float *u, int ldu, void *out, int rows, int n, int dtype, void *stream);
int mrs_hyb_relu_sq(const float *u, void *out, int rows, int ff, int dtype, void *stream);
/* ---- hyb_attn_talk.hip */
const char *mrs_hyb_talk_last_error();
int mrs_hyb_paged_talk_sigmoid_attn(const void *q, const void *k_cache, const void *v_cache, const int *block_tables, const int *tok_pos, const float *talk, const float *pb, const float *slopes, const float *gate, int ldg, void *out, int rows, int H, int G, int D, int Dv, int block_size, int max_blocks, int window, float scale, int dtype, const int *seg_entry, const int *seg_row0, const int *seg_len, int segments, int seg_rows, float *scratch, int scratch_splits, void *stream);
/* ---- hyb_gemm.hip */
const char *mrs_hyb_gemm_last_error();
int mrs_hyb_gemm(const void *A, const void *W, float *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int accumulate, const int *bounds, int groups, long long wstride, int max_rows, void *stream);
int mrs_hyb_gemm_batched(const void *A, const void *W, void *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int batch, long long a_bstride, long long wstride, long long c_bstride, int c_is_T, void *stream);
int mrs_hyb_gemv(const void *A, const void *W, float *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int accumulate, const int *row_group, long long wstride, int in_mode, const int *src_row, const float *src_scale, int src_div, void *stream);
int mrs_hyb_gemv_act(const void *A, const void *W, float *C, int M, int N, int K, int lda, int ldw, int ldc, int dtype, int accumulate, const int *row_group, long long wstride, int in_mode, const int *src_row, const float *src_scale, int src_div, const float *in_bias, float p0, float p1, void *stream);
void *mrs_state_pool_create(size_t num_slots);
void mrs_state_pool_destroy(void *h);
size_t mrs_state_pool_capacity(void *h);
size_t mrs_state_pool_num_free_slots(void *h);
int64_t mrs_state_pool_allocate(void *h, uint64_t request_id);
int64_t mrs_state_pool_slot_of(void *h, uint64_t request_id);
void mrs_state_pool_free(void *h, uint64_t request_id);
#ifdef __cplusplus
}
#endif
#endif
