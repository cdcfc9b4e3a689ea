// Prototypes of the kernel entry points (each defined in the .hip file of its kernel), for host code
// inside the library that queues several of them: the native step (step_plan.hip).  Every entry point
// checks its operands, queues its kernels on `stream` and returns 0, or non-zero with the reason in
// gibbs_last_error().
#pragma once
#include <hip/hip_runtime.h>
#include "attention_decode_api.h"

extern "C" {
int gibbs_embed(const void* table, int dtype, const int* ids, float* x, void* mirror, int n, int hidden, int vocab,
                hipStream_t stream);
int gibbs_embed_general(const void* table, int dtype, const int* ids, float* x, void* mirror, int n, int hidden, int vocab,
                        float scale, const int* pos, const float* inv_freq, float* keep, hipStream_t stream);
int gibbs_rmsnorm_rows(const void* in, int parts, long part_stride, const float* gain, float eps, void* out, int dtype, int n,
                       int hidden, hipStream_t stream);
int gibbs_rmsnorm_rows_add(float* x, const void* in, int parts, long part_stride, const float* gain, float eps, int dtype, int n,
                           int hidden, hipStream_t stream);
int gibbs_rmsnorm_rows_add_norm(float* x, const void* in, int parts, long part_stride, const float* gain_d, float eps_d,
                                const float* gain_n, float eps_n, void* out, int dtype, int n, int hidden, hipStream_t stream);
int gibbs_glu_clamped(const void* gu, void* out, int dtype, int n, int F, float alpha, float limit, hipStream_t stream);
int gibbs_attention_plain_general(const void* q, const void* kpages, const void* vpages, void* out, int dtype, const int* pos,
                                  const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows,
                                  int nh, int nkv, int hd, int vd, long ldq, long ldo, float scale, int window,
                                  const float* slopes, const float* bias, int bias_len, hipStream_t stream);
int gibbs_attention_prefill_masked(const void* q, const void* kpages, const void* vpages, void* out, float* partial, const int* cu,
                                   const int* ctx, const int* table, int n_req, int max_pages, int page_size, int num_pages, int n_rows,
                                   int nh, int nkv, int hd, long ldq, long ldo, float scale, int window, int n_splits, int first_row,
                                   int heads_per_wg, const float* bias, int bias_len, const float* sink, int chunk, float softcap,
                                   hipStream_t stream);
int gibbs_attention_decode_masked(const void* q, const void* kpages, const void* vpages, void* out, float* partial, const int* pos,
                                  const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh,
                                  int nkv, int hd, long ldq, long ldo, float scale, int window, int n_splits, int waves, int kind,
                                  int max_keys, const float* bias, int bias_len, const float* sink, int chunk, float softcap,
                                  hipStream_t stream);
int gibbs_attention_plain_masked(const void* q, const void* kpages, const void* vpages, void* out, int dtype, const int* pos,
                                 const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows,
                                 int nh, int nkv, int hd, int vd, long ldq, long ldo, float scale, int window, const float* slopes,
                                 const float* bias, int bias_len, const float* sink, int chunk, float softcap, hipStream_t stream);
int gibbs_attention_plain_sink(const void* q, const void* kpages, const void* vpages, void* out, int dtype, const int* pos,
                               const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows,
                               int nh, int nkv, int hd, int vd, long ldq, long ldo, float scale, int window,
                               const float* slopes, const float* bias, int bias_len, const float* sink, hipStream_t stream);
int gibbs_attention_prefill_sink(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                                 const int* cu, const int* ctx, const int* table, int n_req, int max_pages, int page_size,
                                 int num_pages, int n_rows, int nh, int nkv, int hd, long ldq, long ldo, float scale, int window,
                                 int n_splits, int first_row, int heads_per_wg, const float* bias, int bias_len,
                                 const float* sink, hipStream_t stream);
// ---- latent.hip: what the latent-attention mixer, hyper-connected streams and their neighbours need
int gibbs_embed_tables(const void* table, const void* pair_table, const void* pos_table, int dtype, const int* ids,
                       const int* pos, const int* row_req, const int* cu, const int* slot, const int* prev, long slot_stride,
                       float* x, int copies, int n, int hidden, int vocab, int buckets, int mul_prev, int mul_cur, int pos_len,
                       hipStream_t stream);
int gibbs_store_last_token(const int* ids, const int* cu, const int* slot, int* prev, long slot_stride, int n_req,
                           hipStream_t stream);
int gibbs_streams_norm(const float* x, int streams, long stream_stride, const float* coef, int kind, const float* gain,
                       const float* bias, float eps, void* out, int dtype, const int* rows, int n_out, int hidden,
                       hipStream_t stream);
int gibbs_streams_write(float* x, int streams, long stream_stride, const float* mix, const float* out_coef, const void* delta,
                        int delta_dtype, int parts, long part_stride, long count, hipStream_t stream);
int gibbs_streams_write_norm(float* x, int streams, long stream_stride, const float* mix, const float* out_coef,
                             const void* delta, int delta_dtype, int parts, long part_stride, int n_rows, int hidden,
                             const float* coef, int kind, const float* gain, const float* bias, float eps, void* out, int dtype,
                             hipStream_t stream);
int gibbs_rms_rows_ld(const void* in, long ld_in, const float* gain, float eps, void* out, long ld_out, int dtype, int n,
                      int width, hipStream_t stream);
int gibbs_latent_prepare(const void* kv, long ld_kv, const void* q, long ld_q, void* q_out, long ld_qo, void* pages, int dtype,
                         const float* gain, float eps, const float* inv_freq, int rot_dims, int variant, const int* pos,
                         const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh,
                         int dim, int rot, int rank, hipStream_t stream);
int gibbs_poly_norm(const void* z, void* out, int dtype, const float* coef, float eps, int n, int F, hipStream_t stream);
int gibbs_gemm_heads(const void* X, long ldx, long head_x, const void* W, long head_w, long ldw, void* Y, long ldy, long head_y,
                     int dtype, int n, int O, int I, int heads, hipStream_t stream);
int gibbs_gemm_heads_gated(const void* X, long ldx, long head_x, const void* W, long head_w, long ldw, void* Y, long ldy,
                           long head_y, const void* G, long ldg, long head_g, int dtype, int n, int O, int I, int heads,
                           hipStream_t stream);
int gibbs_qk_unit_kv(void* rows, long ld, void* kpages, void* vpages, int dtype, const int* pos, const int* row_req,
                     const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh, int nkv, int hd, int vd,
                     float eps, int unit, int norm_dim, float temp_coef, int temp_every, hipStream_t stream);
int gibbs_rmsnorm_rows_mix_add_norm(float* x, const void* in, const int* place, const float* weight, int top, const void* shared,
                                    const float* gate, const float* gain_d, float eps_d, const float* gain_n, float eps_n, void* out,
                                    int dtype, int n, int hidden, hipStream_t stream);
int gibbs_qkv_prepare(void* rows, long ld, void* kpages, void* vpages, int dtype, const float* bias, const float* inv_freq,
                      int rot, int variant, const float* cs_table, int table_len, void* keep, int keep_mode, int vt,
                      const float* lambda, const int* pos, const int* row_req, const int* table, int max_pages, int page_size,
                      int num_pages, int n_rows, int nh, int nkv, int hd, int vd, hipStream_t stream);
int gibbs_qkv_prepare_full(void* rows, long ld, void* kpages, void* vpages, int dtype, const float* bias, const float* inv_freq,
                           int rot, int variant, const float* cs_table, int table_len, void* keep, int keep_mode, int vt,
                           const float* lambda, const int* pos, const int* row_req, const int* table, int max_pages, int page_size,
                           int num_pages, int n_rows, int nh, int nkv, int hd, int vd, const float* q_gain, const float* k_gain,
                           float qk_eps, int norm_dim, int v_from_k, const float* v_inv_freq, int v_rot, hipStream_t stream);
int gibbs_attention_finish(void* att, long ldo, const void* gate, long ld_gate, int gate_head, int dtype, const int* pos,
                           const float* v_inv_freq, int v_rot, int variant, int n_rows, int nh, int vd, int vt, hipStream_t stream);
// ---- moe.hip: mixture of experts
long gibbs_moe_capacity(int n_pairs, int E, int bm);
int gibbs_moe_tile(int n_pairs, int E);
int gibbs_moe_route(const void* h, long ldh, int dtype, const float* router, const float* router_bias, const float* shared_gate,
                    int* chosen, float* weight, float* sgate, int n, int W, int E, int top, hipStream_t stream);
int gibbs_moe_route_mode(const void* h, long ldh, int dtype, const float* router, const float* router_bias, const float* shared_gate,
                         int* chosen, float* weight, float* sgate, int n, int W, int E, int top, int mode, hipStream_t stream);
int gibbs_moe_combine_self(const void* y, const int* pair_pos, const float* weight, const void* shared, const float* sgate,
                           const void* self, void* out, int dtype, int n, int top, int W, hipStream_t stream);
int gibbs_moe_group(const int* chosen, int n_pairs, int E, int bm, int* sorted_pair, int* pair_pos, int* tile_expert, long cap,
                    hipStream_t stream);
int gibbs_moe_gemm(const void* X, long ldx, int top, const int* sorted_pair, const int* tile_expert, long cap, int bm,
                   const void* w_a, const void* w_b, void* Y, long ldy, int dtype, int O, int I, int act, hipStream_t stream);
int gibbs_moe_combine(const void* y, const int* pair_pos, const float* weight, const void* shared, const float* sgate, void* out,
                      int dtype, int n, int top, int W, hipStream_t stream);
int gibbs_causal_conv_silu(const void* in, long ld, int dtype, const float* taps, float* state, long slot_stride,
                           const int* row_req, const int* cu, const int* slot, float* out, int n_rows, int n_req, int C, int K,
                           int update_state, int single_rows, hipStream_t stream);
int gibbs_causal_conv(const void* in, long ld, int dtype, const float* taps, const float* bias, float* state, long slot_stride,
                      const int* row_req, const int* cu, const int* slot, void* out, int out_f32, long ld_out, int n_rows, int n_req,
                      int C, int K, int act, int residual, int update_state, int single_rows, hipStream_t stream);
int gibbs_ssd_prep(const float* xbc, long ld_x, const void* dt_raw, long ld_raw, int dtype, const float* dt_bias, const float* a_log,
                   float* decay, float* log_decay, float* xdt, int n_rows, int H, int V, hipStream_t stream);
// ---- ssd_chunked.hip: the same rule in chunks of 64 tokens, for one request's long stretch of rows
long gibbs_ssd_chunked_workspace(int rows, int H, int D, int V);
int gibbs_ssd_step(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* decay, float* state, long slot_stride,
                   const int* slot, float* out, int n_req, int H, int G, int D, int V, hipStream_t stream);
int gibbs_ssd_chunked(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* log_decay, float* state,
                      long slot_stride, const int* slot, float* out, float* workspace, int rows, int H, int G, int D, int V,
                      hipStream_t stream);
int gibbs_ssd_rule(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* decay, float* state,
                   long slot_stride, const int* cu, const int* slot, float* out, int n_req, int H, int G, int D, int V,
                   hipStream_t stream);
int gibbs_softcap_rows(float* v, long count, float cap, hipStream_t stream);
// ---- norm_groups.hip: RMS norm in groups
int gibbs_group_rmsnorm(float* x, const void* delta, int parts, long part_stride, const float* gain_d, float eps_d, int groups_d,
                        const float* gain_n, float eps_n, int groups_n, void* out, int dtype, const int* rows, int n_out, int H,
                        hipStream_t stream);
int gibbs_gated_group_norm(const float* in, const float* skip, long ld_skip, const float* skip_w, int skip_len, const void* gate,
                           long ld_gate, const float* gain, float eps, int groups, void* y, int dtype, int n, int C,
                           hipStream_t stream);
int gibbs_delta_prep(float* q, float* k, long ldqk, const void* beta_raw, const void* a_head, long ld_raw, int dtype,
                     const float* a_channel, const float* dt_bias, const float* a_log, float* beta, float* decay, int n_rows,
                     int G, int H, int D, float q_scale, float unit_eps, hipStream_t stream);
int gibbs_delta_rule(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* beta, const float* decay,
                     int per_channel, float* state, long slot_stride, const int* cu, const int* slot, float* out, int n_req,
                     int H, int G, int D, int V, hipStream_t stream);
int gibbs_decayed_outer_rule(const void* r, const void* k, const void* v, int dtype, const float* w, const float* bonus,
                             float* state, long slot_stride, const int* cu, const int* slot, float* out, int n_req, int H, int D,
                             hipStream_t stream);
int gibbs_head_norm_gate(const float* o, const float* gain, int gain_len, const void* gate, long ld_gate, void* y, int dtype,
                         int n_rows, int H, int V, float eps, int act, hipStream_t stream);
int gibbs_token_shift(const void* h, int dtype, const float* mu, int n_mix, float* state, long slot_stride, const int* row_req,
                      const int* cu, const int* slot, void* out, int n_rows, int n_req, int W, int update_state, int single_rows,
                      hipStream_t stream);
int gibbs_tanh_rows(const float* in, void* out, int dtype, long count, hipStream_t stream);
int gibbs_double_exp_decay(float* z, const float* bias, long count, int C, hipStream_t stream);
int gibbs_add_rmsnorm(float* x, const void* delta, const float* gain, float eps, void* out, int dtype, const int* rows,
                      int n_out, int hidden, hipStream_t stream);
int gibbs_add_partials_rmsnorm(float* x, const float* partials, int n_partials, long partial_stride, const float* gain,
                               float eps, void* out, int dtype, const int* rows, int n_out, int hidden, hipStream_t stream);
int gibbs_residual_add(float* x, const void* delta, int dtype, int n_partials, long partial_stride, void* mirror,
                       long count, hipStream_t stream);
int gibbs_gemm_f32(const float* A, const float* W, float* C, int N, int O, int I, long lda, long ldw, long ldc,
                   hipStream_t stream);
int gibbs_gemm_bf16_plain(const void* A, const void* W, void* C, int out_dtype, int N, int O, int I, long lda, long ldw,
                          long ldc, hipStream_t stream);
int gibbs_gemm_bf16(const void* A, const void* W, void* C, int out_dtype, int N, int O, int I, long lda, long ldw,
                    long ldc, hipStream_t stream);
int gibbs_gemm_library_init();
int gibbs_gemm_library(const void* A, const void* W, void* C, int N, int O, int I, long lda, long ldw, long ldc,
                       hipStream_t stream);
int gibbs_gemm_skinny(const void* X, const void* W, void* Y, int out_dtype, int N, int O, int I, long ldx, long ldw,
                      long ldy, int k_splits, hipStream_t stream);
int gibbs_skinny_store(const void* X, const void* W, void* Y, int N, int O, int I, long ldx, long ldw, long ldy, int rms,
                       float eps, hipStream_t stream);
int gibbs_skinny_residual(const void* X, const void* W, float* x, void* xb, int N, int O, int I, long ldx, long ldw,
                          hipStream_t stream);
int gibbs_skinny_glu(const void* X, const void* W, void* Y, int N, int F, int I, long ldx, long ldw, long ldy, int rms,
                     float eps, int act, hipStream_t stream);
int gibbs_skinny_glu_general(const void* X, const void* W, void* Y, int N, int F, int I, long ldx, long ldw, long ldy, int rms,
                             float eps, int act, float alpha, float limit, hipStream_t stream);
int gibbs_skinny_conv(const void* X, const void* W, void* Y, int N, int C, int I, long ldx, long ldw, int rms, float eps,
                      const float* taps, const float* bias, float* state, long slot_stride, const int* slot,
                      const int* ctx, int K, hipStream_t stream);
int gibbs_glu(const void* gu, void* out, int dtype, int n, int F, int act, hipStream_t stream);
int gibbs_shortconv(const void* bcx, const float* taps, const float* bias, float* state, long slot_stride, const int* cu,
                    const int* ctx, const int* slot, void* y, int dtype, int n_rows, int n_req, int lead_single, int C, int K,
                    hipStream_t stream);
int gibbs_qk_rope_kv(void* qkv, void* kpages, void* vpages, int dtype, const float* q_gain, const float* k_gain, float eps,
                     const float* inv_freq, int rot, int variant, const float* cs_table, int table_len, const int* pos,
                     const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh,
                     int nkv, int hd, long ld, hipStream_t stream);
int gibbs_attention_plain(const void* q, const void* kpages, const void* vpages, void* out, int dtype, const int* pos,
                          const int* row_req, const int* table, int max_pages, int page_size, int num_pages, int n_rows,
                          int nh, int nkv, int hd, long ldq, long ldo, float scale, int window, const float* slopes,
                          hipStream_t stream);
int gibbs_attention_prefill(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                            const int* cu, const int* ctx, const int* table, int n_req, int max_pages, int page_size,
                            int num_pages, int n_rows, int nh, int nkv, int hd, long ldq, long ldo, float scale, int window,
                            int n_splits, int first_row, int heads_per_wg, hipStream_t stream);
int gibbs_attention_prefill_bias(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                                 const int* cu, const int* ctx, const int* table, int n_req, int max_pages, int page_size,
                                 int num_pages, int n_rows, int nh, int nkv, int hd, long ldq, long ldo, float scale, int window,
                                 int n_splits, int first_row, int heads_per_wg, const float* bias, int bias_len, hipStream_t stream);
int gibbs_attention_decode_fused(const void* qkv, void* kpages, void* vpages, void* out, float* partial,
                                 const float* q_gain, const float* k_gain, float eps, const float* inv_freq, int rot,
                                 int variant, const float* cs_table, int table_len, const int* pos, const int* row_req,
                                 const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh, int nkv,
                                 int hd, long ld, long ldo, float scale, int window, int n_splits, int waves, int kind,
                                 int max_keys, hipStream_t stream);
int gibbs_argmax(const float* logits, int* out, int M, int V, long ld, hipStream_t stream);
int gibbs_sample(const float* logits, int* out, int M, int V, long ld, const float* temperature, const float* top_p,
                 const int* top_k, const float* u, hipStream_t stream);
int gibbs_decode_tail(const float* logits, int V, long ld, int* ids, int* pos, int* ctx, int* log, int* steps, int n,
                      int capacity, float* u, const float* u_all, const void* table, int table_dtype, int vocab, int hidden,
                      float* x, void* mirror, const int* live, hipStream_t stream);
}

// Inside the library only: gibbs_skinny_store with the output's type given (bfloat16 or float32); what
// gibbs_gemm_skinny hands whole sums of up to 16 rows to (gemm_skinny_fused.hip).
int gibbs_skinny_store_as(const void* X, const void* W, void* Y, int out_dtype, int N, int O, int I, long ldx, long ldw,
                          long ldy, int rms, float eps, hipStream_t stream);
