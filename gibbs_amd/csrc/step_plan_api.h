// C interface of the native step (step_plan.hip): a model's step laid down once as a program of
// operations over parts, then run as one call per step.
//
// A plan holds parts (norms; bodies: what reads normed rows and gives a delta for the residual stream,
// a mixer or a feed-forward) and a program of operations over them.  The parts that the library brings
// are made by gibbs_plan_norm_rms / gibbs_plan_body_conv / _attention / _glu; a part from anywhere else
// is a function pointer with a user pointer (gibbs_plan_norm_host / gibbs_plan_body_host): code of
// another library, or a callback into an interpreter.  The program says how a layer arranges its parts;
// every function that appends to it returns the index of what it made, or -1 with the reason in
// gibbs_last_error().
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// One step's operands (the integer metadata lives on the device already).
struct GibbsStepArgs {
  const int* ids;          // [n_rows]
  const int* pos;          // [n_rows]
  const int* row_req;      // [n_rows]
  const int* cu;           // [n_req + 1]
  const int* ctx;          // [n_req]
  const int* slot;         // [n_req]
  const int* logit_rows;   // [n_logits]
  const int* const* tables;   // per cache group: [n_req, widths[g]] page ids
  const int* widths;
  int n_groups;
  int n_rows, n_req, n_logits, max_q, max_seq, lead_single;
  void* workspace;         // device memory for the step's activations (null: only count the bytes)
  long workspace_bytes;
  float* logits;           // [n_logits, vocab] float32 out
  hipStream_t stream;
  // A step that continues a captured decode loop: the rows' embeddings are there already (the end of the
  // previous step wrote them), as the float32 stream x_in [n_rows, hidden] and, for steps that take the fused
  // decode kernels, its bfloat16 mirror.  Null: the step embeds its ids itself.
  float* x_in;
  void* mirror_in;
  // The operations to run (n_ops 0: all of them, then the final norm and the head for the wanted rows), and
  // whether a delta that is still pending at the end is added into x (for a caller that reads x).
  int first_op, n_ops, settle;
};

// out [n_rows, hidden] (the run's activation type) = body(h [n_rows, hidden]); queued on step->stream.
typedef int (*GibbsHostBody)(void* user, const struct GibbsStepArgs* step, const void* h, void* out);
// x (+= delta, when all rows are normed: rows null); out [n_out, hidden] = norm of the rows (all, or `rows`).
// delta: null, [n_rows, hidden] in the activation type (delta_parts 1), or float32 [delta_parts, n_rows, hidden].
typedef int (*GibbsHostNorm)(void* user, const struct GibbsStepArgs* step, float* x, const void* delta, int delta_parts,
                             const int* rows, int n_out, void* out);
// q and k rows of a step, in place, after the q/k norm and before k is cached: qkv [n_rows, ld] in the activation type.
typedef int (*GibbsHostRows)(void* user, const struct GibbsStepArgs* step, void* qkv, long ld);

// dtype: GIBBS_F32 (0) or GIBBS_BF16 (1), of activations, matrices and cache pages.  table / head may be null
// for a plan that only runs parts (no embedding, no logits).
void* gibbs_plan_create(int dtype, int hidden, int vocab, const void* table, int table_dtype, const void* head,
                        const void* head_packed, int fused_rows, int own_gemm);
void gibbs_plan_destroy(void* plan);

// ---- parts
int gibbs_plan_norm_rms(void* plan, const float* gain, float eps);     // gain null: folded into the matrices that follow
int gibbs_plan_norm_host(void* plan, GibbsHostNorm fn, void* user);
int gibbs_plan_body_conv(void* plan, const void* w_in, const void* p_in3, const void* w_out, const void* p_out,
                         const float* taps, const float* bias, int C, int K, float* state, long slot_stride);
int gibbs_plan_body_attention(void* plan, const void* w_qkv, const void* p_qkv, const void* w_out, const void* p_out, int nh,
                              int nkv, int hd, float scale, int window, const float* q_gain, const float* k_gain,
                              float qk_eps, const float* inv_freq, int rot, int variant, const float* cos_sin,
                              int table_len, void* kpages, void* vpages, int num_pages, int page_size, int group,
                              int owns, const float* slopes, GibbsHostRows hook, void* hook_user);
int gibbs_plan_body_glu(void* plan, const void* w_gate_up, const void* p_gate_up2, const void* w_down, const void* p_down,
                        int F, int act);
int gibbs_plan_body_host(void* plan, GibbsHostBody fn, void* user, int group);   // group: the cache group it reads, or -1

// The embedding: rows of the table times `scale`, plus (inv_freq [hidden / 2] not null) a sinusoidal position vector,
// sin(pos * inv_freq[i]) at the even entries 2i and the cosines of the same angles at the odd entries 2i + 1.
int gibbs_plan_embedding(void* plan, float scale, const float* inv_freq);
// An attention body without rotation and q/k gains may have: values of head size vd; q and k divided by their root
// mean square per head (unit_qk, with the body's qk_eps; the mean over the first norm_dim channels of a head, which may
// be stored wider with zeros behind them; 0: the head size); q times 1 + temp_coef * log(1 + (pos + 1) div temp_every)
// (temp_every 0: none); bias [bias_len, heads] added to the scores by distance (the last row for all longer ones),
// and the same table as bias_t [heads, bias_len] divided by the scale (null: the matrix-core kernels are not used).
// Projected rows are then [q: nh*hd | k: nkv*hd | v: nkv*vd].
int gibbs_plan_attention_extras(void* plan, int body, int vd, int unit_qk, int norm_dim, float temp_coef, int temp_every,
                                const float* bias, const float* bias_t, int bias_len);
// An attention body with a rotation (or none) may have: values of head size vd; bias [qkv rows] (float32) added to the
// projected rows; sink [heads]: a term exp(sink[h]) in the softmax's denominator without key or value; value mixing:
// keep_mode 1 publishes the step's values (the first vt channels of every value head) under keep_key for later layers,
// keep_mode 2 mixes what was published under keep_key into its own, v <- (1 - *lambda) v + *lambda v_published, before they
// are cached.  Projected rows are then [q: nh*hd | k: nkv*hd | v: nkv*vd].
int gibbs_plan_attention_projection(void* plan, int body, int vd, const float* bias, const float* sink, int keep_mode,
                                    int keep_key, int vt, const float* lambda);
// Mixture of experts: router [experts, hidden] and router_bias [experts] (float32); gate, up [experts, F, hidden] and down
// [experts, hidden, F]; every row takes its `top` experts with the largest logits, weighted by the softmax over those
// logits; expert: down(act(gate h) * (up h)).  A shared expert (shared_gate_up [2 shared_F, hidden], shared_down [hidden,
// shared_F]; null: none) runs for every row and is added, times sigmoid(shared_gate . h) (shared_gate [hidden] float32;
// null: times 1).
struct GibbsMoeSpec {
  const float* router; const float* router_bias;
  const void* gate; const void* up; const void* down;
  const void* shared_gate_up; const void* shared_down; const float* shared_gate;
  int experts, top, F, act, shared_F, shared_act;
};
int gibbs_plan_body_moe(void* plan, const struct GibbsMoeSpec* spec);
// A gated feed-forward body computes min(gate, limit) * sigmoid(alpha * .) * (clamp(up, -limit, limit) + 1) instead.
int gibbs_plan_glu_clamped(void* plan, int body, float alpha, float limit);

// Gated delta rule with short convolutions.  w_in [in_rows, hidden]: the rows of q (kv_heads*dim), k (the same), v
// (heads*vdim), then at off_b the heads rows of beta's projection, at off_a the decay's (heads rows, or a_rank rows of
// the first matrix of a low-rank pair whose second is w_a2 [heads*dim, a_rank]: one decay per key channel), at off_g the
// gate's (heads*vdim rows and silu, or g_rank rows and w_g2 [heads*vdim, g_rank] and sigmoid).  taps [2 kv_heads dim +
// heads vdim, taps_per_channel], the last one the current token's.
struct GibbsDeltaSpec {
  const void* w_in; const void* w_out; const void* w_a2; const void* w_g2;
  const float* taps; const float* dt_bias; const float* a_log; const float* gain;
  float* conv_state; float* rule_state; long slot_stride;
  int in_rows, heads, kv_heads, dim, vdim, taps_per_channel, off_b, off_a, off_g, a_rank, g_rank;
  float eps, unit_eps, q_scale;
};
int gibbs_plan_body_delta(void* plan, const struct GibbsDeltaSpec* spec);

// Time mixing with a decayed outer-product state.  w_r, w_k, w_v, w_g [heads*dim, hidden], w_1 [rank, hidden], w_2
// [heads*dim, rank], w_out [hidden, heads*dim]; mu [5, hidden] (r, k, v, g, w); w0, gain [heads*dim]; bonus [heads, dim].
struct GibbsTimeMixSpec {
  const void* w_r; const void* w_k; const void* w_v; const void* w_g; const void* w_1; const void* w_2; const void* w_out;
  const float* mu; const float* w0; const float* bonus; const float* gain;
  float* shift_state; float* rule_state; long slot_stride;
  int heads, dim, rank;
  float eps;
};
int gibbs_plan_body_time_mix(void* plan, const struct GibbsTimeMixSpec* spec);

// An attention body that takes the projection options (gibbs_plan_attention_projection first) may further have: q and k
// divided per head by their root mean square over the first norm_dim channels and multiplied by a gain [norm_dim], before the
// rotation; values that are the keys as projected, unnormed and unrotated (v_from_k: the projection has no value rows);
// values turned by their position over their first v_rot channels (pairs as the rotation's variant says, pair m by
// pos * v_inv_freq[m]) before they are cached, and every head's output turned back by its row's position; chunks (a row
// sees the keys of its own stretch of `chunk` positions, counted from 0) instead of a window; scores capped as
// softcap * tanh(s / softcap); and a gate: nh * vd further projected columns whose sigmoid multiplies the heads' outputs.
// Projected rows are then [q: nh*hd | k: nkv*hd | v: nkv*vd (unless v_from_k) | gate: nh*vd (if gate)].
int gibbs_plan_attention_gated(void* plan, int body, const float* q_gain, const float* k_gain, float qk_eps, int norm_dim,
                               int v_from_k, const float* v_inv_freq, int v_rot, int chunk, float softcap, int gate);
// RMS norm in `groups` equal consecutive parts of the row (each divided by its own root mean square), times gain [hidden].
int gibbs_plan_norm_group_rms(void* plan, const float* gain, float eps, int groups);
// A short causal convolution beside the identity, per channel of the model's width: rows -> rows + conv(rows), taps
// [hidden, K] (the last one the current token's), the requests' last K - 1 rows in state [slots][K - 1][hidden].
int gibbs_plan_body_conv_input(void* plan, const float* taps, int K, float* state, long slot_stride);
// State-space mixer.  w_in [2 inner + 2 groups state + heads, hidden] with inner = heads * vdim, rows [z | x | B | C | dt];
// taps [inner + 2 groups state, taps_per_channel] and conv_bias over x, B, C; dt_bias, a_log, skip [heads]; gain [inner];
// the gated read-out is normed in norm_groups parts.  States: conv_state [slots][taps - 1][inner + 2 groups state], rule_state
// [slots][heads][state][vdim], float32.
struct GibbsSsdSpec {
  const void* w_in; const void* w_out;
  const float* taps; const float* conv_bias; const float* dt_bias; const float* a_log; const float* skip; const float* gain;
  float* conv_state; float* rule_state; long slot_stride;
  int heads, vdim, state, groups, taps_per_channel, norm_groups;
  float eps;
};
int gibbs_plan_body_ssd(void* plan, const struct GibbsSsdSpec* spec);
// logits <- cap * tanh(logits / cap) after the head (0: not capped).
int gibbs_plan_logit_softcap(void* plan, float cap);
// A mixture of experts' router: mode 0 as described above; mode 1: scores s = softmax over all router outputs, the `top`
// largest of s + router_bias are chosen, their weights are their scores s over the sum of those (+ 1e-20).  The router
// then has experts + identity outputs, the last `identity` of which are experts without matrices that return their input.
int gibbs_plan_moe_scores(void* plan, int body, int mode, int identity);

// Layer norm with gain and bias (either may be null: 1 and 0).
int gibbs_plan_norm_layer(void* plan, const float* gain, const float* bias, float eps);

// Latent attention: one cached row [latent (rank) | rotated key part (rot)] per token, shared by all heads.  w_in
// [in_rows, hidden]: the rows of the queries (heads * (dim + rot); or, with w_uq [heads * (dim + rot), q_rank], the q_rank
// rows of the queries' own latent, which is RMS-normed with q_gain), at off_kv the rank + rot rows of the keys' and values'
// down-projection (the first rank RMS-normed with kv_gain), at off_g (< 0: none) the heads * vdim rows of a sigmoid gate on
// the heads' outputs.  w_uk_t [heads, rank, dim]: every head's key up-projection, transposed; w_uv [heads * vdim, rank].
// A query head is [dim unrotated | rot rotated]; the first rot_dims entries of a rotated part turn with the position
// (variant 0: pairs (i, i + rot_dims / 2), 1: pairs (2 i, 2 i + 1); inv_freq [rot_dims / 2]).  window 0: all keys;
// sink [heads] or null: a term exp(sink[h]) in the softmax's denominator.  pages: [num_pages, page_size, rank + rot].
struct GibbsLatentSpec {
  const void* w_in; const void* w_uq; const void* w_uk_t; const void* w_uv; const void* w_out;
  const float* q_gain; const float* kv_gain; const float* sink; const float* inv_freq;
  void* pages;
  int in_rows, heads, dim, rot, vdim, rank, q_rank, rot_dims, variant, window, off_kv, off_g, num_pages, page_size, group;
  float scale, eps;
};
int gibbs_plan_body_latent(void* plan, const struct GibbsLatentSpec* spec);
// Dense feed-forward without a gate: down(act(up h)), act(z) = a N(z) + b N(z^2) + c N(z^3) + e with coef = [a, b, c, e]
// on the device and N the division of a row by its root mean square (eps inside the root).
int gibbs_plan_body_mlp(void* plan, const void* w_up, const void* w_down, int F, const float* coef, float eps);

// Several residual streams (1 to 8): every stream starts as the embedding's output, sublayers read and write them
// through hyper-connections (in [streams], mix [streams, streams] indexed [from][to], out [streams]), and the model's
// output is the streams' sum.
int gibbs_plan_streams(void* plan, int streams);
int gibbs_plan_hyper(void* plan, const float* in, const float* mix, const float* out);
// Rows of further tables added to the token table's: pair_table [buckets + 1, hidden], row (previous token * mul_prev +
// token * mul_cur) mod buckets, row `buckets` for a sequence's first token (the previous token of a request's earlier step
// lives at prev_state[slot * prev_stride]); pos_table [pos_len, hidden], row = position.  Either may be null.
int gibbs_plan_embedding_tables(void* plan, const void* pair_table, int buckets, int mul_prev, int mul_cur,
                                const void* pos_table, int pos_len, int* prev_state, long prev_stride);

// ---- the program (values are normed rows or deltas, named by the index their operation returns)
int gibbs_plan_op_half(void* plan, int norm, int body);       // x += body(norm(x)), in fused kernels where it can
int gibbs_plan_op_norm(void* plan, int norm);                 // -> value: norm(x + what is pending)
int gibbs_plan_op_body(void* plan, int body, int value);      // -> value: body(normed rows)
int gibbs_plan_op_rows(void* plan, int body, int value);      // -> value: body(normed rows), read as rows by a later body
int gibbs_plan_op_add(void* plan, int value);                 // x += delta (lazily: it stays pending for the next norm)
int gibbs_plan_op_drop(void* plan, int value);                // the value is not read again
int gibbs_plan_op_norm_delta(void* plan, int norm, int value);   // -> value: norm(a body's delta), the stream untouched
int gibbs_plan_op_add_normed(void* plan, int norm, int value);   // x += norm(a body's delta), in one pass where the norm can
int gibbs_plan_op_streams_norm(void* plan, int norm, int hyper);   // -> value: norm(sum_s in[s] x_s)
int gibbs_plan_op_streams_add(void* plan, int hyper, int value);   // x_t <- sum_s mix[s][t] x_s + out[t] delta, all t at once
int gibbs_plan_op_reinject(void* plan);                       // x += the embedding's output (what the step's first operation saw)
int gibbs_plan_tail(void* plan, int norm);                    // the norm in front of the head
int gibbs_plan_op_count(const void* plan);

// ---- running
long gibbs_plan_workspace(const void* plan, const struct GibbsStepArgs* args);   // bytes of workspace the step needs
int gibbs_plan_step(const void* plan, const struct GibbsStepArgs* args);
int gibbs_plan_last_fused(const void* plan);   // halves of the last step that ran as fused decode kernels
// One part alone.  args->workspace null: returns the bytes of workspace needed.  Else runs it and returns 0 (non-zero:
// failed), with the result at *out_offset bytes into the workspace: [parts, n_rows, hidden] float32 partial sums when
// *parts >= 2, else [n_rows, hidden] in the activation type.
long gibbs_plan_body_forward(const void* plan, int body, const struct GibbsStepArgs* args, const void* h, long* out_offset,
                             int* parts);
long gibbs_plan_norm_forward(const void* plan, int norm, const struct GibbsStepArgs* args, float* x, const void* delta,
                             int delta_parts, const int* rows, int n_out, long* out_offset);

// ---- the dispatch rules, for callers that run a kernel by itself
int gibbs_rule_skinny_splits(int n_out, int inner, int want_blocks, int features, int min_k);
void gibbs_rule_decode_splits(int n_rows, int nkv, int group, int max_seq, int hd, int page_size, int kind, int* n_splits,
                              int* waves);
long gibbs_rule_prefill_tiles(int rows, int reqs);            // query tiles that the rows of a ragged batch make
int gibbs_rule_prefill_splits(long n_tiles, int nh, int max_seq, int window);
int gibbs_rule_prefill_heads(int rows, int reqs, int nh, int nkv, int hd, int max_seq, int n_splits);   // query heads a workgroup
int gibbs_rule_fused_rows(void);                              // rows that the fused decode kernels take at most
// y = x W^T the way a step would run it.  gibbs_linear_splits: the float32 partial sums it would leave (1: the
// finished product [n, O]; s >= 2: [s, n, O] float32).  gibbs_linear: runs it into y (sized by that answer).
int gibbs_linear_splits(int dtype, int n, int O, int I, long ldx, const void* x, const void* w, int out_f32, int partial_ok,
                        int own_gemm);
int gibbs_linear(const void* x, long ldx, const void* w, const void* packed, void* y, int dtype, int n, int O, int I,
                 int out_f32, int partial_ok, int own_gemm, hipStream_t stream);
// x += y W^T, mirror = bfloat16(x), for up to 64 rows: floats of workspace that the route for these sizes needs (0:
// none), and the product itself (ldw 0: W in tile order).
long gibbs_skinny_residual_workspace(int n, int O, int I);
int gibbs_skinny_residual_routed(const void* y, const void* w, long ldw, float* x, void* mirror, int n, int O, int I,
                                 float* workspace, hipStream_t stream);

#ifdef __cplusplus
}
#endif
