// Kernels of mixers that carry a matrix state from token to token: the gated delta rule and the
// decayed outer-product rule of RWKV-style time mixing, with what surrounds them (short causal
// convolutions with state, unit vectors, decays, the shift by one token, the gated norm of a head's
// read-out).  Everything that enters a recurrence is float32, and so is the state.
//
// A step's rows are a ragged batch: request r brings rows cu[r] .. cu[r+1]-1 and keeps its state in
// slot[r] of the arena.  Every kernel treats a token the same way wherever its step was cut: the
// recurrences walk a request's rows in order with a fixed order of additions per token, so a prompt
// in one step, in portions or token by token gives the same bits.
#include "common.h"
#include "lane8.h"

namespace {
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float activate_gate(float z, int act) {   // 0: silu, 1: sigmoid
  return act == 1 ? sigmoid_f(z) : z * sigmoid_f(z);
}

// ------------------------------------------------------------------------------------------------ short causal convolution
// y[n, c] = act(sum_j taps[c, j] * x[t - (K-1) + j, c] + bias[c]) (+ x[t, c]): the last tap is the current token's; inputs
// before the step's first row come from the request's state (its last K-1 inputs, oldest first; zeros at a sequence's
// start).  act: silu or none; `residual`: the input itself is added to the result (a convolution beside the identity).
enum { CONV_ACT_NONE = 0, CONV_ACT_SILU = 1 };
template <typename T, typename TO>
__global__ void causal_conv_silu_kernel(const T* __restrict__ in, long ld, const float* __restrict__ taps, const float* __restrict__ bias,
                                        float* __restrict__ state, long slot_stride, const int* __restrict__ row_req,
                                        const int* __restrict__ cu, const int* __restrict__ slot, TO* __restrict__ out, long ld_out,
                                        int C, int K, int shift_state, int act, int residual) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r = row_req[n], first = cu[r], t = n - first;
  float* st = state + (size_t)slot[r] * slot_stride;
  float acc = 0.f, own = 0.f;
  for (int j = 0; j < K; ++j) {
    const int tt = t - (K - 1) + j;
    const float xv = tt >= 0 ? to_float(in[(size_t)(first + tt) * ld + c]) : st[(size_t)(K - 1 + tt) * C + c];
    acc = fmaf(taps[(size_t)c * K + j], xv, acc);
    own = xv;
    // every request brings one row (shift_state): this thread is the only one that reads or writes the request's
    // inputs of this channel, so it moves them on itself (entry j - 1 has been read already)
    if (shift_state && j >= 1) st[(size_t)(j - 1) * C + c] = xv;
  }
  if (bias) acc += bias[c];
  if (act == CONV_ACT_SILU) acc = acc * sigmoid_f(acc);
  if (residual) acc += own;
  out[(size_t)n * ld_out + c] = from_float<TO>(acc);
}

// The same for bfloat16 inputs whose channels come in whole groups of 8: a thread takes 8 neighbouring channels of a row with
// 16-byte loads.  A workgroup is 64 lanes of channels by CONV_ROWS rows; the taps of its 512 channels, one contiguous stretch of
// the [C, K] table, come into LDS once (each thread's 8 K taps a word further along, so that the lanes read different banks)
// instead of as 8 K scattered words per thread.  Sums in ascending j, as above.
constexpr int CONV_ROWS = 4, CONV_LANES = 64;
template <typename TO>
__global__ __launch_bounds__(CONV_ROWS * CONV_LANES) void causal_conv_vec8_kernel(
    const bf16* __restrict__ in, long ld, const float* __restrict__ taps, const float* __restrict__ bias, float* __restrict__ state,
    long slot_stride, const int* __restrict__ row_req, const int* __restrict__ cu, const int* __restrict__ slot, TO* __restrict__ out,
    long ld_out, int n_rows, int C, int K, int shift_state, int act, int residual) {
  extern __shared__ float s_taps[];    // [CONV_LANES][8 K + 1]
  const int c0 = blockIdx.y * CONV_LANES * 8;
  const int span = min(CONV_LANES * 8, C - c0) * K;      // taps of this workgroup's channels
  const int tid = threadIdx.y * CONV_LANES + threadIdx.x;
  for (int i = tid; i < span; i += CONV_ROWS * CONV_LANES) s_taps[i + i / (8 * K)] = taps[(size_t)c0 * K + i];
  __syncthreads();
  const int n = blockIdx.x * CONV_ROWS + threadIdx.y;
  const int c = c0 + threadIdx.x * 8;
  if (n >= n_rows || c >= C) return;
  const float* tp = s_taps + threadIdx.x * (8 * K + 1);
  const int r = row_req[n], first = cu[r], t = n - first;
  float* st = state + (size_t)slot[r] * slot_stride;
  float acc[8] = {}, own[8] = {};
  for (int j = 0; j < K; ++j) {
    const int tt = t - (K - 1) + j;
    float xv[8];
    if (tt >= 0) {
      unpack8(*(const uint4*)(in + (size_t)(first + tt) * ld + c), xv);
    } else {
      const float4 a = *(const float4*)(st + (size_t)(K - 1 + tt) * C + c), b = *(const float4*)(st + (size_t)(K - 1 + tt) * C + c + 4);
      xv[0] = a.x; xv[1] = a.y; xv[2] = a.z; xv[3] = a.w; xv[4] = b.x; xv[5] = b.y; xv[6] = b.z; xv[7] = b.w;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[i] = fmaf(tp[i * K + j], xv[i], acc[i]);
      own[i] = xv[i];
    }
    if (shift_state && j >= 1) {
      *(float4*)(st + (size_t)(j - 1) * C + c) = make_float4(xv[0], xv[1], xv[2], xv[3]);
      *(float4*)(st + (size_t)(j - 1) * C + c + 4) = make_float4(xv[4], xv[5], xv[6], xv[7]);
    }
  }
  if (bias) {
    const float4 b0 = *(const float4*)(bias + c), b1 = *(const float4*)(bias + c + 4);
    acc[0] += b0.x; acc[1] += b0.y; acc[2] += b0.z; acc[3] += b0.w; acc[4] += b1.x; acc[5] += b1.y; acc[6] += b1.z; acc[7] += b1.w;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (act == CONV_ACT_SILU) acc[i] = acc[i] * sigmoid_f(acc[i]);
    if (residual) acc[i] += own[i];
  }
  TO* o = out + (size_t)n * ld_out + c;
  if constexpr (sizeof(TO) == 2) {
    *(uint4*)o = pack8(acc);
  } else {
    *(float4*)o = make_float4(acc[0], acc[1], acc[2], acc[3]);
    *(float4*)(o + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
  }
}

// The state after the step: the last K-1 inputs of the request (what the step brought, and before that what
// the state held).  One thread per (request, channel), entries in ascending order: entry i reads entry
// i + rows of the old state, which has not been written yet.
template <typename T>
__global__ void causal_conv_state_kernel(const T* __restrict__ in, long ld, float* __restrict__ state, long slot_stride,
                                         const int* __restrict__ cu, const int* __restrict__ slot, int C, int K) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int first = cu[r], rows = cu[r + 1] - first;
  float* st = state + (size_t)slot[r] * slot_stride;
  for (int i = 0; i < K - 1; ++i) {
    const int src = i + rows - (K - 1);
    st[(size_t)i * C + c] = src >= 0 ? to_float(in[(size_t)(first + src) * ld + c]) : st[(size_t)(i + rows) * C + c];
  }
}

// ------------------------------------------------------------------------------------------------ what the delta rule reads
struct DeltaPrepArgs {
  float* q;            // [N, G*D] float32, in place: unit vector * q_scale
  float* k;            // [N, G*D] in place: unit vector
  long ldqk;
  const void* beta_raw;   // [N, ld_raw] in the activation type: W_b h
  long ld_raw;
  const void* a_head;     // head decay: [N, ld_raw] activation type, one per head (null with a_channel)
  const float* a_channel; // channel decay: [N, H*D] float32
  const float* dt_bias;   // [H] or [H*D]
  const float* a_log;     // [H]
  float* beta;            // [N, H]
  float* decay;           // [N, H] or [N, H*D]
  int G, H, D;
  float q_scale, unit_eps;
};

// Block y < G: q and k of kv head y become unit vectors x / sqrt(sum x^2 + eps) (q times q_scale).  Block
// y >= G: head y - G's beta = sigmoid(.) and decay = exp(-rate * softplus(a + dt_bias)) with rate = exp(A_log).
template <typename T>
__global__ __launch_bounds__(64) void delta_prep_kernel(DeltaPrepArgs a) {
  const int n = blockIdx.x, lane = threadIdx.x;
  if ((int)blockIdx.y < a.G) {
    const int g = blockIdx.y;
    float* q = a.q + (size_t)n * a.ldqk + (size_t)g * a.D;
    float* k = a.k + (size_t)n * a.ldqk + (size_t)g * a.D;
    float sq = 0.f, sk = 0.f;
    for (int i = lane; i < a.D; i += WAVE) {
      sq = fmaf(q[i], q[i], sq);
      sk = fmaf(k[i], k[i], sk);
    }
    const float rq = a.q_scale / sqrtf(wave_sum(sq) + a.unit_eps), rk = 1.0f / sqrtf(wave_sum(sk) + a.unit_eps);
    for (int i = lane; i < a.D; i += WAVE) {
      q[i] *= rq;
      k[i] *= rk;
    }
    return;
  }
  const int h = blockIdx.y - a.G;
  const float rate = expf(a.a_log[h]);
  if (lane == 0) a.beta[(size_t)n * a.H + h] = sigmoid_f(to_float(((const T*)a.beta_raw)[(size_t)n * a.ld_raw + h]));
  if (a.a_channel) {
    for (int i = lane; i < a.D; i += WAVE) {
      const size_t at = (size_t)n * a.H * a.D + (size_t)h * a.D + i;
      a.decay[at] = expf(-rate * softplus_f(a.a_channel[at] + a.dt_bias[h * a.D + i]));
    }
  } else if (lane == 0) {
    const float z = to_float(((const T*)a.a_head)[(size_t)n * a.ld_raw + h]) + a.dt_bias[h];
    a.decay[(size_t)n * a.H + h] = expf(-rate * softplus_f(z));
  }
}

// ------------------------------------------------------------------------------------------------ the recurrences
enum { RULE_DELTA = 0, RULE_OUTER = 1, RULE_SSD = 2 };
struct RecurrenceArgs {
  const void* q;       // delta: unit q * scale; outer: the receptance r.  [N, G*D]
  const void* k;       // [N, G*D]
  const void* v;       // [N, H*V]
  long ldq, ldk, ldv;
  const float* decay;  // delta: g [N, H] (per_channel 0) or [N, H*D]; outer: w [N, H*D]
  int per_channel;
  const float* beta;   // delta: [N, H]
  const float* bonus;  // outer: u [H, D], for the current token only
  float* state;        // [slots][H][D][V] float32
  long slot_stride;
  const int* cu;
  const int* slot;
  float* out;          // [N, H*V] float32
  int H, G, D, V;
};

// One wave per (request, head, COLS columns of the state).  A column of S [D, V] is spread over PARTS lanes (lane
// part p holds the DPT key channels p DPT .. p DPT + DPT - 1 in registers; COLS = 64 / PARTS), so that a head
// gives many short waves instead of a few long ones: the walk over a request's tokens is a chain in which every
// token waits for the one before, and what fills the chip is the number of independent chains.  Sums over the
// key channels are folded over the PARTS lanes.  The operands of 8 tokens at a time go through LDS; the next 8
// are on their way from memory into registers meanwhile.
// With M the state [D, V], ' for transposed and .* for element by element along the key channels:
//   delta:  M = decay * M;  w = beta * (v - M' k);  M = M + k w';  read = M' q
//   outer:  read = (M + (bonus .* k) v')' r;  M = decay .* M (row by row) + k v'
//   ssd:    M = decay * M + k v';  read = M' q      (the delta rule without its correction and with beta = 1)
// CH: the decay is one per key channel (always so for the outer rule); else one per head.
template <typename TIn, int RULE, int DPT, int PARTS, bool CH>
__global__ __launch_bounds__(64) void recurrence_kernel(RecurrenceArgs a) {
  constexpr int COLS = WAVE / PARTS, TOK = 8, DMAX = DPT * PARTS, LDP = DPT + 4, PER_LANE = TOK * DMAX / WAVE;
  constexpr int V_PER_LANE = (TOK * COLS + WAVE - 1) / WAVE;
  static_assert(DPT % 4 == 0 && TOK * DMAX % WAVE == 0, "a lane reads its channels four at a time");
  __shared__ __attribute__((aligned(16))) float sq[TOK][PARTS][LDP], sk[TOK][PARTS][LDP], sd[TOK][PARTS][LDP];
  __shared__ float sv[TOK][COLS], sb[TOK], sg[TOK], so[TOK][COLS];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int col = lane / PARTS, part = lane % PARTS;
  const int j = blockIdx.z * COLS + col;
  const int kvh = h / (a.H / a.G);
  const int first = a.cu[r], rows = a.cu[r + 1] - first;
  const int D = a.D, V = a.V;
  float* st = a.state + (size_t)a.slot[r] * a.slot_stride + (size_t)h * D * V;
  float S[DPT], bonus[DPT];
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) {
    const int i = part * DPT + ii;
    S[ii] = (i < D && j < V) ? st[(size_t)i * V + j] : 0.f;
    bonus[ii] = (RULE == RULE_OUTER && i < D) ? a.bonus[(size_t)h * D + i] : 0.f;
  }
  const TIn* q = (const TIn*)a.q;
  const TIn* k = (const TIn*)a.k;
  const TIn* v = (const TIn*)a.v;
  constexpr bool channel_decay = CH;
  // the next 8 tokens' operands, in registers until the current 8 are done with LDS
  float rq[PER_LANE], rk[PER_LANE], rd[PER_LANE], rv[V_PER_LANE], rb = 0.f, rg = 1.f;
  auto ask = [&](int t0) {
    const int nt = min(TOK, rows - t0);
#pragma unroll
    for (int e = 0; e < PER_LANE; ++e) {
      const int idx = e * WAVE + lane, t = idx / DMAX, i = idx % DMAX;
      const bool live = t < nt && i < D;
      const size_t row = (size_t)(first + t0 + (t < nt ? t : 0));
      const int ic = i < D ? i : 0;
      rq[e] = live ? to_float(q[row * a.ldq + (size_t)kvh * D + ic]) : 0.f;
      rk[e] = live ? to_float(k[row * a.ldk + (size_t)kvh * D + ic]) : 0.f;
      rd[e] = (channel_decay && live) ? a.decay[row * a.H * D + (size_t)h * D + ic] : 1.f;
    }
#pragma unroll
    for (int e = 0; e < V_PER_LANE; ++e) {
      const int idx = e * WAVE + lane, t = idx / COLS, jj = blockIdx.z * COLS + idx % COLS;
      rv[e] = (t < nt && jj < V) ? to_float(v[(size_t)(first + t0 + t) * a.ldv + (size_t)h * V + jj]) : 0.f;
    }
    if (RULE != RULE_OUTER && lane < TOK) {
      const bool live = lane < nt;
      const size_t row = (size_t)(first + t0 + (live ? lane : 0));
      rb = (live && RULE == RULE_DELTA) ? a.beta[row * a.H + h] : 0.f;
      rg = (live && !a.per_channel) ? a.decay[row * a.H + h] : 1.f;
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int e = 0; e < PER_LANE; ++e) {
      const int idx = e * WAVE + lane, t = idx / DMAX, i = idx % DMAX;
      sq[t][i / DPT][i % DPT] = rq[e];
      sk[t][i / DPT][i % DPT] = rk[e];
      sd[t][i / DPT][i % DPT] = rd[e];
    }
#pragma unroll
    for (int e = 0; e < V_PER_LANE; ++e) {
      const int idx = e * WAVE + lane;
      if (idx < TOK * COLS) sv[idx / COLS][idx % COLS] = rv[e];
    }
    if (RULE != RULE_OUTER && lane < TOK) {
      sb[lane] = rb;
      sg[lane] = rg;
    }
  };
  // (the PARTS lanes of a column are neighbours within a row of 16 lanes: data-parallel moves, a few cycles each)
  auto fold = [&](float x) { return group_sum<PARTS>(x); };
  // The read-outs of 8 tokens leave together, right after the next tokens' operands have arrived and before the ones
  // after them are asked for: whatever the wave then waits for in memory was asked a whole round of tokens ago.
  auto flush = [&](int t0, int nt) {
    for (int idx = lane; idx < TOK * COLS; idx += WAVE) {
      const int t = idx / COLS, jj = blockIdx.z * COLS + idx % COLS;
      if (t < nt && jj < V) a.out[(size_t)(first + t0 + t) * a.H * V + (size_t)h * V + jj] = so[t][idx % COLS];
    }
  };
  if (rows > 0) ask(0);
  for (int t0 = 0; t0 < rows; t0 += TOK) {
    const int nt = min(TOK, rows - t0);
    __syncthreads();   // everyone is done with the tokens before
    put();
    if (t0 > 0) flush(t0 - TOK, TOK);
    __syncthreads();
    if (t0 + TOK < rows) ask(t0 + TOK);
    // a token's operands are read from LDS while the token before it is worked on
    float kk[DPT], qq[DPT], dd[DPT], vj, beta_t, g_head;
    auto read = [&](int t, float (&k_)[DPT], float (&q_)[DPT], float (&d_)[DPT], float& v_, float& b_, float& g_) {
#pragma unroll
      for (int c = 0; c < DPT / 4; ++c) {
        const float4 k4 = *(const float4*)&sk[t][part][c * 4], q4 = *(const float4*)&sq[t][part][c * 4];
        k_[c * 4] = k4.x; k_[c * 4 + 1] = k4.y; k_[c * 4 + 2] = k4.z; k_[c * 4 + 3] = k4.w;
        q_[c * 4] = q4.x; q_[c * 4 + 1] = q4.y; q_[c * 4 + 2] = q4.z; q_[c * 4 + 3] = q4.w;
        if (channel_decay) {
          const float4 d4 = *(const float4*)&sd[t][part][c * 4];
          d_[c * 4] = d4.x; d_[c * 4 + 1] = d4.y; d_[c * 4 + 2] = d4.z; d_[c * 4 + 3] = d4.w;
        } else {
          d_[c * 4] = d_[c * 4 + 1] = d_[c * 4 + 2] = d_[c * 4 + 3] = 1.f;
        }
      }
      v_ = sv[t][col];
      b_ = RULE == RULE_DELTA ? sb[t] : 0.f;
      g_ = RULE != RULE_OUTER ? sg[t] : 1.f;
    };
    auto step = [&](int t, const float (&k_)[DPT], const float (&q_)[DPT], const float (&d_)[DPT], float v_, float b_, float g_) {
      float o0 = 0.f, o1 = 0.f;
      if (RULE == RULE_SSD) {
#pragma unroll
        for (int ii = 0; ii < DPT; ii += 2) {
          S[ii] = fmaf(channel_decay ? d_[ii] : g_, S[ii], k_[ii] * v_);
          S[ii + 1] = fmaf(channel_decay ? d_[ii + 1] : g_, S[ii + 1], k_[ii + 1] * v_);
          o0 = fmaf(S[ii], q_[ii], o0);
          o1 = fmaf(S[ii + 1], q_[ii + 1], o1);
        }
      } else if (RULE == RULE_DELTA) {
        float dot0 = 0.f, dot1 = 0.f;
#pragma unroll
        for (int ii = 0; ii < DPT; ii += 2) {
          S[ii] *= channel_decay ? d_[ii] : g_;
          S[ii + 1] *= channel_decay ? d_[ii + 1] : g_;
          dot0 = fmaf(S[ii], k_[ii], dot0);
          dot1 = fmaf(S[ii + 1], k_[ii + 1], dot1);
        }
        const float u = b_ * (v_ - fold(dot0 + dot1));
#pragma unroll
        for (int ii = 0; ii < DPT; ii += 2) {
          S[ii] = fmaf(k_[ii], u, S[ii]);
          S[ii + 1] = fmaf(k_[ii + 1], u, S[ii + 1]);
          o0 = fmaf(S[ii], q_[ii], o0);
          o1 = fmaf(S[ii + 1], q_[ii + 1], o1);
        }
      } else {
#pragma unroll
        for (int ii = 0; ii < DPT; ii += 2) {
          const float kv0 = k_[ii] * v_, kv1 = k_[ii + 1] * v_;
          o0 = fmaf(q_[ii], fmaf(bonus[ii], kv0, S[ii]), o0);
          o1 = fmaf(q_[ii + 1], fmaf(bonus[ii + 1], kv1, S[ii + 1]), o1);
          S[ii] = fmaf(d_[ii], S[ii], kv0);
          S[ii + 1] = fmaf(d_[ii + 1], S[ii + 1], kv1);
        }
      }
      const float o = fold(o0 + o1);
      if (part == 0) so[t][col] = o;
    };
    // two sets of registers take turns: while one token is worked on, the next one's operands arrive in the other
    float k2[DPT], q2[DPT], d2[DPT], v2, b2, g2;
    read(0, kk, qq, dd, vj, beta_t, g_head);
    for (int t = 0; t < nt; t += 2) {
      read(min(t + 1, TOK - 1), k2, q2, d2, v2, b2, g2);
      step(t, kk, qq, dd, vj, beta_t, g_head);
      if (t + 1 < nt) {
        read(min(t + 2, TOK - 1), kk, qq, dd, vj, beta_t, g_head);
        step(t + 1, k2, q2, d2, v2, b2, g2);
      }
    }
  }
  if (rows > 0) {
    __syncthreads();
    flush((rows - 1) / TOK * TOK, rows - (rows - 1) / TOK * TOK);
  }
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) {
    const int i = part * DPT + ii;
    if (i < D && j < V) st[(size_t)i * V + j] = S[ii];
  }
}

// Lanes per column by the key size: 8 channels a lane up to 128 channels, 16 beyond.
template <typename TIn, int RULE, bool CH>
void launch_recurrence_sized(const RecurrenceArgs& a, int n_req, hipStream_t stream) {
  if (a.D <= 32) recurrence_kernel<TIn, RULE, 8, 4, CH><<<dim3(n_req, a.H, ceil_div(a.V, 16)), 64, 0, stream>>>(a);
  else if (a.D <= 64) recurrence_kernel<TIn, RULE, 8, 8, CH><<<dim3(n_req, a.H, ceil_div(a.V, 8)), 64, 0, stream>>>(a);
  else if (a.D <= 128) recurrence_kernel<TIn, RULE, 8, 16, CH><<<dim3(n_req, a.H, ceil_div(a.V, 4)), 64, 0, stream>>>(a);
  else recurrence_kernel<TIn, RULE, 16, 16, CH><<<dim3(n_req, a.H, ceil_div(a.V, 4)), 64, 0, stream>>>(a);
}
template <typename TIn, int RULE>
int launch_recurrence(const RecurrenceArgs& a, int n_req, hipStream_t stream) {
  if (RULE == RULE_OUTER || a.per_channel) launch_recurrence_sized<TIn, RULE, true>(a, n_req, stream);
  else launch_recurrence_sized<TIn, RULE, false>(a, n_req, stream);
  return 0;
}

// ------------------------------------------------------------------------------------------------ a head's read-out, normed and gated
// y[n, h, :] = o[n, h, :] / sqrt(mean(o^2) + eps) * gain[(h V + j) % gain_len] * act(gate[n, h V + j])
template <typename T>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ gain,
                                                            int gain_len, const T* __restrict__ gate, long ld_gate,
                                                            T* __restrict__ y, int H, int V, float eps, int act) {
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* row = o + (size_t)n * H * V + (size_t)h * V;
  float ss = 0.f;
  for (int j = lane; j < V; j += WAVE) ss = fmaf(row[j], row[j], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)V + eps);
  for (int j = lane; j < V; j += WAVE) {
    const int c = h * V + j;
    const float g = activate_gate(to_float(gate[(size_t)n * ld_gate + c]), act);
    y[(size_t)n * H * V + c] = from_float<T>(row[j] * inv * gain[c % gain_len] * g);
  }
}

// ------------------------------------------------------------------------------------------------ shift by one token
// out[s, n, c] = h[n, c] + (prev[n, c] - h[n, c]) * mu[s, c]; prev is the request's previous token's h: the row
// before, or for a step's first row the request's state (zeros at a sequence's start).
template <typename T>
__global__ void token_shift_kernel(const T* __restrict__ h, const float* __restrict__ mu, int n_mix,
                                   float* __restrict__ state, long slot_stride, const int* __restrict__ row_req,
                                   const int* __restrict__ cu, const int* __restrict__ slot, T* __restrict__ out, int N, int W,
                                   int keep_row) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int r = row_req[n];
  const float cur = to_float(h[(size_t)n * W + c]);
  const float prev = n > cu[r] ? to_float(h[(size_t)(n - 1) * W + c]) : state[(size_t)slot[r] * slot_stride + c];
  if (keep_row) state[(size_t)slot[r] * slot_stride + c] = cur;   // (every request brings one row: it is the next step's previous row)
  for (int s = 0; s < n_mix; ++s)
    out[((size_t)s * N + n) * W + c] = from_float<T>(fmaf(prev - cur, mu[(size_t)s * W + c], cur));
}
template <typename T>
__global__ void token_shift_state_kernel(const T* __restrict__ h, float* __restrict__ state, long slot_stride,
                                         const int* __restrict__ cu, const int* __restrict__ slot, int W) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  state[(size_t)slot[r] * slot_stride + c] = to_float(h[(size_t)(cu[r + 1] - 1) * W + c]);
}

// out = tanh(in) (float32 in, the activation type out); and decay = exp(-exp(z + bias)) in place.
template <typename T>
__global__ void tanh_kernel(const float* __restrict__ in, T* __restrict__ out, long count) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) out[i] = from_float<T>(tanhf(in[i]));
}
__global__ void double_exp_decay_kernel(float* __restrict__ z, const float* __restrict__ bias, long count, int C) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) z[i] = expf(-expf(z[i] + bias[i % C]));
}
}  // namespace

#define BY_DTYPE(dtype, what, call_f32, call_bf16)         \
  do {                                                     \
    if ((dtype) == GIBBS_F32) { call_f32; }                \
    else if ((dtype) == GIBBS_BF16) { call_bf16; }         \
    else return gibbs_fail(what ": unknown dtype %d", (dtype)); \
  } while (0)

// The general entry point: an optional bias [C], act 0 none / 1 silu, `residual` (the input is added to the result), and the
// result as float32 (out_f32) or in the input's type, in rows of ld_out values.  `in` and `out` must not overlap.
GIBBS_EXPORT int gibbs_causal_conv(const void* in, long ld, int dtype, const float* taps, const float* bias, float* state, long slot_stride,
                                   const int* row_req, const int* cu, const int* slot, void* out, int out_f32, long ld_out, int n_rows,
                                   int n_req, int C, int K, int act, int residual, int update_state, int single_rows, hipStream_t stream) {
  // single_rows: every request brings exactly one row (a step of decoded tokens): the state moves on in the same kernel
  const int shift = update_state && single_rows && K > 1 && n_rows == n_req;
  GIBBS_REQUIRE(in && taps && state && out && n_rows > 0 && n_req > 0 && C > 0 && K >= 1 && ld >= C && ld_out >= C && slot_stride >= (long)(K - 1) * C,
                "causal_conv: bad operands rows=%d requests=%d C=%d K=%d", n_rows, n_req, C, K);
  const dim3 rows(n_rows, ceil_div(C, 256)), reqs(n_req, ceil_div(C, 256));
#define CONV_ARGS taps, bias, state, slot_stride, row_req, cu, slot
  // (steps of few rows are served faster by the kernel with a thread per channel: more, shorter workgroups; measured at 8 rows)
  const bool vec8 = dtype == GIBBS_BF16 && n_rows >= 64 && C % 8 == 0 && ld % 8 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                    ld_out % (out_f32 ? 4 : 8) == 0 && slot_stride % 4 == 0 && ((uintptr_t)state % 16) == 0 && ((uintptr_t)bias % 16) == 0 && K <= 16;
  if (vec8) {
    const dim3 grid(ceil_div(n_rows, CONV_ROWS), ceil_div(C, CONV_LANES * 8)), block(CONV_LANES, CONV_ROWS);
    const size_t lds = (size_t)CONV_LANES * (8 * K + 1) * sizeof(float);
    if (out_f32) causal_conv_vec8_kernel<float><<<grid, block, lds, stream>>>((const bf16*)in, ld, CONV_ARGS, (float*)out, ld_out, n_rows, C, K, shift, act, residual);
    else causal_conv_vec8_kernel<bf16><<<grid, block, lds, stream>>>((const bf16*)in, ld, CONV_ARGS, (bf16*)out, ld_out, n_rows, C, K, shift, act, residual);
  } else if (out_f32 || dtype == GIBBS_F32)
    BY_DTYPE(dtype, "causal_conv",
             (causal_conv_silu_kernel<float, float><<<rows, 256, 0, stream>>>((const float*)in, ld, CONV_ARGS, (float*)out, ld_out, C, K, shift, act, residual)),
             (causal_conv_silu_kernel<bf16, float><<<rows, 256, 0, stream>>>((const bf16*)in, ld, CONV_ARGS, (float*)out, ld_out, C, K, shift, act, residual)));
  else if (dtype == GIBBS_BF16)
    causal_conv_silu_kernel<bf16, bf16><<<rows, 256, 0, stream>>>((const bf16*)in, ld, CONV_ARGS, (bf16*)out, ld_out, C, K, shift, act, residual);
  else
    return gibbs_fail("causal_conv: unknown dtype %d", dtype);
#undef CONV_ARGS
  if (update_state && K > 1 && !shift)
    BY_DTYPE(dtype, "causal_conv",
             (causal_conv_state_kernel<float><<<reqs, 256, 0, stream>>>((const float*)in, ld, state, slot_stride, cu, slot, C, K)),
             (causal_conv_state_kernel<bf16><<<reqs, 256, 0, stream>>>((const bf16*)in, ld, state, slot_stride, cu, slot, C, K)));
  GIBBS_LAUNCH_STATUS("causal_conv");
}
GIBBS_EXPORT int gibbs_causal_conv_silu(const void* in, long ld, int dtype, const float* taps, float* state, long slot_stride,
                                        const int* row_req, const int* cu, const int* slot, float* out, int n_rows, int n_req,
                                        int C, int K, int update_state, int single_rows, hipStream_t stream) {
  return gibbs_causal_conv(in, ld, dtype, taps, nullptr, state, slot_stride, row_req, cu, slot, out, 1, C, n_rows, n_req, C, K, 1, 0,
                           update_state, single_rows, stream);
}

GIBBS_EXPORT int gibbs_delta_prep(float* q, float* k, long ldqk, const void* beta_raw, const void* a_head, long ld_raw, int dtype,
                                  const float* a_channel, const float* dt_bias, const float* a_log, float* beta, float* decay,
                                  int n_rows, int G, int H, int D, float q_scale, float unit_eps, hipStream_t stream) {
  GIBBS_REQUIRE(q && k && beta_raw && (a_head || a_channel) && dt_bias && a_log && beta && decay && n_rows > 0 && G > 0 && H > 0 && D > 0,
                "delta_prep: bad operands rows=%d kv heads=%d heads=%d D=%d", n_rows, G, H, D);
  DeltaPrepArgs a{q, k, ldqk, beta_raw, ld_raw, a_channel ? nullptr : a_head, a_channel, dt_bias, a_log, beta, decay, G, H, D, q_scale, unit_eps};
  const dim3 grid(n_rows, G + H);
  BY_DTYPE(dtype, "delta_prep", (delta_prep_kernel<float><<<grid, 64, 0, stream>>>(a)), (delta_prep_kernel<bf16><<<grid, 64, 0, stream>>>(a)));
  GIBBS_LAUNCH_STATUS("delta_prep");
}

namespace {
int check_recurrence(const char* what, int n_req, int H, int G, int D, int V, long slot_stride) {
  GIBBS_REQUIRE(n_req > 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && D <= 256 && V > 0,
                "%s: bad sizes requests=%d heads=%d kv heads=%d D=%d (up to 256) V=%d", what, n_req, H, G, D, V);
  GIBBS_REQUIRE(slot_stride >= (long)H * D * V, "%s: a slot of %ld floats cannot hold %d x %d x %d", what, slot_stride, H, D, V);
  return 0;
}
}  // namespace

// What the state-space rule reads, from the convolved rows xbc [N, ld_x] (float32: x [H*V] first) and the projected rows'
// dt entries (raw [N, ld_raw] in the activation type, H values from column 0 of `dt_raw`):
//   dt = softplus(dt_raw + dt_bias);  decay = exp(-exp(a_log) dt);  xdt = dt x      (all float32)
template <typename T>
__global__ void ssd_prep_kernel(const float* __restrict__ xbc, long ld_x, const T* __restrict__ dt_raw, long ld_raw,
                                const float* __restrict__ dt_bias, const float* __restrict__ a_log, float* __restrict__ decay,
                                float* __restrict__ log_decay, float* __restrict__ xdt, int H, int V) {
  const int n = blockIdx.x, h = blockIdx.y;
  const float dt = softplus_f(to_float(dt_raw[(size_t)n * ld_raw + h]) + dt_bias[h]);
  if (threadIdx.x == 0) {
    const float la = -expf(a_log[h]) * dt;
    decay[(size_t)n * H + h] = expf(la);
    if (log_decay) log_decay[(size_t)n * H + h] = la;
  }
  for (int j = threadIdx.x; j < V; j += blockDim.x) xdt[(size_t)n * H * V + (size_t)h * V + j] = dt * xbc[(size_t)n * ld_x + (size_t)h * V + j];
}
// (log_decay [N, H], optional: the decay's logarithm, -exp(a_log) dt, for the rule in chunks)
GIBBS_EXPORT int gibbs_ssd_prep(const float* xbc, long ld_x, const void* dt_raw, long ld_raw, int dtype, const float* dt_bias,
                                const float* a_log, float* decay, float* log_decay, float* xdt, int n_rows, int H, int V, hipStream_t stream) {
  GIBBS_REQUIRE(xbc && dt_raw && dt_bias && a_log && decay && xdt && n_rows > 0 && H > 0 && V > 0 && ld_x >= (long)H * V && ld_raw >= H,
                "ssd_prep: bad operands rows=%d heads=%d V=%d", n_rows, H, V);
  GIBBS_REQUIRE(H <= 65535, "ssd_prep: too many heads (%d)", H);
  const dim3 grid(n_rows, H);
  BY_DTYPE(dtype, "ssd_prep",
           (ssd_prep_kernel<float><<<grid, WAVE, 0, stream>>>(xbc, ld_x, (const float*)dt_raw, ld_raw, dt_bias, a_log, decay, log_decay, xdt, H, V)),
           (ssd_prep_kernel<bf16><<<grid, WAVE, 0, stream>>>(xbc, ld_x, (const bf16*)dt_raw, ld_raw, dt_bias, a_log, decay, log_decay, xdt, H, V)));
  GIBBS_LAUNCH_STATUS("ssd_prep");
}

// The decayed outer-product rule with one decay per head and the read-out after the write (see recurrence_kernel): the
// recurrence of a state-space mixer, M [D, V] with D the state size: k = B, q = C (G groups of D), v = dt x.  All float32.
GIBBS_EXPORT int gibbs_ssd_rule(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* decay, float* state,
                                long slot_stride, const int* cu, const int* slot, float* out, int n_req, int H, int G, int D, int V,
                                hipStream_t stream) {
  GIBBS_REQUIRE(q && k && v && decay && state && cu && slot && out && ldqk >= (long)G * D && ldv >= (long)H * V, "ssd_rule: null operand or short rows");
  if (check_recurrence("ssd_rule", n_req, H, G, D, V, slot_stride)) return 1;
  RecurrenceArgs a{q, k, v, ldqk, ldqk, ldv, decay, 0, nullptr, nullptr, state, slot_stride, cu, slot, out, H, G, D, V};
  launch_recurrence<float, RULE_SSD>(a, n_req, stream);
  GIBBS_LAUNCH_STATUS("ssd_rule");
}

// The gated delta rule over a ragged batch; q, k (unit vectors, q scaled), v, beta, decay float32.
GIBBS_EXPORT int gibbs_delta_rule(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* beta, const float* decay,
                                  int per_channel, float* state, long slot_stride, const int* cu, const int* slot, float* out,
                                  int n_req, int H, int G, int D, int V, hipStream_t stream) {
  GIBBS_REQUIRE(q && k && v && beta && decay && state && cu && slot && out && ldqk >= (long)G * D && ldv >= (long)H * V, "delta_rule: null operand or short rows");
  if (check_recurrence("delta_rule", n_req, H, G, D, V, slot_stride)) return 1;
  RecurrenceArgs a{q, k, v, ldqk, ldqk, ldv, decay, per_channel, beta, nullptr, state, slot_stride, cu, slot, out, H, G, D, V};
  launch_recurrence<float, RULE_DELTA>(a, n_req, stream);
  GIBBS_LAUNCH_STATUS("delta_rule");
}

// The decayed outer-product rule (see recurrence_kernel) over a ragged batch; r, k, v [N, H*D] in the activation type, w float32.
GIBBS_EXPORT int gibbs_decayed_outer_rule(const void* r, const void* k, const void* v, int dtype, const float* w, const float* bonus,
                                          float* state, long slot_stride, const int* cu, const int* slot, float* out, int n_req,
                                          int H, int D, hipStream_t stream) {
  GIBBS_REQUIRE(r && k && v && w && bonus && state && cu && slot && out, "decayed_outer_rule: null operand");
  if (check_recurrence("decayed_outer_rule", n_req, H, H, D, D, slot_stride)) return 1;
  RecurrenceArgs a{r, k, v, (long)H * D, (long)H * D, (long)H * D, w, 1, nullptr, bonus, state, slot_stride, cu, slot, out, H, H, D, D};
  BY_DTYPE(dtype, "decayed_outer_rule", (launch_recurrence<float, RULE_OUTER>(a, n_req, stream)),
           (launch_recurrence<bf16, RULE_OUTER>(a, n_req, stream)));
  GIBBS_LAUNCH_STATUS("decayed_outer_rule");
}

GIBBS_EXPORT int gibbs_head_norm_gate(const float* o, const float* gain, int gain_len, const void* gate, long ld_gate, void* y,
                                      int dtype, int n_rows, int H, int V, float eps, int act, hipStream_t stream) {
  GIBBS_REQUIRE(o && gain && gate && y && n_rows > 0 && H > 0 && V > 0 && gain_len > 0 && ld_gate >= (long)H * V && (act == 0 || act == 1),
                "head_norm_gate: bad operands rows=%d heads=%d V=%d", n_rows, H, V);
  const dim3 grid(n_rows, H);
  BY_DTYPE(dtype, "head_norm_gate",
           (head_norm_gate_kernel<float><<<grid, 64, 0, stream>>>(o, gain, gain_len, (const float*)gate, ld_gate, (float*)y, H, V, eps, act)),
           (head_norm_gate_kernel<bf16><<<grid, 64, 0, stream>>>(o, gain, gain_len, (const bf16*)gate, ld_gate, (bf16*)y, H, V, eps, act)));
  GIBBS_LAUNCH_STATUS("head_norm_gate");
}

GIBBS_EXPORT int gibbs_token_shift(const void* h, int dtype, const float* mu, int n_mix, float* state, long slot_stride,
                                   const int* row_req, const int* cu, const int* slot, void* out, int n_rows, int n_req, int W,
                                   int update_state, int single_rows, hipStream_t stream) {
  const int keep = update_state && single_rows && n_rows == n_req;
  GIBBS_REQUIRE(h && mu && state && out && n_rows > 0 && n_req > 0 && W > 0 && n_mix > 0 && slot_stride >= W,
                "token_shift: bad operands rows=%d requests=%d W=%d", n_rows, n_req, W);
  const dim3 rows(n_rows, ceil_div(W, 256)), reqs(n_req, ceil_div(W, 256));
  BY_DTYPE(dtype, "token_shift",
           (token_shift_kernel<float><<<rows, 256, 0, stream>>>((const float*)h, mu, n_mix, state, slot_stride, row_req, cu, slot, (float*)out, n_rows, W, keep)),
           (token_shift_kernel<bf16><<<rows, 256, 0, stream>>>((const bf16*)h, mu, n_mix, state, slot_stride, row_req, cu, slot, (bf16*)out, n_rows, W, keep)));
  if (update_state && !keep)
    BY_DTYPE(dtype, "token_shift",
             (token_shift_state_kernel<float><<<reqs, 256, 0, stream>>>((const float*)h, state, slot_stride, cu, slot, W)),
             (token_shift_state_kernel<bf16><<<reqs, 256, 0, stream>>>((const bf16*)h, state, slot_stride, cu, slot, W)));
  GIBBS_LAUNCH_STATUS("token_shift");
}

GIBBS_EXPORT int gibbs_tanh_rows(const float* in, void* out, int dtype, long count, hipStream_t stream) {
  GIBBS_REQUIRE(in && out && count > 0, "tanh: bad operands");
  BY_DTYPE(dtype, "tanh", (tanh_kernel<float><<<ceil_div(count, 256), 256, 0, stream>>>(in, (float*)out, count)),
           (tanh_kernel<bf16><<<ceil_div(count, 256), 256, 0, stream>>>(in, (bf16*)out, count)));
  GIBBS_LAUNCH_STATUS("tanh");
}

GIBBS_EXPORT int gibbs_double_exp_decay(float* z, const float* bias, long count, int C, hipStream_t stream) {
  GIBBS_REQUIRE(z && bias && count > 0 && C > 0, "double_exp_decay: bad operands");
  double_exp_decay_kernel<<<ceil_div(count, 256), 256, 0, stream>>>(z, bias, count, C);
  GIBBS_LAUNCH_STATUS("double_exp_decay");
}
