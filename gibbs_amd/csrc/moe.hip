// Mixture of experts: a router picks `top` of E small gated feed-forwards for every row, and the row's result is
// the weighted sum of theirs; a shared expert may run for every row beside them, times a sigmoid gate of its own.
//
//   route      z = W_r h + b in float32 (h as the step holds it); the `top` largest logits (the lower index among
//              equals); weights = softmax over the chosen logits alone; gate = sigmoid(w_sg . h) for the shared expert
//              (mode 1: scores s = softmax(z) over all router outputs; the `top` largest of s + correction; weights = the
//              chosen scores s divided by their sum + 1e-20.  Router outputs from `E_real` on are identity experts: they
//              have no matrices, their result is the row itself, and their pairs take no place in the tiles)
//   group      the step's (row, choice) pairs sorted by expert into tiles of `bm` pairs that belong to one expert
//              each (every expert's stretch is padded to whole tiles); nothing goes back to the host, so a step
//              with experts can be captured in a graph: the products below run over the worst-case number of tiles
//              and a tile without an expert returns at once
//   gate_up    act[m] = activation(W_gate,e h[row(m)]) * (W_up,e h[row(m)]) for every sorted pair m (rows gathered)
//   down       y[m] = W_down,e act[m]
//   combine    out[row] = sum_c weight[row][c] y[place(row, c)] (ascending c) + gate[row] shared[row], float32 sums
//
// A pair's result depends on nothing but its own row and expert (no sum runs over pairs), so where a pair lands
// among its expert's pairs, which the atomic counters of `group` decide, changes no value: a row's result is the
// same whatever else is in the batch.  Products: plain FMA in ascending k for float32 and for bfloat16 operands
// that are not 16-byte aligned; on the matrix cores for aligned bfloat16, float32 accumulators, the activation in
// float32: tiles of 16 pairs for steps of few pairs (the experts' matrices are streamed once, a workgroup's four
// waves split k, operands straight from memory: rows of h and of every W are contiguous along k), tiles of 128
// pairs beyond (128 pairs x 128 or 256 rows of W through LDS in tiles of 32 along k, double-buffered).
#include "common.h"
#include "activation.h"
#include <algorithm>

namespace {
constexpr int MOE_MAX_EXPERTS = 1024;

// ------------------------------------------------------------------------------------------------- route
// 4 neighbouring values of a row as float32 (16-byte or 8-byte loads)
__device__ __forceinline__ float4 load4f(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 load4f(const bf16* p) {
  const uint2 raw = *(const uint2*)p;
  return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                     __uint_as_float(raw.y & 0xffff0000u));
}
__device__ __forceinline__ void store4f(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void store4f(bf16* p, float4 v) {
  union { bf16 h[4]; uint2 u; } o;
  o.h[0] = (bf16)v.x; o.h[1] = (bf16)v.y; o.h[2] = (bf16)v.z; o.h[3] = (bf16)v.w;
  *(uint2*)p = o.u;
}
// One wave's inner products of a row with NV float32 vectors (the row is loaded once); `vec`: the width is a multiple of 4
// and all are aligned, so a lane takes 4 neighbouring values at a time.  Every sum is one chain of additions in ascending
// k per lane, so its value depends on the width alone, not on NV or on how many steps are asked for together.
template <typename T, int NV>
__device__ __forceinline__ void wave_dots(const T* __restrict__ row, const float* const (&w)[NV], float (&out)[NV], int W, int lane, bool vec) {
  float s[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) s[v] = 0.f;
  if (vec) {
    int k = lane * 4;
    // (eight steps at a time, then four: their loads are asked for together)
    for (; k + 7 * WAVE * 4 < W; k += 8 * WAVE * 4) {
      float4 a[8], b[NV][8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        a[u] = load4f(row + k + u * WAVE * 4);
#pragma unroll
        for (int v = 0; v < NV; ++v) b[v][u] = *(const float4*)(w[v] + k + u * WAVE * 4);
      }
#pragma unroll
      for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int u = 0; u < 8; ++u) { s[v] = fmaf(a[u].x, b[v][u].x, s[v]); s[v] = fmaf(a[u].y, b[v][u].y, s[v]); s[v] = fmaf(a[u].z, b[v][u].z, s[v]); s[v] = fmaf(a[u].w, b[v][u].w, s[v]); }
    }
    for (; k + 3 * WAVE * 4 < W; k += 4 * WAVE * 4) {
      float4 a[4], b[NV][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        a[u] = load4f(row + k + u * WAVE * 4);
#pragma unroll
        for (int v = 0; v < NV; ++v) b[v][u] = *(const float4*)(w[v] + k + u * WAVE * 4);
      }
#pragma unroll
      for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int u = 0; u < 4; ++u) { s[v] = fmaf(a[u].x, b[v][u].x, s[v]); s[v] = fmaf(a[u].y, b[v][u].y, s[v]); s[v] = fmaf(a[u].z, b[v][u].z, s[v]); s[v] = fmaf(a[u].w, b[v][u].w, s[v]); }
    }
    for (; k < W; k += WAVE * 4) {
      const float4 a = load4f(row + k);
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const float4 c = *(const float4*)(w[v] + k);
        s[v] = fmaf(a.x, c.x, s[v]); s[v] = fmaf(a.y, c.y, s[v]); s[v] = fmaf(a.z, c.z, s[v]); s[v] = fmaf(a.w, c.w, s[v]);
      }
    }
  } else {
    for (int k = lane; k < W; k += WAVE) {
      const float a = to_float(row[k]);
#pragma unroll
      for (int v = 0; v < NV; ++v) s[v] = fmaf(a, w[v][k], s[v]);
    }
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) out[v] = wave_sum(s[v]);
}
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ row, const float* __restrict__ w, int W, int lane, bool vec) {
  const float* const ws[1] = {w};
  float out[1];
  wave_dots<T, 1>(row, ws, out, W, lane, vec);
  return out[0];
}

template <typename T>
__global__ __launch_bounds__(1024) void moe_route_kernel(const T* __restrict__ h, long ldh, const float* __restrict__ router,
                                                        const float* __restrict__ router_bias, const float* __restrict__ shared_gate,
                                                        int* __restrict__ chosen, float* __restrict__ weight, float* __restrict__ sgate,
                                                        int W, int E, int top, int mode) {
  extern __shared__ float z[];   // [E] (mode 1: and the scores behind them, [E])
  const int n = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, n_waves = blockDim.x / WAVE;
  const T* row = h + (size_t)n * ldh;
  const bool vec = W % 4 == 0 && ldh % 4 == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)router % 16) == 0 && ((uintptr_t)shared_gate % 16) == 0;
  // the last wave also has the shared expert's gate: with its last expert's logit in one pass over the row
  bool gate_left = shared_gate && wave == n_waves - 1;
  for (int e = wave; e < E; e += n_waves) {
    float s;
    if (gate_left && e + n_waves >= E) {
      const float* const ws[2] = {router + (size_t)e * W, shared_gate};
      float both[2];
      wave_dots<T, 2>(row, ws, both, W, lane, vec);
      s = both[0];
      if (lane == 0) sgate[n] = 1.0f / (1.0f + expf(-both[1]));
      gate_left = false;
    } else {
      s = wave_dot(row, router + (size_t)e * W, W, lane, vec);
    }
    if (lane == 0) z[e] = s + ((router_bias && mode == 0) ? router_bias[e] : 0.f);
  }
  if (gate_left) {
    const float s = wave_dot(row, shared_gate, W, lane, vec);
    if (lane == 0) sgate[n] = 1.0f / (1.0f + expf(-s));
  }
  __syncthreads();
  if (wave != 0) return;
  // the `top` largest, in descending order, the lower index among equal logits (one wave: a lane scans its share of
  // the experts, the lanes' bests are folded by exchanges); a logit that was taken becomes NaN; then the softmax
  // over the chosen logits alone
  int* mine = chosen + (size_t)n * top;
  float* wts = weight + (size_t)n * top;
  float* score = z + E;
  if (mode == 1) {
    // scores over all outputs; what is compared is the score plus the output's correction
    float zmax = -INFINITY;
    for (int e = lane; e < E; e += WAVE) zmax = fmaxf(zmax, z[e]);
    zmax = wave_max(zmax);
    float total = 0.f;
    for (int e = lane; e < E; e += WAVE) total += expf(z[e] - zmax);
    total = wave_sum(total);
    for (int e = lane; e < E; e += WAVE) {
      const float sc = expf(z[e] - zmax) / total;
      score[e] = sc;
      z[e] = sc + (router_bias ? router_bias[e] : 0.f);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_wave_barrier();
  }
  float best = 0.f, sum = 0.f;
  for (int c = 0; c < top; ++c) {
    float pv = -INFINITY;
    int pick = 0x7fffffff;
    for (int e = lane; e < E; e += WAVE) {
      const float v = z[e];
      if (v == v && (v > pv || (v == pv && e < pick) || pick == 0x7fffffff)) { pv = v; pick = e; }
    }
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(pv, o, WAVE);
      const int op = __shfl_xor(pick, o, WAVE);
      if (op != 0x7fffffff && (pick == 0x7fffffff || ov > pv || (ov == pv && op < pick))) { pv = ov; pick = op; }
    }
    if (pick == 0x7fffffff) {   // (fewer usable logits than choices: the first expert not taken yet, with no weight)
      for (int e = 0; e < E && pick == 0x7fffffff; ++e) {
        bool taken = false;
        for (int d = 0; d < c; ++d) taken |= mine[d] == e;
        if (!taken) pick = e;
      }
      pv = -INFINITY;
    }
    if (c == 0) best = pv;
    const float w = mode == 1 ? score[pick] : (pv == -INFINITY ? 0.f : expf(pv - best));
    sum += w;
    if (lane == 0) {
      mine[c] = pick;
      wts[c] = w;
      z[pick] = __builtin_nanf("");
    }
    __builtin_amdgcn_s_waitcnt(0);   // (the wave's own LDS write above is read by its next scan)
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) {
    if (mode == 1)
      for (int c = 0; c < top; ++c) wts[c] = wts[c] / (sum + 1e-20f);
    else
      for (int c = 0; c < top; ++c) wts[c] = sum > 0.f ? wts[c] / sum : 0.f;
  }
}

// ------------------------------------------------------------------------------------------------- group
// One workgroup: counts per expert, every expert's stretch rounded up to whole tiles, then each pair takes the next
// free place of its expert's stretch.  sorted_pair [cap]: the pair at each place (-1: padding); pair_pos [n_pairs]:
// each pair's place; tile_expert [cap / bm]: the expert of each tile (-1: beyond the last stretch).
// (a pair whose expert is E or beyond, an identity expert, gets the place -1)
__global__ __launch_bounds__(1024) void moe_group_kernel(const int* __restrict__ chosen, int n_pairs, int E, int bm,
                                                         int* __restrict__ sorted_pair, int* __restrict__ pair_pos,
                                                         int* __restrict__ tile_expert, int cap) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int start[MOE_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  for (int m = threadIdx.x; m < cap; m += blockDim.x) sorted_pair[m] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x)
    if (chosen[i] < E) atomicAdd(&count[chosen[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      at += (count[e] + bm - 1) / bm * bm;
    }
    start[E] = at;
  }
  __syncthreads();
  for (int t = threadIdx.x; t < cap / bm; t += blockDim.x) {
    const int m = t * bm;
    int e = -1;
    if (m < start[E]) {   // the expert whose stretch holds place m
      int lo = 0, hi = E - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) / 2;
        if (start[mid] <= m) lo = mid; else hi = mid - 1;
      }
      e = lo;
    }
    tile_expert[t] = e;
  }
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    const int e = chosen[i];
    if (e >= E) { pair_pos[i] = -1; continue; }
    const int m = start[e] + atomicAdd(&count[e], 1);
    sorted_pair[m] = i;
    pair_pos[i] = m;
  }
}

// ------------------------------------------------------------------------------------------------- products, plain
// Tile of BM places x 64 features; thread (feature tx, row lane ty of 4) keeps BM / 4 rows of its feature; every sum
// in ascending k.  GLU: two matrices and act(gate) * up; else one matrix.  X rows: gathered by pair (pair / top) when
// `top` > 0, else the places themselves.
template <typename T, int BM, bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_plain_kernel(const T* __restrict__ X, long ldx, int top, const int* __restrict__ sorted_pair,
                                                             const int* __restrict__ tile_expert, const T* __restrict__ Wa,
                                                             const T* __restrict__ Wb, long expert_stride, T* __restrict__ Y, long ldy,
                                                             int O, int I, int act) {
  constexpr int TK = 16, RPT = BM / 4;
  __shared__ float sx[TK][BM + 1];
  __shared__ float sa[TK][64 + 1];
  __shared__ float sb[GLU ? TK : 1][64 + 1];
  __shared__ int src[BM];
  const int tile = blockIdx.y, e = tile_expert[tile];
  if (e < 0) return;
  const int col0 = blockIdx.x * 64, tx = threadIdx.x % 64, ty = threadIdx.x / 64;
  if (threadIdx.x < BM) {
    const int pair = sorted_pair[tile * BM + threadIdx.x];
    src[threadIdx.x] = pair < 0 ? -1 : (top > 0 ? pair / top : tile * BM + threadIdx.x);
  }
  __syncthreads();
  const T* wa = Wa + (size_t)e * expert_stride;
  const T* wb = GLU ? Wb + (size_t)e * expert_stride : nullptr;
  float acc_a[RPT] = {}, acc_b[RPT] = {};
  for (int k0 = 0; k0 < I; k0 += TK) {
    for (int i = threadIdx.x; i < TK * BM; i += 256) {
      const int r = i / TK, k = i % TK;
      sx[k][r] = (src[r] >= 0 && k0 + k < I) ? to_float(X[(size_t)src[r] * ldx + k0 + k]) : 0.f;
    }
    for (int i = threadIdx.x; i < TK * 64; i += 256) {
      const int c = i / TK, k = i % TK;
      const bool in = col0 + c < O && k0 + k < I;
      sa[k][c] = in ? to_float(wa[(size_t)(col0 + c) * I + k0 + k]) : 0.f;
      if (GLU) sb[k][c] = in ? to_float(wb[(size_t)(col0 + c) * I + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      const float a = sa[k][tx], b = GLU ? sb[k][tx] : 0.f;
#pragma unroll
      for (int r = 0; r < RPT; ++r) {
        const float x = sx[k][ty + 4 * r];
        acc_a[r] = fmaf(x, a, acc_a[r]);
        if (GLU) acc_b[r] = fmaf(x, b, acc_b[r]);
      }
    }
    __syncthreads();
  }
  if (col0 + tx >= O) return;
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int row = ty + 4 * r;
    if (src[row] < 0) continue;
    const float v = GLU ? activate(acc_a[r], act) * acc_b[r] : acc_a[r];
    Y[(size_t)(tile * BM + row) * ldy + col0 + tx] = from_float<T>(v);
  }
}

// ------------------------------------------------------------------------------------------------- products, matrix cores
// bfloat16, inner size a multiple of 8, rows 16-byte aligned.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

// Few pairs: a tile is 16 places, a workgroup takes 32 features of it (of both matrices, GLU) and its four waves a
// quarter of k each, so that the experts' matrices, which are read once, are spread over many workgroups; the waves'
// sums meet in LDS and the first wave adds them in wave order.  W is the first operand of the 16 x 16 x 32 product (the
// tile is Y^T = W X^T): lane l holds 8 values along k of feature or place l % 16, and its four results are four
// neighbouring features of place l % 16.  Operands come straight from memory.
template <bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_few_kernel(const bf16* __restrict__ X, long ldx, int top, const int* __restrict__ sorted_pair,
                                                           const int* __restrict__ tile_expert, const bf16* __restrict__ Wa,
                                                           const bf16* __restrict__ Wb, long expert_stride, bf16* __restrict__ Y, long ldy,
                                                           int O, int I, int act) {
  constexpr int NF = 2, NA = GLU ? 2 * NF : NF;    // feature tiles of 16 a workgroup; accumulators a wave
  __shared__ float part[4][NA][WAVE][4];
  const int tile = blockIdx.y, e = tile_expert[tile];
  if (e < 0) return;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, lr = lane % 16, lg = lane / 16;
  const int place = tile * 16 + lr;
  const int col0 = blockIdx.x * (16 * NF);
  const int pair = sorted_pair[place];
  const long src = pair < 0 ? -1 : (top > 0 ? pair / top : place);
  const bf16* xr = X + (size_t)(src < 0 ? 0 : src) * ldx;
  const bf16* wa = Wa + (size_t)e * expert_stride;
  const bf16* wb = GLU ? Wb + (size_t)e * expert_stride : nullptr;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  floatx4 acc[NA];
#pragma unroll
  for (int t = 0; t < NA; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  // wave w takes the stretches of 64 along k whose number is w modulo 4, in ascending order.  A lane group holds 16
  // neighbouring values of a stretch as the operands of two products (the order along k inside a product is free as long as
  // both operands agree), so that the wave asks for whole lines of 128 bytes of every row; two stretches at a time
#pragma unroll 2
  for (int k0 = wave * 64; k0 < I; k0 += 256) {
    bf16x8 x8[2], a8[2][NF], b8[2][NF];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int k = k0 + lg * 16 + u * 8;
      x8[u] = (src >= 0 && k < I) ? *(const bf16x8*)(xr + k) : zero8;
#pragma unroll
      for (int t = 0; t < NF; ++t) {
        const int col = col0 + t * 16 + lr;
        const bool in = col < O && k < I;
        a8[u][t] = in ? *(const bf16x8*)(wa + (size_t)col * I + k) : zero8;
        if (GLU) b8[u][t] = in ? *(const bf16x8*)(wb + (size_t)col * I + k) : zero8;
      }
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < NF; ++t) {
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a8[u][t], x8[u], acc[t], 0, 0, 0);
        if (GLU) acc[NF + t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b8[u][t], x8[u], acc[NF + t], 0, 0, 0);
      }
  }
#pragma unroll
  for (int t = 0; t < NA; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][t][lane][i] = acc[t][i];
  __syncthreads();
  if (wave != 0 || src < 0) return;
#pragma unroll
  for (int t = 0; t < NF; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = col0 + t * 16 + lg * 4 + i;
      if (col >= O) continue;
      float a = 0.f, b = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        a += part[w][t][lane][i];
        if (GLU) b += part[w][NF + t][lane][i];
      }
      Y[(size_t)place * ldy + col] = (bf16)(GLU ? activate(a, act) * b : a);
    }
}

// Many pairs: a tile is 128 places, a workgroup of NW waves computes 128 places x BN rows of W (GLU: BN / 2 features of both
// matrices), each wave 64 x 64 as 2 x 2 products of 32 x 32 x 16; tiles of BK along k go through LDS (rows padded by 16
// bytes against bank conflicts), double-buffered, and a further tile waits in registers, so that a tile's loads have
// two tiles' work to arrive.  The rows of X are gathered by the tile's pairs as they are loaded.
constexpr int TBM = 128;
template <int BK, int BN>
struct MoeTile {
  bf16 a[TBM][BK + 8];
  bf16 w[BN][BK + 8];
};
template <bool GLU, int BK, int BN, int NW>
__global__ __launch_bounds__(NW * WAVE) void moe_gemm_tiled_kernel(const bf16* __restrict__ X, long ldx, int top, const int* __restrict__ sorted_pair,
                                                             const int* __restrict__ tile_expert, const bf16* __restrict__ Wa,
                                                             const bf16* __restrict__ Wb, long expert_stride, bf16* __restrict__ Y, long ldy,
                                                             int O, int I, int act) {
  using Tile = MoeTile<BK, BN>;
  constexpr int KC = BK / 8;                        // chunks of 16 bytes in a row of a tile
  constexpr int THREADS = NW * WAVE, WN = NW / 2;   // waves: 2 along the places, WN along the rows of W
  constexpr int CA = TBM * KC / THREADS, CW = BN * KC / THREADS;   // chunks a thread moves per operand and tile of k
  constexpr int NT = BN / WN / 32;                  // column blocks of 32 a wave
  static_assert(CA >= 1 && CW >= 1 && NT >= (GLU ? 2 : 1) && NT % (GLU ? 2 : 1) == 0, "tile sizes");
  extern __shared__ __attribute__((aligned(16))) char moe_lds[];
  Tile* tiles = (Tile*)moe_lds;                     // [2]
  int* srcs = (int*)(moe_lds + 2 * sizeof(Tile));   // [TBM]
  const int tile = blockIdx.y, e = tile_expert[tile];
  if (e < 0) return;
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
  constexpr int COLS = GLU ? BN / 2 : BN;           // features of the result that a workgroup takes
  const int col0 = blockIdx.x * COLS;
  if (tid < TBM) {
    const int pair = sorted_pair[tile * TBM + tid];
    srcs[tid] = pair < 0 ? -1 : (top > 0 ? pair / top : tile * TBM + tid);
  }
  __syncthreads();
  const bf16* wa = Wa + (size_t)e * expert_stride;
  const bf16* wb = GLU ? Wb + (size_t)e * expert_stride : nullptr;
  const int wr = (wave / WN) * 64;
  // a thread's rows stay the same from tile to tile
  const bf16* pa[CA];
  const bf16* pw[CW];
#pragma unroll
  for (int i = 0; i < CA; ++i) {
    const int r = (tid + i * THREADS) / KC;
    pa[i] = srcs[r] >= 0 ? X + (size_t)srcs[r] * ldx : nullptr;
  }
#pragma unroll
  for (int i = 0; i < CW; ++i) {
    const int r = (tid + i * THREADS) / KC;
    const int col = col0 + (GLU ? r % COLS : r);
    pw[i] = col < O ? ((GLU && r >= COLS) ? wb : wa) + (size_t)col * I : nullptr;
  }
  // two register sets take turns: a tile's loads are asked for two tiles ahead of its use
  uint4 ra[2][CA], rw[2][CW];
  auto load_global = [&](int k0, uint4* a, uint4* w) {
    const int gk = k0 + (tid % KC) * 8;
#pragma unroll
    for (int i = 0; i < CA; ++i) a[i] = (pa[i] && gk < I) ? *(const uint4*)(pa[i] + gk) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < CW; ++i) w[i] = (pw[i] && gk < I) ? *(const uint4*)(pw[i] + gk) : make_uint4(0, 0, 0, 0);
  };
  auto store_lds = [&](Tile& t, const uint4* a, const uint4* w) {
    const int kc = (tid % KC) * 8;
#pragma unroll
    for (int i = 0; i < CA; ++i) *(uint4*)&t.a[(tid + i * THREADS) / KC][kc] = a[i];
#pragma unroll
    for (int i = 0; i < CW; ++i) *(uint4*)&t.w[(tid + i * THREADS) / KC][kc] = w[i];
  };
  floatx16 acc[2][NT];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[m][n][i] = 0.f;
  // the wave's column blocks of 32 in the W tile: neighbours (one matrix), or the same features of gate (the first half of
  // its blocks) and up (the second half)
  int wc[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n)
    wc[n] = GLU ? (n / (NT / 2)) * COLS + (wave % WN) * (COLS / WN) + (n % (NT / 2)) * 32 : (wave % WN) * (BN / WN) + n * 32;
  const int n_tiles = (I + BK - 1) / BK;
  auto compute = [&](const Tile& cur) {
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 fa[2], fw[NT];
      const int k = kk * 16 + (lane / 32) * 8;
#pragma unroll
      for (int m = 0; m < 2; ++m) fa[m] = *(const bf16x8*)&cur.a[wr + m * 32 + lane % 32][k];
#pragma unroll
      for (int n = 0; n < NT; ++n) fw[n] = *(const bf16x8*)&cur.w[wc[n] + lane % 32][k];
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[m], fw[n], acc[m][n], 0, 0, 0);
    }
  };
  load_global(0, ra[0], rw[0]);
  store_lds(tiles[0], ra[0], rw[0]);
  load_global(BK, ra[0], rw[0]);
  __syncthreads();
  // tile t is in LDS buffer t % 2; while it is worked on, tile t + 1 waits in one register set and tile t + 2 is on its
  // way into the other; a buffer is written again only after the barrier behind its last reader
  // (an odd number of tiles is worked on as the next even one: loads beyond the inner size give zeros)
  for (int t = 0; t < n_tiles; t += 2) {
    load_global((t + 2) * BK, ra[1], rw[1]);
    compute(tiles[0]);
    store_lds(tiles[1], ra[0], rw[0]);
    __syncthreads();
    load_global((t + 3) * BK, ra[0], rw[0]);
    compute(tiles[1]);
    store_lds(tiles[0], ra[1], rw[1]);
    __syncthreads();
  }
  // a lane holds column lane % 32 of a block and its rows (i / 4) * 8 + (lane / 32) * 4 + i % 4
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = wr + m * 32 + (i / 4) * 8 + (lane / 32) * 4 + i % 4;
      if (srcs[row] < 0) continue;
      bf16* y = Y + (size_t)(tile * TBM + row) * ldy;
      if (GLU) {
#pragma unroll
        for (int n = 0; n < NT / 2; ++n) {
          const int col = col0 + wc[n] + lane % 32;
          if (col < O) y[col] = (bf16)(activate(acc[m][n][i], act) * acc[m][NT / 2 + n][i]);
        }
      } else {
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          const int col = col0 + wc[n] + lane % 32;
          if (col < O) y[col] = (bf16)acc[m][n][i];
        }
      }
    }
}

template <bool GLU, int BK, int BN, int NW>
int launch_tiled_as(const bf16* X, long ldx, int top, const int* sorted_pair, const int* tile_expert, int tiles, const bf16* wa, const bf16* wb,
                    long stride, bf16* Y, long ldy, int O, int I, int act, hipStream_t stream) {
  constexpr int LDS = 2 * (int)sizeof(MoeTile<BK, BN>) + TBM * (int)sizeof(int);
  static bool prepared = false;    // (one flag per instantiation)
  if (!prepared) {
    hipError_t e = hipFuncSetAttribute((const void*)moe_gemm_tiled_kernel<GLU, BK, BN, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (e != hipSuccess) return gibbs_fail("moe_gemm: %s", hipGetErrorString(e));
    prepared = true;
  }
  moe_gemm_tiled_kernel<GLU, BK, BN, NW><<<dim3(ceil_div(O, GLU ? BN / 2 : BN), tiles), NW * WAVE, LDS, stream>>>(X, ldx, top, sorted_pair, tile_expert, wa, wb,
                                                                                                        stride, Y, ldy, O, I, act);
  return 0;
}
template <bool GLU>
int launch_tiled(const bf16* X, long ldx, int top, const int* sorted_pair, const int* tile_expert, int tiles, const bf16* wa, const bf16* wb,
                 long stride, bf16* Y, long ldy, int O, int I, int act, hipStream_t stream) {
  // wide results with a long inner size: 256 rows of W a workgroup and 8 waves (the tile of X is read by half as many
  // workgroups); otherwise 128 rows and 4 waves, which leaves more workgroups to spread
  if (I > 1024 && O >= 512)
    return launch_tiled_as<GLU, 32, 256, 8>(X, ldx, top, sorted_pair, tile_expert, tiles, wa, wb, stride, Y, ldy, O, I, act, stream);
  return launch_tiled_as<GLU, 32, 128, 4>(X, ldx, top, sorted_pair, tile_expert, tiles, wa, wb, stride, Y, ldy, O, I, act, stream);
}

// ------------------------------------------------------------------------------------------------- combine
// (`self` [n, W], not null: a choice whose place is -1 is an identity expert, its result the row of `self`)
template <typename T, bool VEC>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ pair_pos, const float* __restrict__ weight,
                                   const T* __restrict__ shared, const float* __restrict__ sgate, const T* __restrict__ self,
                                   T* __restrict__ out, int top, int W) {
  constexpr int MOST = 8;      // choices whose places and weights a thread keeps in registers
  const int n = blockIdx.x;
  const float g = shared ? (sgate ? sgate[n] : 1.0f) : 0.f;
  const T* at[MOST];
  float w[MOST];
  auto row_of = [&](int s) -> const T* {
    const int place = pair_pos[(size_t)n * top + s];
    return (self && place < 0) ? self + (size_t)n * W : y + (size_t)place * W;
  };
#pragma unroll
  for (int s = 0; s < MOST; ++s) {
    at[s] = s < top ? row_of(s) : y;
    w[s] = s < top ? weight[(size_t)n * top + s] : 0.f;
  }
  if (VEC) {
    for (int c = threadIdx.x * 4; c < W; c += blockDim.x * 4) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int s = 0; s < MOST; ++s)
        if (s < top) {
          const float4 r = load4f(at[s] + c);
          v.x = fmaf(w[s], r.x, v.x); v.y = fmaf(w[s], r.y, v.y); v.z = fmaf(w[s], r.z, v.z); v.w = fmaf(w[s], r.w, v.w);
        }
      for (int s = MOST; s < top; ++s) {
        const float ws = weight[(size_t)n * top + s];
        const float4 r = load4f(row_of(s) + c);
        v.x = fmaf(ws, r.x, v.x); v.y = fmaf(ws, r.y, v.y); v.z = fmaf(ws, r.z, v.z); v.w = fmaf(ws, r.w, v.w);
      }
      if (shared) {
        const float4 r = load4f(shared + (size_t)n * W + c);
        v.x = fmaf(g, r.x, v.x); v.y = fmaf(g, r.y, v.y); v.z = fmaf(g, r.z, v.z); v.w = fmaf(g, r.w, v.w);
      }
      store4f(out + (size_t)n * W + c, v);
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < top; ++s) v = fmaf(weight[(size_t)n * top + s], to_float(row_of(s)[c]), v);
    if (shared) v = fmaf(g, to_float(shared[(size_t)n * W + c]), v);
    out[(size_t)n * W + c] = from_float<T>(v);
  }
}
}  // namespace

// Places that the sorted pairs of a step can take at most: every expert's stretch rounded up to whole tiles.
GIBBS_EXPORT long gibbs_moe_capacity(int n_pairs, int E, int bm) {
  return ((long)n_pairs + (long)E * (bm - 1) + bm - 1) / bm * bm;
}
// Tiles of pairs: 16 while the matrices are streamed for few pairs each (at most 64 an expert on average), 128 beyond.
GIBBS_EXPORT int gibbs_moe_tile(int n_pairs, int E) { return (long)n_pairs <= 64L * E ? 16 : 128; }

// mode 0: the largest logits (+ bias), weights by the softmax over the chosen; mode 1: scores by the softmax over all E
// outputs, the largest of score + router_bias (a correction that only the choice sees), weights the chosen scores over their sum.
GIBBS_EXPORT int gibbs_moe_route_mode(const void* h, long ldh, int dtype, const float* router, const float* router_bias,
                                      const float* shared_gate, int* chosen, float* weight, float* sgate, int n, int W, int E, int top,
                                      int mode, hipStream_t stream) {
  GIBBS_REQUIRE(mode == 0 || mode == 1, "moe_route: mode %d", mode);
  GIBBS_REQUIRE(h && router && chosen && weight && n > 0 && W > 0 && ldh >= W, "moe_route: bad operands n=%d width=%d", n, W);
  GIBBS_REQUIRE(E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= E, "moe_route: %d of %d experts (at most %d)", top, E, MOE_MAX_EXPERTS);
  GIBBS_REQUIRE(!shared_gate || sgate, "moe_route: a shared expert's gate needs its output");
  const size_t lds = (size_t)E * sizeof(float) * (mode == 1 ? 2 : 1);
  // few rows: a wave per expert (and one for the shared expert's gate) up to 16 waves; many rows fill the chip with 4
  const int threads = n >= 512 ? 256 : WAVE * std::min(16, std::max(4, E + 1));
  if (dtype == GIBBS_F32)
    moe_route_kernel<float><<<n, threads, lds, stream>>>((const float*)h, ldh, router, router_bias, shared_gate, chosen, weight, sgate, W, E, top, mode);
  else if (dtype == GIBBS_BF16)
    moe_route_kernel<bf16><<<n, threads, lds, stream>>>((const bf16*)h, ldh, router, router_bias, shared_gate, chosen, weight, sgate, W, E, top, mode);
  else
    return gibbs_fail("moe_route: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("moe_route");
}
GIBBS_EXPORT int gibbs_moe_route(const void* h, long ldh, int dtype, const float* router, const float* router_bias,
                                 const float* shared_gate, int* chosen, float* weight, float* sgate, int n, int W, int E, int top,
                                 hipStream_t stream) {
  return gibbs_moe_route_mode(h, ldh, dtype, router, router_bias, shared_gate, chosen, weight, sgate, n, W, E, top, 0, stream);
}

GIBBS_EXPORT int gibbs_moe_group(const int* chosen, int n_pairs, int E, int bm, int* sorted_pair, int* pair_pos, int* tile_expert,
                                 long cap, hipStream_t stream) {
  GIBBS_REQUIRE(chosen && sorted_pair && pair_pos && tile_expert && n_pairs > 0, "moe_group: bad operands pairs=%d", n_pairs);
  GIBBS_REQUIRE(E > 0 && E <= MOE_MAX_EXPERTS && (bm == 16 || bm == 128), "moe_group: %d experts (at most %d) in tiles of %d (16 or 128)", E, MOE_MAX_EXPERTS, bm);
  GIBBS_REQUIRE(cap >= gibbs_moe_capacity(n_pairs, E, bm) && cap % bm == 0 && cap < (1L << 31), "moe_group: %ld places for %d pairs of %d experts", cap, n_pairs, E);
  moe_group_kernel<<<1, 1024, 0, stream>>>(chosen, n_pairs, E, bm, sorted_pair, pair_pos, tile_expert, (int)cap);
  GIBBS_LAUNCH_STATUS("moe_group");
}

// Y[m] = W_a,e X[src(m)] (w_b null), or act(W_a,e X[src(m)]) * (W_b,e X[src(m)]), for every place m of the sorted pairs; e the
// expert of m's tile; src(m) = pair / top (top > 0: rows of the step, gathered) or m itself (top 0: X is in sorted order).
// W_a, W_b: [experts, O, I].
GIBBS_EXPORT int gibbs_moe_gemm(const void* X, long ldx, int top, const int* sorted_pair, const int* tile_expert, long cap, int bm,
                                const void* w_a, const void* w_b, void* Y, long ldy, int dtype, int O, int I, int act,
                                hipStream_t stream) {
  GIBBS_REQUIRE(X && sorted_pair && tile_expert && w_a && Y && O > 0 && I > 0 && ldx >= I && ldy >= O, "moe_gemm: bad operands O=%d I=%d", O, I);
  GIBBS_REQUIRE((bm == 16 || bm == 128) && cap > 0 && cap % bm == 0 && cap / bm <= 65535, "moe_gemm: %ld places in tiles of %d", cap, bm);
  GIBBS_REQUIRE(top >= 0 && act >= 0 && act < ACT_COUNT, "moe_gemm: bad choice count or activation");
  const long stride = (long)O * I;
  const int tiles = (int)(cap / bm);
#define MOE_PLAIN(T, BM, GLU)                                                                                                     \
  moe_gemm_plain_kernel<T, BM, GLU><<<dim3(ceil_div(O, 64), tiles), 256, 0, stream>>>((const T*)X, ldx, top, sorted_pair, tile_expert, \
                                                                                     (const T*)w_a, (const T*)w_b, stride, (T*)Y, ldy, O, I, act)
#define MOE_PLAIN_ANY(T)                                                                  \
  do {                                                                                    \
    if (bm == 128) { if (w_b) MOE_PLAIN(T, 128, true); else MOE_PLAIN(T, 128, false); }    \
    else { if (w_b) MOE_PLAIN(T, 16, true); else MOE_PLAIN(T, 16, false); }                \
  } while (0)
  if (dtype == GIBBS_F32) {
    MOE_PLAIN_ANY(float);
  } else if (dtype == GIBBS_BF16) {
    const bool aligned = I % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)X % 16) == 0 && ((uintptr_t)w_a % 16) == 0 && ((uintptr_t)w_b % 16) == 0;
    if (!aligned) {
      MOE_PLAIN_ANY(bf16);
    } else if (bm == 128) {
      if (w_b ? launch_tiled<true>((const bf16*)X, ldx, top, sorted_pair, tile_expert, tiles, (const bf16*)w_a, (const bf16*)w_b, stride, (bf16*)Y, ldy, O, I, act, stream)
              : launch_tiled<false>((const bf16*)X, ldx, top, sorted_pair, tile_expert, tiles, (const bf16*)w_a, nullptr, stride, (bf16*)Y, ldy, O, I, act, stream))
        return 1;
    } else if (w_b) {
      moe_gemm_few_kernel<true><<<dim3(ceil_div(O, 32), tiles), 256, 0, stream>>>((const bf16*)X, ldx, top, sorted_pair, tile_expert, (const bf16*)w_a,
                                                                                 (const bf16*)w_b, stride, (bf16*)Y, ldy, O, I, act);
    } else {
      moe_gemm_few_kernel<false><<<dim3(ceil_div(O, 32), tiles), 256, 0, stream>>>((const bf16*)X, ldx, top, sorted_pair, tile_expert, (const bf16*)w_a,
                                                                                  nullptr, stride, (bf16*)Y, ldy, O, I, act);
    }
  } else {
    return gibbs_fail("moe_gemm: unknown dtype %d", dtype);
  }
#undef MOE_PLAIN_ANY
#undef MOE_PLAIN
  GIBBS_LAUNCH_STATUS("moe_gemm");
}

// out[n] = sum_c weight[n][c] y[pair_pos[n * top + c]] + sgate[n] shared[n]  (shared null: no shared expert; sgate null: 1).
GIBBS_EXPORT int gibbs_moe_combine(const void* y, const int* pair_pos, const float* weight, const void* shared, const float* sgate,
                                   void* out, int dtype, int n, int top, int W, hipStream_t stream) {
  return gibbs_moe_combine_self(y, pair_pos, weight, shared, sgate, nullptr, out, dtype, n, top, W, stream);
}
// self [n, W] (null: none): the rows themselves, which a choice without a place (-1: an identity expert) stands for.
GIBBS_EXPORT int gibbs_moe_combine_self(const void* y, const int* pair_pos, const float* weight, const void* shared, const float* sgate,
                                        const void* self, void* out, int dtype, int n, int top, int W, hipStream_t stream) {
  GIBBS_REQUIRE(y && pair_pos && weight && out && n > 0 && top > 0 && W > 0, "moe_combine: bad operands n=%d top=%d width=%d", n, top, W);
  const size_t bytes = dtype == GIBBS_F32 ? 16 : 8;
  const bool vec = W % 4 == 0 && ((uintptr_t)y % bytes) == 0 && ((uintptr_t)shared % bytes) == 0 && ((uintptr_t)out % bytes) == 0 && ((uintptr_t)self % bytes) == 0;
  const int threads = vec ? (W >= 4096 ? 1024 : (W >= 1024 ? 256 : 64)) : (W >= 1024 ? 256 : 64);
#define MOE_COMBINE(T, V) moe_combine_kernel<T, V><<<n, threads, 0, stream>>>((const T*)y, pair_pos, weight, (const T*)shared, sgate, (const T*)self, (T*)out, top, W)
  if (dtype == GIBBS_F32) {
    if (vec) MOE_COMBINE(float, true); else MOE_COMBINE(float, false);
  } else if (dtype == GIBBS_BF16) {
    if (vec) MOE_COMBINE(bf16, true); else MOE_COMBINE(bf16, false);
  } else
    return gibbs_fail("moe_combine: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("moe_combine");
}
