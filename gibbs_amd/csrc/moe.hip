// Mixture of experts: a router picks `top` of E small gated feed-forwards for every row, and the row's result is
// the weighted sum of theirs; a shared expert may run for every row beside them, times a sigmoid gate of its own.
//
//   route      z = W_r h + b in float32 (h as the step holds it); the `top` largest logits (the lower index among
//              equals); weights = softmax over the chosen logits alone; gate = sigmoid(w_sg . h) for the shared expert
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
// that are not 16-byte aligned; 16 x 16 x 32 matrix-core products for aligned bfloat16 (operands straight from
// memory: rows of h and of every W are contiguous along k), float32 accumulators, the activation in float32.
#include "common.h"
#include "activation.h"

namespace {
constexpr int MOE_MAX_EXPERTS = 1024;

// ------------------------------------------------------------------------------------------------- route
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, long ldh, const float* __restrict__ router,
                                                        const float* __restrict__ router_bias, const float* __restrict__ shared_gate,
                                                        int* __restrict__ chosen, float* __restrict__ weight, float* __restrict__ sgate,
                                                        int W, int E, int top) {
  extern __shared__ float z[];   // [E]
  const int n = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, n_waves = blockDim.x / WAVE;
  const T* row = h + (size_t)n * ldh;
  for (int e = wave; e < E; e += n_waves) {
    const float* w = router + (size_t)e * W;
    float s = 0.f;
    for (int k = lane; k < W; k += WAVE) s = fmaf(to_float(row[k]), w[k], s);
    s = wave_sum(s);
    if (lane == 0) z[e] = s + (router_bias ? router_bias[e] : 0.f);
  }
  if (shared_gate && wave == 0) {
    float s = 0.f;
    for (int k = lane; k < W; k += WAVE) s = fmaf(to_float(row[k]), shared_gate[k], s);
    s = wave_sum(s);
    if (lane == 0) sgate[n] = 1.0f / (1.0f + expf(-s));
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  // the `top` largest, in descending order; the lower index among equal logits; then the softmax over them alone
  int* mine = chosen + (size_t)n * top;
  float* wts = weight + (size_t)n * top;
  float best = 0.f;
  for (int c = 0; c < top; ++c) {
    int pick = -1;
    float pv = 0.f;
    for (int e = 0; e < E; ++e) {
      const float v = z[e];
      if (v != v) continue;
      bool taken = false;
      for (int d = 0; d < c; ++d) taken |= mine[d] == e;
      if (!taken && (pick < 0 || v > pv)) { pick = e; pv = v; }
    }
    if (pick < 0) {   // (fewer usable logits than choices: the first expert not taken yet, with no weight)
      for (int e = 0; e < E && pick < 0; ++e) {
        bool taken = false;
        for (int d = 0; d < c; ++d) taken |= mine[d] == e;
        if (!taken) pick = e;
      }
      pv = -INFINITY;
    }
    mine[c] = pick;
    wts[c] = pv;
    if (c == 0) best = pv;
  }
  float sum = 0.f;
  for (int c = 0; c < top; ++c) {
    const float e = wts[c] == -INFINITY ? 0.f : expf(wts[c] - best);
    wts[c] = e;
    sum += e;
  }
  for (int c = 0; c < top; ++c) wts[c] = sum > 0.f ? wts[c] / sum : 0.f;
}

// ------------------------------------------------------------------------------------------------- group
// One workgroup: counts per expert, every expert's stretch rounded up to whole tiles, then each pair takes the next
// free place of its expert's stretch.  sorted_pair [cap]: the pair at each place (-1: padding); pair_pos [n_pairs]:
// each pair's place; tile_expert [cap / bm]: the expert of each tile (-1: beyond the last stretch).
__global__ __launch_bounds__(1024) void moe_group_kernel(const int* __restrict__ chosen, int n_pairs, int E, int bm,
                                                         int* __restrict__ sorted_pair, int* __restrict__ pair_pos,
                                                         int* __restrict__ tile_expert, int cap) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int start[MOE_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  for (int m = threadIdx.x; m < cap; m += blockDim.x) sorted_pair[m] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) atomicAdd(&count[chosen[i]], 1);
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
// bfloat16, inner size a multiple of 8, rows 16-byte aligned.  W is the first operand (the tile is Y^T = W X^T): lane l
// holds the 8 values k = (l / 16) * 8 .. + 8 of feature or row l % 16, and its four results are four neighbouring
// features of row l % 16.  BM 64: a workgroup's four waves take 16 places each and the same 64 features.  BM 16: all
// four take the same 16 places and 64 features each (256 a workgroup): few pairs, the matrices are streamed once.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
template <int BM, bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16* __restrict__ X, long ldx, int top, const int* __restrict__ sorted_pair,
                                                            const int* __restrict__ tile_expert, const bf16* __restrict__ Wa,
                                                            const bf16* __restrict__ Wb, long expert_stride, bf16* __restrict__ Y, long ldy,
                                                            int O, int I, int act) {
  const int tile = blockIdx.y, e = tile_expert[tile];
  if (e < 0) return;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, lr = lane % 16, lg = lane / 16;
  const int place = tile * BM + (BM == 64 ? wave * 16 : 0) + lr;
  const int col0 = BM == 64 ? blockIdx.x * 64 : blockIdx.x * 256 + wave * 64;
  if (col0 >= O) return;
  const int pair = sorted_pair[place];
  const long src = pair < 0 ? -1 : (top > 0 ? pair / top : place);
  const bf16* xr = X + (size_t)(src < 0 ? 0 : src) * ldx;
  const bf16* wa = Wa + (size_t)e * expert_stride;
  const bf16* wb = GLU ? Wb + (size_t)e * expert_stride : nullptr;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  floatx4 acc_a[4], acc_b[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) acc_a[t] = acc_b[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < I; k0 += 32) {
    const int k = k0 + lg * 8;
    const bf16x8 x8 = (src >= 0 && k < I) ? *(const bf16x8*)(xr + k) : zero8;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int col = col0 + t * 16 + lr;
      const bool in = col < O && k < I;
      const bf16x8 a8 = in ? *(const bf16x8*)(wa + (size_t)col * I + k) : zero8;
      acc_a[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a8, x8, acc_a[t], 0, 0, 0);
      if (GLU) {
        const bf16x8 b8 = in ? *(const bf16x8*)(wb + (size_t)col * I + k) : zero8;
        acc_b[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b8, x8, acc_b[t], 0, 0, 0);
      }
    }
  }
  if (src < 0) return;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = col0 + t * 16 + lg * 4 + i;
      if (col >= O) continue;
      const float v = GLU ? activate(acc_a[t][i], act) * acc_b[t][i] : acc_a[t][i];
      Y[(size_t)place * ldy + col] = (bf16)v;
    }
}

// ------------------------------------------------------------------------------------------------- combine
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ pair_pos, const float* __restrict__ weight,
                                   const T* __restrict__ shared, const float* __restrict__ sgate, T* __restrict__ out, int top, int W) {
  const int n = blockIdx.x;
  const float g = shared ? (sgate ? sgate[n] : 1.0f) : 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < top; ++s) v = fmaf(weight[(size_t)n * top + s], to_float(y[(size_t)pair_pos[(size_t)n * top + s] * W + c]), v);
    if (shared) v = fmaf(g, to_float(shared[(size_t)n * W + c]), v);
    out[(size_t)n * W + c] = from_float<T>(v);
  }
}
}  // namespace

// Places that the sorted pairs of a step can take at most: every expert's stretch rounded up to whole tiles.
GIBBS_EXPORT long gibbs_moe_capacity(int n_pairs, int E, int bm) {
  return ((long)n_pairs + (long)E * (bm - 1) + bm - 1) / bm * bm;
}
// Tiles of pairs: 16 while the matrices are streamed for few pairs each, 64 beyond.
GIBBS_EXPORT int gibbs_moe_tile(int n_pairs, int E) { return (long)n_pairs <= 32L * E ? 16 : 64; }

GIBBS_EXPORT int gibbs_moe_route(const void* h, long ldh, int dtype, const float* router, const float* router_bias,
                                 const float* shared_gate, int* chosen, float* weight, float* sgate, int n, int W, int E, int top,
                                 hipStream_t stream) {
  GIBBS_REQUIRE(h && router && chosen && weight && n > 0 && W > 0 && ldh >= W, "moe_route: bad operands n=%d width=%d", n, W);
  GIBBS_REQUIRE(E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= E, "moe_route: %d of %d experts (at most %d)", top, E, MOE_MAX_EXPERTS);
  GIBBS_REQUIRE(!shared_gate || sgate, "moe_route: a shared expert's gate needs its output");
  const size_t lds = (size_t)E * sizeof(float);
  if (dtype == GIBBS_F32)
    moe_route_kernel<float><<<n, 256, lds, stream>>>((const float*)h, ldh, router, router_bias, shared_gate, chosen, weight, sgate, W, E, top);
  else if (dtype == GIBBS_BF16)
    moe_route_kernel<bf16><<<n, 256, lds, stream>>>((const bf16*)h, ldh, router, router_bias, shared_gate, chosen, weight, sgate, W, E, top);
  else
    return gibbs_fail("moe_route: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("moe_route");
}

GIBBS_EXPORT int gibbs_moe_group(const int* chosen, int n_pairs, int E, int bm, int* sorted_pair, int* pair_pos, int* tile_expert,
                                 long cap, hipStream_t stream) {
  GIBBS_REQUIRE(chosen && sorted_pair && pair_pos && tile_expert && n_pairs > 0, "moe_group: bad operands pairs=%d", n_pairs);
  GIBBS_REQUIRE(E > 0 && E <= MOE_MAX_EXPERTS && (bm == 16 || bm == 64), "moe_group: %d experts (at most %d) in tiles of %d (16 or 64)", E, MOE_MAX_EXPERTS, bm);
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
  GIBBS_REQUIRE((bm == 16 || bm == 64) && cap > 0 && cap % bm == 0 && cap / bm <= 65535, "moe_gemm: %ld places in tiles of %d", cap, bm);
  GIBBS_REQUIRE(top >= 0 && act >= 0 && act < ACT_COUNT, "moe_gemm: bad choice count or activation");
  const long stride = (long)O * I;
  const int tiles = (int)(cap / bm);
#define MOE_PLAIN(T, BM, GLU)                                                                                                     \
  moe_gemm_plain_kernel<T, BM, GLU><<<dim3(ceil_div(O, 64), tiles), 256, 0, stream>>>((const T*)X, ldx, top, sorted_pair, tile_expert, \
                                                                                     (const T*)w_a, (const T*)w_b, stride, (T*)Y, ldy, O, I, act)
#define MOE_MFMA(BM, GLU)                                                                                                          \
  moe_gemm_mfma_kernel<BM, GLU><<<dim3(ceil_div(O, BM == 64 ? 64 : 256), tiles), 256, 0, stream>>>(                                 \
      (const bf16*)X, ldx, top, sorted_pair, tile_expert, (const bf16*)w_a, (const bf16*)w_b, stride, (bf16*)Y, ldy, O, I, act)
#define MOE_PICK(LAUNCH, ...)                                        \
  do {                                                               \
    if (bm == 64) { if (w_b) LAUNCH(__VA_ARGS__ 64, true); else LAUNCH(__VA_ARGS__ 64, false); } \
    else { if (w_b) LAUNCH(__VA_ARGS__ 16, true); else LAUNCH(__VA_ARGS__ 16, false); }          \
  } while (0)
  if (dtype == GIBBS_F32) {
    MOE_PICK(MOE_PLAIN, float,);
  } else if (dtype == GIBBS_BF16) {
    const bool aligned = I % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)X % 16) == 0 && ((uintptr_t)w_a % 16) == 0 && ((uintptr_t)w_b % 16) == 0;
    if (aligned) MOE_PICK(MOE_MFMA,); else MOE_PICK(MOE_PLAIN, bf16,);
  } else {
    return gibbs_fail("moe_gemm: unknown dtype %d", dtype);
  }
#undef MOE_PICK
#undef MOE_MFMA
#undef MOE_PLAIN
  GIBBS_LAUNCH_STATUS("moe_gemm");
}

// out[n] = sum_c weight[n][c] y[pair_pos[n * top + c]] + sgate[n] shared[n]  (shared null: no shared expert; sgate null: 1).
GIBBS_EXPORT int gibbs_moe_combine(const void* y, const int* pair_pos, const float* weight, const void* shared, const float* sgate,
                                   void* out, int dtype, int n, int top, int W, hipStream_t stream) {
  GIBBS_REQUIRE(y && pair_pos && weight && out && n > 0 && top > 0 && W > 0, "moe_combine: bad operands n=%d top=%d width=%d", n, top, W);
  const int threads = W >= 1024 ? 256 : 64;
  if (dtype == GIBBS_F32)
    moe_combine_kernel<float><<<n, threads, 0, stream>>>((const float*)y, pair_pos, weight, (const float*)shared, sgate, (float*)out, top, W);
  else if (dtype == GIBBS_BF16)
    moe_combine_kernel<bf16><<<n, threads, 0, stream>>>((const bf16*)y, pair_pos, weight, (const bf16*)shared, sgate, (bf16*)out, top, W);
  else
    return gibbs_fail("moe_combine: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("moe_combine");
}
