// The state-space rule in chunks, for one request's long stretch of rows: what recurrent.hip's walk does token by token,
//   S_t = a_t S_(t-1) + k_t v_t',   y_t = S_t' q_t        (S [D, V]; one decay a_t per head and token; all float32),
// regrouped so that every product is a small matrix product and only a sum over chunks runs in order.  With chunks of
// L = 64 tokens, c_t = sum of log a over the chunk's tokens up to t, and S_0 the state in front of the chunk:
//   y_t = exp(c_t) S_0' q_t + sum_(s <= t) exp(c_t - c_s) (k_s . q_t) v_s         S_L = exp(c_L) S_0 + sum_s exp(c_L - c_s) k_s v_s'
// (A step of one token per request has a kernel of its own at the end of this file.)
// Three kernels: (1) per (chunk, head, 64 columns of V): G = mask .* (Q K'), Y = G V, and the chunk's own contribution
// U = K' diag(exp(c_L - c_s)) V; (2) per element of the state, over the chunks in order: what stood in front of each
// chunk (written where U was) and the state behind the last; (3) per (chunk, head, columns): Y += diag(exp(c_t)) Q S_0.
// The exponents are differences of sums of logarithms of decays, never positive, so nothing overflows.  The order of
// additions differs from the walk's: a prompt cut elsewhere agrees to rounding, not to the bit.
#include "common.h"

namespace {
constexpr int L = 64, VB = 64, DMAX = 128, NT = 256;
constexpr int RT = L * 16 / NT;        // rows of a thread's RT x 4 tile of a 64 x 64 result (16 threads across the columns)
constexpr int ROWG = NT / 16;          // row groups of the tiles
constexpr int VEC_LOADS = L * DMAX / 4 / NT;   // 16-byte vectors a thread brings in for a 64 x 128 operand
constexpr int DH = 64;                 // channels of Q and K that the local kernel holds in LDS at a time
constexpr int LDQ = DMAX + 4, LDH = DH + 4, LDV = VB + 4, LDG = L + 4;

struct ChunkArgs {
  const float* q; const float* k; long ldqk;      // [rows, G * D]: C and B of the rows
  const float* v; long ldv;                       // [rows, H * V]: dt x
  const float* log_decay;                         // [rows, H]: log a_t (never positive)
  float* u;                                       // [chunks, H, D, V] workspace: U, then the state in front of each chunk
  float* total_log;                               // [chunks, H] workspace: every chunk's sum of log decays
  float* state_base; long slot_stride; const int* slot;   // the request's state [H, D, V] is state_base + slot[0] * slot_stride
  float* out;                                     // [rows, H * V]
  int rows, H, G, D, V;
};

// c_t for the chunk's 64 tokens (rows beyond the request's end: as the last real one, so that they change nothing)
__device__ __forceinline__ void chunk_sums(const ChunkArgs& a, int t0, int h, float* cum) {
  if (threadIdx.x < WAVE) {
    const int t = t0 + threadIdx.x;
    float x = t < a.rows ? a.log_decay[(size_t)t * a.H + h] : 0.f;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
      const float y = __shfl_up(x, o, WAVE);
      if ((int)threadIdx.x >= o) x += y;
    }
    cum[threadIdx.x] = x;
  }
}
// rows t0 .. t0 + 63 of a [rows, ld] matrix, `width` columns from column c0 (both multiples of 4, rows 16-byte aligned), into
// LDS rows of `lds_ld` (zeros beyond): a thread's vectors are all asked for before the first is stored
__device__ __forceinline__ void load_rows(const float* src, long ld, int c0, int width, int pad_width, int t0, int rows, float* dst, int lds_ld) {
  const int per_row = pad_width / 4, count = L * per_row;
  float4 r[VEC_LOADS];
#pragma unroll
  for (int u = 0; u < VEC_LOADS; ++u) {
    const int i = threadIdx.x + u * NT, t = i / per_row, c = (i % per_row) * 4;
    r[u] = (i < count && t0 + t < rows && c < width) ? *(const float4*)(src + (size_t)(t0 + t) * ld + c0 + c) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int u = 0; u < VEC_LOADS; ++u) {
    const int i = threadIdx.x + u * NT, t = i / per_row, c = (i % per_row) * 4;
    if (i < count) *(float4*)(dst + t * lds_ld + c) = r[u];
  }
}

__global__ __launch_bounds__(NT) void ssd_chunk_local_kernel(ChunkArgs a) {
  // Q and K come through LDS in halves of 64 channels (70 KB in all: two workgroups a compute unit, so that one's waits
  // for LDS are the other's arithmetic); the scores' tile stays in registers across the halves.
  extern __shared__ float lds[];
  float* sQ = lds;                    // [L][LDH]: 64 channels of Q
  float* sK = sQ + L * LDH;           // [L][LDH]
  float* sV = sK + L * LDH;           // [L][LDV]
  float* sG = sV + L * LDV;           // [L][LDG]
  float* cum = sG + L * LDG;          // [L]
  float* sW = cum + L;                // [L]: exp(c_L - c_s)
  const int chunk = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * VB;
  const int t0 = chunk * L, g = h / (a.H / a.G), D = a.D;
  const int vw = min(VB, a.V - j0);
  const int ty = threadIdx.x / 16, tx = threadIdx.x % 16;      // an RT x 4 tile of a 64 x 64 result
  chunk_sums(a, t0, h, cum);
  load_rows(a.v, a.ldv, h * a.V + j0, vw, VB, t0, a.rows, sV, LDV);
  __syncthreads();
  if (blockIdx.z == 0 && threadIdx.x == 0) a.total_log[(size_t)chunk * a.H + h] = cum[L - 1];
  if (threadIdx.x < L) sW[threadIdx.x] = expf(cum[L - 1] - cum[threadIdx.x]);      // (read behind the next barrier)
  float* u = a.u + ((size_t)chunk * a.H + h) * D * a.V;
  float gacc[RT][4] = {};
  for (int d0 = 0; d0 < D; d0 += DH) {
    const int dw = min(DH, D - d0);
    __syncthreads();      // (everyone is done with the half before)
    load_rows(a.q, a.ldqk, g * D + d0, dw, DH, t0, a.rows, sQ, LDH);
    load_rows(a.k, a.ldqk, g * D + d0, dw, DH, t0, a.rows, sK, LDH);
    __syncthreads();
    // G[t][s] += q_t . k_s over this half's channels
    for (int d = 0; d < DH; d += 4) {
      float4 qa[RT], kb[4];
#pragma unroll
      for (int i = 0; i < RT; ++i) qa[i] = *(const float4*)&sQ[(RT * ty + i) * LDH + d];
#pragma unroll
      for (int i = 0; i < 4; ++i) kb[i] = *(const float4*)&sK[(4 * tx + i) * LDH + d];
#pragma unroll
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          gacc[i][j] = fmaf(qa[i].x, kb[j].x, gacc[i][j]); gacc[i][j] = fmaf(qa[i].y, kb[j].y, gacc[i][j]);
          gacc[i][j] = fmaf(qa[i].z, kb[j].z, gacc[i][j]); gacc[i][j] = fmaf(qa[i].w, kb[j].w, gacc[i][j]);
        }
    }
    // U[i][j] = sum_s exp(c_L - c_s) K[s][i] V[s][j] for this half's rows i = d0 + ty + ROWG m: 4 columns of V a thread
    float acc[DH / ROWG][4] = {};
    for (int s = 0; s < L; ++s) {
      const float w = sW[s];
      const float4 vb = *(const float4*)&sV[s * LDV + 4 * tx];
      const float4 wv = make_float4(w * vb.x, w * vb.y, w * vb.z, w * vb.w);
#pragma unroll
      for (int m = 0; m < DH / ROWG; ++m) {
        const float kv = sK[s * LDH + ty + ROWG * m];
        acc[m][0] = fmaf(kv, wv.x, acc[m][0]); acc[m][1] = fmaf(kv, wv.y, acc[m][1]);
        acc[m][2] = fmaf(kv, wv.z, acc[m][2]); acc[m][3] = fmaf(kv, wv.w, acc[m][3]);
      }
    }
#pragma unroll
    for (int m = 0; m < DH / ROWG; ++m) {
      const int i = d0 + ty + ROWG * m;
      if (i >= D) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (4 * tx + j < vw) u[(size_t)i * a.V + j0 + 4 * tx + j] = acc[m][j];
    }
  }
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = RT * ty + i, s = 4 * tx + j;
      sG[t * LDG + s] = s <= t ? gacc[i][j] * expf(cum[t] - cum[s]) : 0.f;
    }
  __syncthreads();
  // Y[t][j] = sum_s G[t][s] V[s][j]
  float acc[RT][4] = {};
  for (int s = 0; s < L; s += 4) {
    float4 ga[RT], vb[4];
#pragma unroll
    for (int i = 0; i < RT; ++i) ga[i] = *(const float4*)&sG[(RT * ty + i) * LDG + s];
#pragma unroll
    for (int i = 0; i < 4; ++i) vb[i] = *(const float4*)&sV[(s + i) * LDV + 4 * tx];
#pragma unroll
    for (int i = 0; i < RT; ++i) {
      const float gs[4] = {ga[i].x, ga[i].y, ga[i].z, ga[i].w};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        acc[i][0] = fmaf(gs[kk], vb[kk].x, acc[i][0]); acc[i][1] = fmaf(gs[kk], vb[kk].y, acc[i][1]);
        acc[i][2] = fmaf(gs[kk], vb[kk].z, acc[i][2]); acc[i][3] = fmaf(gs[kk], vb[kk].w, acc[i][3]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    const int t = t0 + RT * ty + i;
    if (t >= a.rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (4 * tx + j < vw) a.out[(size_t)t * a.H * a.V + (size_t)h * a.V + j0 + 4 * tx + j] = acc[i][j];
  }
}

// Over the chunks in order, per element of the state: u[c] becomes the state in front of chunk c, the slot's state the one
// behind the last chunk.
__global__ void ssd_chunk_scan_kernel(ChunkArgs a, int chunks) {
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t per_head = (size_t)a.D * a.V, total = (size_t)a.H * per_head;
  if (e >= total) return;
  const int h = (int)(e / per_head);
  float* state = a.state_base + (size_t)a.slot[0] * a.slot_stride;
  float S = state[e];
  for (int c = 0; c < chunks; ++c) {
    float* u = a.u + (size_t)c * total + e;
    const float own = *u;
    *u = S;
    S = fmaf(expf(a.total_log[(size_t)c * a.H + h]), S, own);
  }
  state[e] = S;
}

__global__ __launch_bounds__(NT) void ssd_chunk_carry_kernel(ChunkArgs a) {
  extern __shared__ float lds[];
  float* sQ = lds;                    // [L][LDQ]
  float* sS = sQ + L * LDQ;           // [DMAX][LDV]: the state in front of the chunk, 64 columns of it
  float* cum = sS + DMAX * LDV;       // [L]
  const int chunk = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * VB;
  const int t0 = chunk * L, g = h / (a.H / a.G), D = a.D, Dp = (D + 3) / 4 * 4;
  const int vw = min(VB, a.V - j0);
  chunk_sums(a, t0, h, cum);
  load_rows(a.q, a.ldqk, g * D, D, Dp, t0, a.rows, sQ, LDQ);
  const float* s0 = a.u + ((size_t)chunk * a.H + h) * D * a.V;
  {   // the state's 64 columns: D x 16 vectors, asked for together
    float4 r[VEC_LOADS];
#pragma unroll
    for (int u = 0; u < VEC_LOADS; ++u) {
      const int i = threadIdx.x + u * NT, row = i / (VB / 4), c = (i % (VB / 4)) * 4;
      r[u] = (row < D && c < vw) ? *(const float4*)(s0 + (size_t)row * a.V + j0 + c) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < VEC_LOADS; ++u) {
      const int i = threadIdx.x + u * NT, row = i / (VB / 4), c = (i % (VB / 4)) * 4;
      if (row < Dp) *(float4*)(sS + row * LDV + c) = r[u];
    }
  }
  __syncthreads();
  const int ty = threadIdx.x / 16, tx = threadIdx.x % 16;
  float acc[RT][4] = {};
  for (int d = 0; d < Dp; d += 4) {
    float4 qa[RT], sb[4];
#pragma unroll
    for (int i = 0; i < RT; ++i) qa[i] = *(const float4*)&sQ[(RT * ty + i) * LDQ + d];
#pragma unroll
    for (int i = 0; i < 4; ++i) sb[i] = *(const float4*)&sS[(d + i) * LDV + 4 * tx];
#pragma unroll
    for (int i = 0; i < RT; ++i) {
      const float qs[4] = {qa[i].x, qa[i].y, qa[i].z, qa[i].w};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        acc[i][0] = fmaf(qs[kk], sb[kk].x, acc[i][0]); acc[i][1] = fmaf(qs[kk], sb[kk].y, acc[i][1]);
        acc[i][2] = fmaf(qs[kk], sb[kk].z, acc[i][2]); acc[i][3] = fmaf(qs[kk], sb[kk].w, acc[i][3]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    const int t = t0 + RT * ty + i;
    if (t >= a.rows) continue;
    const float e = expf(cum[RT * ty + i]);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (4 * tx + j < vw) {
        float* o = a.out + (size_t)t * a.H * a.V + (size_t)h * a.V + j0 + 4 * tx + j;
        *o = fmaf(e, acc[i][j], *o);
      }
  }
}
// One token per request (a step of decoded tokens): the state is streamed once, in whole rows.  A workgroup takes 64 columns
// of one head's state; thread (lane, part) owns column j and the rows i = part, part + STEP_PARTS, ...: S_ij = a S_ij + k_i v_j
// (the walk's own arithmetic, so the state is the walk's to the bit), y_j = sum_i S_ij q_i by parts that are added in order.
constexpr int STEP_PARTS = 4;
__global__ __launch_bounds__(64 * STEP_PARTS) void ssd_step_kernel(const float* __restrict__ q, const float* __restrict__ k, long ldqk,
                                                                   const float* __restrict__ v, long ldv, const float* __restrict__ decay,
                                                                   float* __restrict__ state, long slot_stride, const int* __restrict__ slot,
                                                                   float* __restrict__ out, int H, int G, int D, int V) {
  __shared__ float sq[256], sk[256], sy[STEP_PARTS][64];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, part = threadIdx.y;
  const int j = blockIdx.z * 64 + lane, g = h / (H / G);
  for (int i = part * 64 + lane; i < D; i += 64 * STEP_PARTS) {
    sq[i] = q[(size_t)n * ldqk + (size_t)g * D + i];
    sk[i] = k[(size_t)n * ldqk + (size_t)g * D + i];
  }
  __syncthreads();
  float y = 0.f;
  if (j < V) {
    const float a = decay[(size_t)n * H + h], vj = v[(size_t)n * ldv + (size_t)h * V + j];
    float* st = state + (size_t)slot[n] * slot_stride + (size_t)h * D * V + j;
    // (eight rows at a time: their loads are all asked for before the first store, which the compiler must take to alias them)
    for (int i0 = part; i0 < D; i0 += 8 * STEP_PARTS) {
      float s[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u * STEP_PARTS;
        s[u] = i < D ? st[(size_t)i * V] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u * STEP_PARTS;
        if (i < D) {
          s[u] = fmaf(a, s[u], sk[i] * vj);
          st[(size_t)i * V] = s[u];
          y = fmaf(s[u], sq[i], y);
        }
      }
    }
  }
  sy[part][lane] = y;
  __syncthreads();
  if (part == 0 && j < V) {
    float total = sy[0][lane];
#pragma unroll
    for (int p = 1; p < STEP_PARTS; ++p) total += sy[p][lane];
    out[(size_t)n * H * V + (size_t)h * V + j] = total;
  }
}
}  // namespace

// Floats of workspace that `rows` rows of one request need (0: the chunked form does not take these sizes).
GIBBS_EXPORT long gibbs_ssd_chunked_workspace(int rows, int H, int D, int V) {
  if (rows <= 0 || H <= 0 || D <= 0 || D > DMAX || D % 4 || V <= 0 || V % 4) return 0;
  return (long)ceil_div(rows, L) * H * ((long)D * V + 1);
}

// One request's rows through the rule in chunks of 64: q, k [rows, >= G D] (row stride ldqk), v [rows, >= H V] (stride ldv),
// log_decay [rows, H]; the request's state [H, D, V] at state + slot[0] * slot_stride (slot on the device) is read and left as
// the rule leaves it; out [rows, H V]; workspace of gibbs_ssd_chunked_workspace floats.  All float32.
GIBBS_EXPORT int gibbs_ssd_chunked(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* log_decay, float* state,
                                   long slot_stride, const int* slot, float* out, float* workspace, int rows, int H, int G, int D, int V,
                                   hipStream_t stream) {
  GIBBS_REQUIRE(q && k && v && log_decay && state && slot && out && workspace && rows > 0, "ssd_chunked: null operand or no rows");
  GIBBS_REQUIRE(slot_stride >= (long)H * D * V, "ssd_chunked: a slot of %ld floats cannot hold %d x %d x %d", slot_stride, H, D, V);
  GIBBS_REQUIRE(H > 0 && G > 0 && H % G == 0 && D > 0 && D <= DMAX && V > 0 && ldqk >= (long)G * D && ldv >= (long)H * V,
                "ssd_chunked: bad sizes heads=%d groups=%d D=%d (up to %d) V=%d", H, G, D, DMAX, V);
  GIBBS_REQUIRE(D % 4 == 0 && V % 4 == 0 && ldqk % 4 == 0 && ldv % 4 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0 &&
                ((uintptr_t)workspace % 16) == 0, "ssd_chunked: sizes and row strides in whole 16 bytes (D=%d V=%d strides %ld, %ld)", D, V, ldqk, ldv);
  const int chunks = ceil_div(rows, L);
  GIBBS_REQUIRE(H <= 65535 && ceil_div(V, VB) <= 65535, "ssd_chunked: too many heads or columns");
  ChunkArgs a{q, k, ldqk, v, ldv, log_decay, workspace, workspace + (size_t)chunks * H * D * V, state, slot_stride, slot, out, rows, H, G, D, V};
  const dim3 grid(chunks, H, ceil_div(V, VB));
  const size_t lds_local = (size_t)(2 * L * LDH + L * LDV + L * LDG + 2 * L) * sizeof(float);
  const size_t lds_carry = (size_t)(L * LDQ + DMAX * LDV + L) * sizeof(float);
  static bool raised = false;
  if (!raised) {
    if (hipFuncSetAttribute((const void*)ssd_chunk_local_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_local) != hipSuccess ||
        hipFuncSetAttribute((const void*)ssd_chunk_carry_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_carry) != hipSuccess)
      return gibbs_fail("ssd_chunked: the kernels' LDS could not be reserved");
    raised = true;
  }
  ssd_chunk_local_kernel<<<grid, NT, lds_local, stream>>>(a);
  const long total = (long)H * D * V;
  ssd_chunk_scan_kernel<<<ceil_div(total, 256), 256, 0, stream>>>(a, chunks);
  ssd_chunk_carry_kernel<<<grid, NT, lds_carry, stream>>>(a);
  GIBBS_LAUNCH_STATUS("ssd_chunked");
}

// The rule for a step in which every request brings one row (row n is request n): q, k [n_req, >= G D], v [n_req, >= H V], decay
// [n_req, H], the requests' states at state + slot[n] * slot_stride, out [n_req, H V].  All float32; D up to 256.
GIBBS_EXPORT int gibbs_ssd_step(const float* q, const float* k, long ldqk, const float* v, long ldv, const float* decay, float* state,
                                long slot_stride, const int* slot, float* out, int n_req, int H, int G, int D, int V, hipStream_t stream) {
  GIBBS_REQUIRE(q && k && v && decay && state && slot && out && n_req > 0, "ssd_step: null operand or no rows");
  GIBBS_REQUIRE(H > 0 && G > 0 && H % G == 0 && D > 0 && D <= 256 && V > 0 && ldqk >= (long)G * D && ldv >= (long)H * V && slot_stride >= (long)H * D * V,
                "ssd_step: bad sizes heads=%d groups=%d D=%d (up to 256) V=%d", H, G, D, V);
  GIBBS_REQUIRE(H <= 65535 && ceil_div(V, 64) <= 65535, "ssd_step: too many heads or columns");
  ssd_step_kernel<<<dim3(n_req, H, ceil_div(V, 64)), dim3(64, STEP_PARTS), 0, stream>>>(q, k, ldqk, v, ldv, decay, state, slot_stride, slot, out, H, G, D, V);
  GIBBS_LAUNCH_STATUS("ssd_step");
}
