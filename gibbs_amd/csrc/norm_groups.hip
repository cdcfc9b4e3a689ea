// RMS norm in groups: a row of H values is cut into G equal consecutive parts, each part is divided by its own
// sqrt(mean(part^2) + eps), and the whole is multiplied by a gain [H].  G = 1 is the plain RMS norm.
//
// One kernel does what a sublayer normed on both sides needs at its borders, a workgroup per row, the row in LDS
// between the two norms, everything in float32:
//
//   x += norm_Gd(delta) gain_d        (delta: [N, H] in the activation type, or float32 partial sums added in order)
//   out = norm_Gn(x) gain_n           (all rows, or the rows that `rows` names: then there is no delta)
//
// either of which may be left out.  The sums of squares of a part are taken by `S` waves over equal stretches of it
// (S chosen by H and G alone) and folded in a fixed order, so a row's result depends on nothing but the row.
#include "common.h"
#include <algorithm>

namespace {
constexpr int GN_THREADS = 256, GN_WAVES = GN_THREADS / WAVE, GN_MAX_UNITS = 1024;

// inv[g] = 1 / sqrt(mean(v[part g]^2) + eps) for every part, v in LDS
__device__ __forceinline__ void group_inverse_roots(const float* v, int H, int G, int S, float eps, float* unit_sums, float* inv) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int part = H / G, seg = (part + S - 1) / S;
  for (int u = wave; u < G * S; u += GN_WAVES) {
    const int g = u / S, s = u % S;
    const int lo = g * part + s * seg, hi = min(g * part + part, lo + seg);
    float ss = 0.f;
    for (int i = lo + lane; i < hi; i += WAVE) ss = fmaf(v[i], v[i], ss);
    ss = wave_sum(ss);
    if (lane == 0) unit_sums[u] = ss;
  }
  __syncthreads();
  for (int g = threadIdx.x; g < G; g += GN_THREADS) {
    float total = 0.f;
    for (int s = 0; s < S; ++s) total += unit_sums[g * S + s];
    inv[g] = 1.0f / sqrtf(total / (float)part + eps);
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(GN_THREADS) void group_norm_kernel(float* __restrict__ x, const void* __restrict__ delta, int parts,
                                                               size_t part_stride, const float* __restrict__ gain_d, float eps_d,
                                                               int groups_d, const float* __restrict__ gain_n, float eps_n, int groups_n,
                                                               T* __restrict__ out, const int* __restrict__ rows, int H) {
  extern __shared__ float lds[];     // [H] the row, [units] partial sums, [groups] inverse roots
  const int Gmax = max(groups_d, groups_n);
  const int Sd = max(1, GN_WAVES / max(groups_d, 1)), Sn = max(1, GN_WAVES / max(groups_n, 1));
  float* v = lds;
  float* unit_sums = lds + H;
  float* inv = unit_sums + Gmax * max(Sd, Sn);
  const int n_out = blockIdx.x;
  const int n = rows ? rows[n_out] : n_out;
  float* xr = x + (size_t)n * H;
  if (delta) {
    if (parts >= 2) {
      const float* d = (const float*)delta + (size_t)n * H;
      for (int i = threadIdx.x; i < H; i += GN_THREADS) {
        float s = d[i];
        for (int p = 1; p < parts; ++p) s += d[(size_t)p * part_stride + i];
        v[i] = s;
      }
    } else {
      const T* d = (const T*)delta + (size_t)n * H;
      for (int i = threadIdx.x; i < H; i += GN_THREADS) v[i] = to_float(d[i]);
    }
    __syncthreads();
    group_inverse_roots(v, H, groups_d, Sd, eps_d, unit_sums, inv);
    const int part = H / groups_d;
    for (int i = threadIdx.x; i < H; i += GN_THREADS) {
      const float nv = xr[i] + v[i] * inv[i / part] * gain_d[i];
      xr[i] = nv;
      v[i] = nv;
    }
    __syncthreads();
  } else if (out) {
    for (int i = threadIdx.x; i < H; i += GN_THREADS) v[i] = xr[i];
    __syncthreads();
  }
  if (!out) return;
  group_inverse_roots(v, H, groups_n, Sn, eps_n, unit_sums, inv);
  const int part = H / groups_n;
  T* o = out + (size_t)n_out * H;
  for (int i = threadIdx.x; i < H; i += GN_THREADS) o[i] = from_float<T>(v[i] * inv[i / part] * gain_n[i]);
}

// y[n, :] = norm_G(in[n, :] (* act(gate[n, :]))) * gain: the norm of rows that are not the residual stream (a mixer's
// read-out), float32 in; with a gate the rows are multiplied by silu(gate) first, and `skip` [n, C] times `skip_w[c / skip_len]`
// is added before that.
template <typename T>
__global__ __launch_bounds__(GN_THREADS) void gated_group_norm_kernel(const float* __restrict__ in, const float* __restrict__ skip, long ld_skip,
                                                                     const float* __restrict__ skip_w, int skip_len,
                                                                     const T* __restrict__ gate, long ld_gate, const float* __restrict__ gain,
                                                                     float eps, int groups, T* __restrict__ y, int C) {
  extern __shared__ float lds[];
  const int S = max(1, GN_WAVES / groups);
  float* v = lds;
  float* unit_sums = lds + C;
  float* inv = unit_sums + groups * S;
  const int n = blockIdx.x;
  for (int i = threadIdx.x; i < C; i += GN_THREADS) {
    float o = in[(size_t)n * C + i];
    if (skip) o = fmaf(skip_w[i / skip_len], skip[(size_t)n * ld_skip + i], o);
    if (gate) {
      const float z = to_float(gate[(size_t)n * ld_gate + i]);
      o *= z / (1.0f + expf(-z));
    }
    v[i] = o;
  }
  __syncthreads();
  group_inverse_roots(v, C, groups, S, eps, unit_sums, inv);
  const int part = C / groups;
  for (int i = threadIdx.x; i < C; i += GN_THREADS) y[(size_t)n * C + i] = from_float<T>(v[i] * inv[i / part] * gain[i]);
}
}  // namespace

// x [N, H] float32.  delta (null: none): what is normed in `groups_d` parts, multiplied by gain_d and added into x.
// out (null: none): [n_out, H] in `dtype`, the norm of x (after the addition) in `groups_n` parts times gain_n, of
// all rows (rows null, n_out = N) or of the rows that `rows` names (then delta must be null).
GIBBS_EXPORT int gibbs_group_rmsnorm(float* x, const void* delta, int parts, long part_stride, const float* gain_d, float eps_d,
                                     int groups_d, const float* gain_n, float eps_n, int groups_n, void* out, int dtype,
                                     const int* rows, int n_out, int H, hipStream_t stream) {
  GIBBS_REQUIRE(x && n_out > 0 && H > 0 && (delta || out), "group_rmsnorm: bad operands rows=%d width=%d", n_out, H);
  GIBBS_REQUIRE(!delta || (gain_d && groups_d > 0 && H % groups_d == 0 && parts >= 1 && !rows), "group_rmsnorm: %d parts of a delta of width %d", groups_d, H);
  GIBBS_REQUIRE(!out || (gain_n && groups_n > 0 && H % groups_n == 0), "group_rmsnorm: %d parts of a row of width %d", groups_n, H);
  if (!delta) groups_d = 0;
  if (!out) groups_n = 0;
  const int Gmax = std::max(groups_d, groups_n);
  const int Sd = std::max(1, GN_WAVES / std::max(groups_d, 1)), Sn = std::max(1, GN_WAVES / std::max(groups_n, 1));
  const int units = std::max(Gmax, 1) * std::max(Sd, Sn);      // (the kernel lays its partial sums out for the larger of both)
  GIBBS_REQUIRE(units <= GN_MAX_UNITS, "group_rmsnorm: %d parts (at most %d)", Gmax, GN_MAX_UNITS / GN_WAVES);
  const size_t lds = ((size_t)H + units + std::max(Gmax, 1)) * sizeof(float);
  GIBBS_REQUIRE(lds <= 64 * 1024, "group_rmsnorm: rows of %d values do not fit a workgroup's memory", H);
  if (dtype == GIBBS_F32)
    group_norm_kernel<float><<<n_out, GN_THREADS, lds, stream>>>(x, delta, parts, (size_t)part_stride, gain_d, eps_d, std::max(groups_d, 1), gain_n, eps_n,
                                                                 std::max(groups_n, 1), (float*)out, rows, H);
  else if (dtype == GIBBS_BF16)
    group_norm_kernel<bf16><<<n_out, GN_THREADS, lds, stream>>>(x, delta, parts, (size_t)part_stride, gain_d, eps_d, std::max(groups_d, 1), gain_n, eps_n,
                                                                std::max(groups_n, 1), (bf16*)out, rows, H);
  else
    return gibbs_fail("group_rmsnorm: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("group_rmsnorm");
}

// y [N, C] (`dtype`) = norm in `groups` parts of (in + skip_w[c / skip_len] * skip) * silu(gate), times gain; in and skip
// are float32 (skip null: none; row stride ld_skip), gate is in `dtype` with row stride ld_gate (null: no gate).
GIBBS_EXPORT int gibbs_gated_group_norm(const float* in, const float* skip, long ld_skip, const float* skip_w, int skip_len,
                                        const void* gate, long ld_gate, const float* gain, float eps, int groups, void* y,
                                        int dtype, int n, int C, hipStream_t stream) {
  GIBBS_REQUIRE(in && gain && y && n > 0 && C > 0 && groups > 0 && C % groups == 0, "gated_group_norm: bad operands rows=%d width=%d parts=%d", n, C, groups);
  GIBBS_REQUIRE(!skip || (skip_w && skip_len > 0 && ld_skip >= C), "gated_group_norm: a skip path needs its weights");
  const int units = groups * std::max(1, GN_WAVES / groups);
  GIBBS_REQUIRE(units <= GN_MAX_UNITS, "gated_group_norm: %d parts (at most %d)", groups, GN_MAX_UNITS);
  const size_t lds = ((size_t)C + units + groups) * sizeof(float);
  GIBBS_REQUIRE(lds <= 64 * 1024, "gated_group_norm: rows of %d values do not fit a workgroup's memory", C);
  if (dtype == GIBBS_F32)
    gated_group_norm_kernel<float><<<n, GN_THREADS, lds, stream>>>(in, skip, ld_skip, skip_w, skip_len, (const float*)gate, ld_gate, gain, eps, groups, (float*)y, C);
  else if (dtype == GIBBS_BF16)
    gated_group_norm_kernel<bf16><<<n, GN_THREADS, lds, stream>>>(in, skip, ld_skip, skip_w, skip_len, (const bf16*)gate, ld_gate, gain, eps, groups, (bf16*)y, C);
  else
    return gibbs_fail("gated_group_norm: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("gated_group_norm");
}
