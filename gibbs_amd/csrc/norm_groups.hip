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
// ---- the same two kernels for rows of whole 4-value vectors that a workgroup's threads hold in registers (VPT vectors a
// thread): every global load of a row is asked for before the first one is waited for, so that a row costs one trip to
// memory instead of one per phase (steps of few rows are chains of such trips).  The sums are the generic kernels' sums.
__device__ __forceinline__ float4 ld4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 ld4(const bf16* p) {
  const uint2 raw = *(const uint2*)p;
  return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                     __uint_as_float(raw.y & 0xffff0000u));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void st4(bf16* p, float4 v) {
  union { bf16 h[4]; uint2 u; } o;
  o.h[0] = (bf16)v.x; o.h[1] = (bf16)v.y; o.h[2] = (bf16)v.z; o.h[3] = (bf16)v.w;
  *(uint2*)p = o.u;
}

template <typename T, int VPT>
__global__ __launch_bounds__(GN_THREADS) void group_norm_vec_kernel(float* __restrict__ x, const void* __restrict__ delta, int parts,
                                                                   size_t part_stride, const float* __restrict__ gain_d, float eps_d,
                                                                   int groups_d, const float* __restrict__ gain_n, float eps_n, int groups_n,
                                                                   T* __restrict__ out, const int* __restrict__ rows, int H) {
  extern __shared__ float lds[];
  const int Gmax = max(groups_d, groups_n);
  const int Sd = max(1, GN_WAVES / max(groups_d, 1)), Sn = max(1, GN_WAVES / max(groups_n, 1));
  float* v = lds;
  float* unit_sums = lds + H;
  float* inv = unit_sums + Gmax * max(Sd, Sn);
  const int n_out = blockIdx.x;
  const int n = rows ? rows[n_out] : n_out;
  float* xr = x + (size_t)n * H;
  float4 xv[VPT], dv[VPT], gd[VPT], gn[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = (threadIdx.x + j * GN_THREADS) * 4;
    const bool live = c < H;
    const int cc = live ? c : 0;
    xv[j] = ld4(xr + cc);
    gn[j] = out ? ld4(gain_n + cc) : make_float4(0.f, 0.f, 0.f, 0.f);
    dv[j] = gd[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (delta) {
      gd[j] = ld4(gain_d + cc);
      if (parts >= 2) {
        const float* d = (const float*)delta + (size_t)n * H + cc;
        float4 sum = ld4(d);
        for (int p = 1; p < parts; ++p) {
          const float4 a = ld4(d + (size_t)p * part_stride);
          sum.x += a.x; sum.y += a.y; sum.z += a.z; sum.w += a.w;
        }
        dv[j] = sum;
      } else {
        dv[j] = ld4((const T*)delta + (size_t)n * H + cc);
      }
    }
  }
  if (delta) {
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int c = (threadIdx.x + j * GN_THREADS) * 4;
      if (c < H) *(float4*)(v + c) = dv[j];
    }
    __syncthreads();
    group_inverse_roots(v, H, groups_d, Sd, eps_d, unit_sums, inv);
    const int part = H / groups_d;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int c = (threadIdx.x + j * GN_THREADS) * 4;
      if (c < H) {
        xv[j].x += dv[j].x * inv[c / part] * gd[j].x;
        xv[j].y += dv[j].y * inv[(c + 1) / part] * gd[j].y;
        xv[j].z += dv[j].z * inv[(c + 2) / part] * gd[j].z;
        xv[j].w += dv[j].w * inv[(c + 3) / part] * gd[j].w;
        st4(xr + c, xv[j]);
      }
    }
    __syncthreads();      // (everyone has read the delta's roots before they are overwritten)
  }
  if (!out) return;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = (threadIdx.x + j * GN_THREADS) * 4;
    if (c < H) *(float4*)(v + c) = xv[j];
  }
  __syncthreads();
  group_inverse_roots(v, H, groups_n, Sn, eps_n, unit_sums, inv);
  const int part = H / groups_n;
  T* o = out + (size_t)n_out * H;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = (threadIdx.x + j * GN_THREADS) * 4;
    if (c < H)
      st4(o + c, make_float4(xv[j].x * inv[c / part] * gn[j].x, xv[j].y * inv[(c + 1) / part] * gn[j].y, xv[j].z * inv[(c + 2) / part] * gn[j].z,
                             xv[j].w * inv[(c + 3) / part] * gn[j].w));
  }
}

template <typename T, int VPT>
__global__ __launch_bounds__(GN_THREADS) void gated_group_norm_vec_kernel(const float* __restrict__ in, const float* __restrict__ skip, long ld_skip,
                                                                         const float* __restrict__ skip_w, int skip_len,
                                                                         const T* __restrict__ gate, long ld_gate, const float* __restrict__ gain,
                                                                         float eps, int groups, T* __restrict__ y, int C) {
  extern __shared__ float lds[];
  const int S = max(1, GN_WAVES / groups);
  float* v = lds;
  float* unit_sums = lds + C;
  float* inv = unit_sums + groups * S;
  const int n = blockIdx.x;
  float4 ov[VPT], sv[VPT], gv[VPT], wv[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = (threadIdx.x + j * GN_THREADS) * 4;
    const int cc = c < C ? c : 0;
    ov[j] = ld4(in + (size_t)n * C + cc);
    wv[j] = ld4(gain + cc);
    sv[j] = skip ? ld4(skip + (size_t)n * ld_skip + cc) : make_float4(0.f, 0.f, 0.f, 0.f);
    gv[j] = gate ? ld4(gate + (size_t)n * ld_gate + cc) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  auto gated = [&](float o, float s, float z, int c) -> float {
    if (skip) o = fmaf(skip_w[c / skip_len], s, o);
    if (gate) o *= z / (1.0f + expf(-z));
    return o;
  };
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = (threadIdx.x + j * GN_THREADS) * 4;
    if (c < C) {
      ov[j] = make_float4(gated(ov[j].x, sv[j].x, gv[j].x, c), gated(ov[j].y, sv[j].y, gv[j].y, c + 1), gated(ov[j].z, sv[j].z, gv[j].z, c + 2),
                          gated(ov[j].w, sv[j].w, gv[j].w, c + 3));
      *(float4*)(v + c) = ov[j];
    }
  }
  __syncthreads();
  group_inverse_roots(v, C, groups, S, eps, unit_sums, inv);
  const int part = C / groups;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = (threadIdx.x + j * GN_THREADS) * 4;
    if (c < C)
      st4(y + (size_t)n * C + c, make_float4(ov[j].x * inv[c / part] * wv[j].x, ov[j].y * inv[(c + 1) / part] * wv[j].y,
                                             ov[j].z * inv[(c + 2) / part] * wv[j].z, ov[j].w * inv[(c + 3) / part] * wv[j].w));
  }
}

inline bool aligned_to(const void* p, size_t bytes) { return ((uintptr_t)p % bytes) == 0; }
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
  // rows of whole vectors that the threads hold in registers: the kernel that asks for everything at once
  const size_t esz = dtype == GIBBS_F32 ? 4 : 2;
  const bool vec = (dtype == GIBBS_F32 || dtype == GIBBS_BF16) && H % 4 == 0 && H <= 8 * GN_THREADS * 4 && aligned_to(x, 16) && aligned_to(gain_d, 16) &&
                   aligned_to(gain_n, 16) && aligned_to(out, 4 * esz) && aligned_to(delta, parts >= 2 ? 16 : 4 * esz) && (parts < 2 || part_stride % 4 == 0);
  if (vec) {
    const int vpt = H <= GN_THREADS * 4 ? 1 : (H <= 2 * GN_THREADS * 4 ? 2 : (H <= 4 * GN_THREADS * 4 ? 4 : 8));
#define GN_VEC(T, V) group_norm_vec_kernel<T, V><<<n_out, GN_THREADS, lds, stream>>>(x, delta, parts, (size_t)part_stride, gain_d, eps_d, std::max(groups_d, 1), \
                                                                                   gain_n, eps_n, std::max(groups_n, 1), (T*)out, rows, H)
#define GN_VEC_ANY(T) do { if (vpt == 1) GN_VEC(T, 1); else if (vpt == 2) GN_VEC(T, 2); else if (vpt == 4) GN_VEC(T, 4); else GN_VEC(T, 8); } while (0)
    if (dtype == GIBBS_F32) GN_VEC_ANY(float); else GN_VEC_ANY(bf16);
#undef GN_VEC_ANY
#undef GN_VEC
    GIBBS_LAUNCH_STATUS("group_rmsnorm");
  }
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
  const size_t esz = dtype == GIBBS_F32 ? 4 : 2;
  const bool vec = (dtype == GIBBS_F32 || dtype == GIBBS_BF16) && C % 4 == 0 && C <= 8 * GN_THREADS * 4 && aligned_to(in, 16) && aligned_to(gain, 16) &&
                   aligned_to(skip, 16) && ld_skip % 4 == 0 && aligned_to(gate, 4 * esz) && ld_gate % 4 == 0 && aligned_to(y, 4 * esz);
  if (vec) {
    const int vpt = C <= GN_THREADS * 4 ? 1 : (C <= 2 * GN_THREADS * 4 ? 2 : (C <= 4 * GN_THREADS * 4 ? 4 : 8));
#define GGN_VEC(T, V) gated_group_norm_vec_kernel<T, V><<<n, GN_THREADS, lds, stream>>>(in, skip, ld_skip, skip_w, skip_len, (const T*)gate, ld_gate, gain, eps, groups, (T*)y, C)
#define GGN_VEC_ANY(T) do { if (vpt == 1) GGN_VEC(T, 1); else if (vpt == 2) GGN_VEC(T, 2); else if (vpt == 4) GGN_VEC(T, 4); else GGN_VEC(T, 8); } while (0)
    if (dtype == GIBBS_F32) GGN_VEC_ANY(float); else GGN_VEC_ANY(bf16);
#undef GGN_VEC_ANY
#undef GGN_VEC
    GIBBS_LAUNCH_STATUS("gated_group_norm");
  }
  if (dtype == GIBBS_F32)
    gated_group_norm_kernel<float><<<n, GN_THREADS, lds, stream>>>(in, skip, ld_skip, skip_w, skip_len, (const float*)gate, ld_gate, gain, eps, groups, (float*)y, C);
  else if (dtype == GIBBS_BF16)
    gated_group_norm_kernel<bf16><<<n, GN_THREADS, lds, stream>>>(in, skip, ld_skip, skip_w, skip_len, (const bf16*)gate, ld_gate, gain, eps, groups, (bf16*)y, C);
  else
    return gibbs_fail("gated_group_norm: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("gated_group_norm");
}
