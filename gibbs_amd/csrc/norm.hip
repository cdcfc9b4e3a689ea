// RMSNorm over rows of the float32 residual stream, fused with the residual add that
// precedes it:  v = x[r] (+ delta[r]);  (x[r] = v);  out[m] = v * rsqrt(mean(v^2) + eps) * gain.
// Sums, the root and the gain product are float32; the output takes the activation type.
// `rows` (optional) selects which rows are normed: out[m] comes from row rows[m].
#include "common.h"

template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                   const float* __restrict__ gain, float eps, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, int write_x) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int r = rows ? rows[m] : m;
  float* xr = x + (size_t)r * hidden;
  const T* dr = delta ? delta + (size_t)r * hidden : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = xr[i];
    if (dr) {
      v += to_float(dr[i]);
      if (write_x) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* o = out + (size_t)m * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = xr[i];
    if (dr && !write_x) v += to_float(dr[i]);
    o[i] = from_float<T>(gain ? v * scale * gain[i] : v * scale);
  }
}

// Four consecutive elements as one access.
__device__ __forceinline__ float4 load4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 load4(const bf16* p) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
  const bf16x4 v = *(const bf16x4*)p;
  return make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
}
__device__ __forceinline__ void store4(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
  *(bf16x4*)p = bf16x4{(bf16)v.x, (bf16)v.y, (bf16)v.z, (bf16)v.w};
}

// The same for hidden sizes in steps of 4 up to 4 * CHUNKS * blockDim: a thread keeps its elements in
// registers between the sum and the scaling (one pass over memory, 16-byte accesses of the stream).
template <typename T, int CHUNKS>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                       const float* __restrict__ gain, float eps, T* __restrict__ out,
                                       const int* __restrict__ rows, int hidden, int write_x) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int r = rows ? rows[m] : m;
  float* xr = x + (size_t)r * hidden;
  const T* dr = delta ? delta + (size_t)r * hidden : nullptr;
  float4 v[CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 4;
    v[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < hidden) {
      v[c] = *(const float4*)(xr + i);
      if (dr) {
        const float4 d = load4(dr + i);
        v[c].x += d.x; v[c].y += d.y; v[c].z += d.z; v[c].w += d.w;
        if (write_x) *(float4*)(xr + i) = v[c];
      }
      ss += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
    }
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* o = out + (size_t)m * hidden;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 4;
    if (i < hidden) {
      float4 g = make_float4(1.f, 1.f, 1.f, 1.f);
      if (gain) g = *(const float4*)(gain + i);
      store4(o + i, make_float4(v[c].x * scale * g.x, v[c].y * scale * g.y, v[c].z * scale * g.z, v[c].w * scale * g.w));
    }
  }
}

template <typename T>
bool launch_vec(float* x, const T* delta, const float* gain, float eps, T* out, const int* rows, int n_out, int hidden,
                int write_x, hipStream_t stream) {
  const uintptr_t vec = 4 * sizeof(T);
  if (hidden % 4 || ((uintptr_t)x % 16) || (gain && ((uintptr_t)gain % 16)) || ((uintptr_t)out % vec) ||
      (delta && ((uintptr_t)delta % vec)))
    return false;
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  const int chunks = ceil_div(hidden, 4 * threads);
  if (chunks == 1) add_rmsnorm_vec_kernel<T, 1><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else if (chunks == 2) add_rmsnorm_vec_kernel<T, 2><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else if (chunks <= 4) add_rmsnorm_vec_kernel<T, 4><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else if (chunks <= 8) add_rmsnorm_vec_kernel<T, 8><<<n_out, threads, 0, stream>>>(x, delta, gain, eps, out, rows, hidden, write_x);
  else return false;
  return true;
}

// x: [n_x, hidden] float32 residual stream (updated in place when delta is given and rows is null);
// out: [n_out, hidden]; rows: n_out row indices into x, or null with n_out == n_x.
GIBBS_EXPORT int gibbs_add_rmsnorm(float* x, const void* delta, const float* gain, float eps, void* out,
                                   int dtype, const int* rows, int n_out, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(n_out >= 0 && hidden > 0, "rmsnorm: bad sizes n=%d hidden=%d", n_out, hidden);
  if (n_out == 0) return 0;
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  const int write_x = rows == nullptr;
  if (dtype == GIBBS_F32) {
    if (!launch_vec<float>(x, (const float*)delta, gain, eps, (float*)out, rows, n_out, hidden, write_x, stream))
      add_rmsnorm_kernel<float><<<n_out, threads, 0, stream>>>(x, (const float*)delta, gain, eps, (float*)out, rows, hidden, write_x);
  } else if (dtype == GIBBS_BF16) {
    if (!launch_vec<bf16>(x, (const bf16*)delta, gain, eps, (bf16*)out, rows, n_out, hidden, write_x, stream))
      add_rmsnorm_kernel<bf16><<<n_out, threads, 0, stream>>>(x, (const bf16*)delta, gain, eps, (bf16*)out, rows, hidden, write_x);
  } else {
    return gibbs_fail("rmsnorm: unknown dtype %d", dtype);
  }
  GIBBS_LAUNCH_STATUS("rmsnorm");
}

// The same with the delta given as float32 partial sums of a product split over k:
// delta[r] = sum_s partials[s][r], added in ascending s.
template <typename T>
__global__ void add_partials_rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ partials, int n_partials,
                                            long partial_stride, const float* __restrict__ gain, float eps,
                                            T* __restrict__ out, const int* __restrict__ rows, int hidden,
                                            int write_x) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int r = rows ? rows[m] : m;
  float* xr = x + (size_t)r * hidden;
  const float* pr = partials + (size_t)r * hidden;
  T* o = out + (size_t)m * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float d = 0.f;
    for (int s = 0; s < n_partials; ++s) d += pr[(size_t)s * partial_stride + i];
    const float v = xr[i] + d;
    if (write_x) xr[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = xr[i];
    if (!write_x) {
      float d = 0.f;
      for (int s = 0; s < n_partials; ++s) d += pr[(size_t)s * partial_stride + i];
      v += d;
    }
    o[i] = from_float<T>(gain ? v * scale * gain[i] : v * scale);
  }
}

// partials: [n_partials, n_x, hidden] float32 (stride between partials given in elements).
GIBBS_EXPORT int gibbs_add_partials_rmsnorm(float* x, const float* partials, int n_partials, long partial_stride,
                                            const float* gain, float eps, void* out, int dtype, const int* rows,
                                            int n_out, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(n_out >= 0 && hidden > 0 && n_partials >= 1, "rmsnorm: bad sizes n=%d hidden=%d partials=%d", n_out, hidden, n_partials);
  if (n_out == 0) return 0;
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  const int write_x = rows == nullptr;
  if (dtype == GIBBS_F32)
    add_partials_rmsnorm_kernel<float><<<n_out, threads, 0, stream>>>(x, partials, n_partials, partial_stride, gain, eps, (float*)out, rows, hidden, write_x);
  else if (dtype == GIBBS_BF16)
    add_partials_rmsnorm_kernel<bf16><<<n_out, threads, 0, stream>>>(x, partials, n_partials, partial_stride, gain, eps, (bf16*)out, rows, hidden, write_x);
  else
    return gibbs_fail("rmsnorm: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("rmsnorm");
}

// x[r] += delta[r] alone (the last residual add of a model whose tail norms only some rows
// still has to leave x whole for callers that read it).  float32 delta may be `n_partials` partial
// sums, `partial_stride` elements apart, added in ascending order.
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ delta, int n_partials,
                                    size_t partial_stride, bf16* __restrict__ mirror, size_t count) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) {
    float v = x[i];
    if (delta)
      for (int s = 0; s < n_partials; ++s) v += to_float(delta[s * partial_stride + i]);
    x[i] = v;
    if (mirror) mirror[i] = (bf16)v;
  }
}

// x += delta (delta may be null); mirror (optional) = bfloat16(x).
GIBBS_EXPORT int gibbs_residual_add(float* x, const void* delta, int dtype, int n_partials, long partial_stride,
                                    void* mirror, long count, hipStream_t stream) {
  GIBBS_REQUIRE(count >= 0 && n_partials >= 1 && (n_partials == 1 || (dtype == GIBBS_F32 && partial_stride >= count)),
                "residual_add: bad count %ld or partial sums (%d, stride %ld)", count, n_partials, partial_stride);
  if (count == 0) return 0;
  const int blocks = ceil_div(count, 256);
  if (dtype == GIBBS_F32)
    residual_add_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)delta, n_partials, (size_t)partial_stride, (bf16*)mirror, (size_t)count);
  else if (dtype == GIBBS_BF16)
    residual_add_kernel<bf16><<<blocks, 256, 0, stream>>>(x, (const bf16*)delta, 1, 0, (bf16*)mirror, (size_t)count);
  else
    return gibbs_fail("residual_add: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("residual_add");
}

// RMSNorm of rows that are not the residual stream (a part's result, normed before it is added):
// v = sum of the `parts` partial sums of the row (one, in the activation type, or several in float32);
// out = v * rsqrt(mean(v^2) + eps) * gain, in the activation type.
template <typename T>
__global__ void rmsnorm_rows_kernel(const void* __restrict__ in, int parts, size_t part_stride, const float* __restrict__ gain,
                                    float eps, T* __restrict__ out, int hidden) {
  __shared__ float scratch[16];
  const size_t at = (size_t)blockIdx.x * hidden;
  auto value = [&](int i) -> float {
    if (parts == 1) return to_float(((const T*)in)[at + i]);
    float v = 0.f;
    for (int s = 0; s < parts; ++s) v += ((const float*)in)[s * part_stride + at + i];
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = value(i);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[at + i] = from_float<T>(gain ? value(i) * scale * gain[i] : value(i) * scale);
}

// The same added straight into the float32 stream: x += v * rsqrt(mean(v^2) + eps) * gain (no rounding of the normed rows).
template <typename T>
__global__ void rmsnorm_rows_add_kernel(float* __restrict__ x, const void* __restrict__ in, int parts, size_t part_stride,
                                        const float* __restrict__ gain, float eps, int hidden) {
  __shared__ float scratch[16];
  const size_t at = (size_t)blockIdx.x * hidden;
  auto value = [&](int i) -> float {
    if (parts == 1) return to_float(((const T*)in)[at + i]);
    float v = 0.f;
    for (int s = 0; s < parts; ++s) v += ((const float*)in)[s * part_stride + at + i];
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = value(i);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) x[at + i] += gain ? value(i) * scale * gain[i] : value(i) * scale;
}

// A sublayer's boundary in one pass: x += v * rsqrt(mean(v^2) + eps_d) * gain_d, v the sum of the `parts` partial sums of a
// part's result (one, in the activation type, or several in float32); and, with `out`, out = x * rsqrt(mean(x^2) + eps_n) *
// gain_n of the new x (the next sublayer's norm).  A thread keeps its elements of the row in registers between the sums and
// the scalings: 16-byte accesses, hidden sizes in steps of 4 up to 4 * CHUNKS * blockDim.  Sums, roots and x are float32.
// MIX: the part's result is itself a weighted sum that no kernel has written yet (a mixture of experts' combination):
// v = sum_s weight[n][s] * in[place[n][s]] (ascending s, rows of `in` in the activation type) + gate[n] * shared[n]
// (shared null: none; gate null: 1), float32 throughout.
struct RowMix {
  const int* place;       // [n, top]
  const float* weight;    // [n, top]
  const void* shared;     // [n, hidden] or null
  const float* gate;      // [n] or null
  int top;
};
template <typename T, int CHUNKS, bool MIX>
__global__ void rows_add_norm_vec_kernel(float* __restrict__ x, const void* __restrict__ in, int parts, size_t part_stride,
                                         const float* __restrict__ gain_d, float eps_d, const float* __restrict__ gain_n, float eps_n,
                                         T* __restrict__ out, int hidden, RowMix mix) {
  __shared__ float scratch[16];
  const size_t at = (size_t)blockIdx.x * hidden;
  float4 v[CHUNKS], xv[CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 4;
    v[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < hidden) {
      xv[c] = *(const float4*)(x + at + i);
      if (MIX) {
        const size_t first = (size_t)blockIdx.x * mix.top;
        for (int s = 0; s < mix.top; ++s) {
          const float w = mix.weight[first + s];
          const float4 r = load4((const T*)in + (size_t)mix.place[first + s] * hidden + i);
          v[c].x = fmaf(w, r.x, v[c].x); v[c].y = fmaf(w, r.y, v[c].y); v[c].z = fmaf(w, r.z, v[c].z); v[c].w = fmaf(w, r.w, v[c].w);
        }
        if (mix.shared) {
          const float g = mix.gate ? mix.gate[blockIdx.x] : 1.0f;
          const float4 r = load4((const T*)mix.shared + at + i);
          v[c].x = fmaf(g, r.x, v[c].x); v[c].y = fmaf(g, r.y, v[c].y); v[c].z = fmaf(g, r.z, v[c].z); v[c].w = fmaf(g, r.w, v[c].w);
        }
      } else if (parts == 1) {
        v[c] = load4((const T*)in + at + i);
      } else {
        for (int s = 0; s < parts; ++s) {
          const float4 d = *(const float4*)((const float*)in + s * part_stride + at + i);
          v[c].x += d.x; v[c].y += d.y; v[c].z += d.z; v[c].w += d.w;
        }
      }
      ss += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
    }
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)hidden + eps_d);
  float sx = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 4;
    if (i < hidden) {
      float4 g = make_float4(1.f, 1.f, 1.f, 1.f);
      if (gain_d) g = *(const float4*)(gain_d + i);
      xv[c].x += v[c].x * scale * g.x; xv[c].y += v[c].y * scale * g.y; xv[c].z += v[c].z * scale * g.z; xv[c].w += v[c].w * scale * g.w;
      *(float4*)(x + at + i) = xv[c];
      sx += xv[c].x * xv[c].x + xv[c].y * xv[c].y + xv[c].z * xv[c].z + xv[c].w * xv[c].w;
    }
  }
  if (!out) return;
  sx = block_sum(sx, scratch);
  const float scale_n = 1.0f / sqrtf(sx / (float)hidden + eps_n);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 4;
    if (i < hidden) {
      float4 g = make_float4(1.f, 1.f, 1.f, 1.f);
      if (gain_n) g = *(const float4*)(gain_n + i);
      store4(out + at + i, make_float4(xv[c].x * scale_n * g.x, xv[c].y * scale_n * g.y, xv[c].z * scale_n * g.z, xv[c].w * scale_n * g.w));
    }
  }
}

template <typename T>
bool launch_rows_add_norm(float* x, const void* in, int parts, long part_stride, const float* gain_d, float eps_d, const float* gain_n,
                          float eps_n, T* out, int n, int hidden, hipStream_t stream, const RowMix* mixed = nullptr) {
  const uintptr_t vec = parts == 1 ? 4 * sizeof(T) : 16;
  if (hidden % 4 || ((uintptr_t)x % 16) || ((uintptr_t)in % vec) || (parts > 1 && part_stride % 4) || (gain_d && ((uintptr_t)gain_d % 16)) ||
      (gain_n && ((uintptr_t)gain_n % 16)) || (out && ((uintptr_t)out % (4 * sizeof(T)))) ||
      (mixed && (parts != 1 || ((uintptr_t)mixed->shared % (4 * sizeof(T))))))
    return false;
  // (few rows: wide workgroups, every load of the row in flight at once)
  const int threads = hidden >= 4096 ? 1024 : (hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64));
  const int chunks = ceil_div(hidden, 4 * threads);
#define GIBBS_ROWS_ADD_NORM(C)                                                                                                              \
  do {                                                                                                                                      \
    if (mixed) rows_add_norm_vec_kernel<T, C, true><<<n, threads, 0, stream>>>(x, in, parts, (size_t)part_stride, gain_d, eps_d, gain_n, eps_n, out, hidden, *mixed); \
    else rows_add_norm_vec_kernel<T, C, false><<<n, threads, 0, stream>>>(x, in, parts, (size_t)part_stride, gain_d, eps_d, gain_n, eps_n, out, hidden, RowMix{}); \
  } while (0)
  if (chunks == 1) GIBBS_ROWS_ADD_NORM(1);
  else if (chunks == 2) GIBBS_ROWS_ADD_NORM(2);
  else if (chunks <= 4) GIBBS_ROWS_ADD_NORM(4);
  else return false;
#undef GIBBS_ROWS_ADD_NORM
  return true;
}

// x += norm(in) (gain_d, eps_d) and out = norm(x) (gain_n, eps_n) of all n rows in one kernel.  Returns 0 when it was queued,
// -1 when the sizes or addresses do not allow it (nothing was queued: the caller runs the two passes), 1 on an error.
GIBBS_EXPORT int gibbs_rmsnorm_rows_add_norm(float* x, const void* in, int parts, long part_stride, const float* gain_d, float eps_d,
                                             const float* gain_n, float eps_n, void* out, int dtype, int n, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(x && in && out && n >= 0 && hidden > 0 && parts >= 1, "rmsnorm_rows_add_norm: bad sizes n=%d hidden=%d parts=%d", n, hidden, parts);
  if (n == 0) return 0;
  bool queued;
  if (dtype == GIBBS_F32) queued = launch_rows_add_norm<float>(x, in, parts, part_stride, gain_d, eps_d, gain_n, eps_n, (float*)out, n, hidden, stream);
  else if (dtype == GIBBS_BF16) queued = launch_rows_add_norm<bf16>(x, in, parts, part_stride, gain_d, eps_d, gain_n, eps_n, (bf16*)out, n, hidden, stream);
  else return gibbs_fail("rmsnorm_rows_add_norm: unknown dtype %d", dtype);
  if (!queued) return -1;
  GIBBS_LAUNCH_STATUS("rmsnorm_rows_add_norm");
}

// The same with the part's result still to be summed: in [places, hidden] holds the results of a row's `top` choices at
// place[n][s], v = sum_s weight[n][s] in[place[n][s]] + gate[n] shared[n] (a mixture of experts' combination, float32).
GIBBS_EXPORT int gibbs_rmsnorm_rows_mix_add_norm(float* x, const void* in, const int* place, const float* weight, int top, const void* shared,
                                                 const float* gate, const float* gain_d, float eps_d, const float* gain_n, float eps_n,
                                                 void* out, int dtype, int n, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(x && in && place && weight && out && n >= 0 && hidden > 0 && top >= 1, "rmsnorm_rows_mix_add_norm: bad sizes n=%d hidden=%d top=%d", n, hidden, top);
  if (n == 0) return 0;
  const RowMix mixed{place, weight, shared, gate, top};
  bool queued;
  if (dtype == GIBBS_F32) queued = launch_rows_add_norm<float>(x, in, 1, 0, gain_d, eps_d, gain_n, eps_n, (float*)out, n, hidden, stream, &mixed);
  else if (dtype == GIBBS_BF16) queued = launch_rows_add_norm<bf16>(x, in, 1, 0, gain_d, eps_d, gain_n, eps_n, (bf16*)out, n, hidden, stream, &mixed);
  else return gibbs_fail("rmsnorm_rows_mix_add_norm: unknown dtype %d", dtype);
  if (!queued) return -1;
  GIBBS_LAUNCH_STATUS("rmsnorm_rows_mix_add_norm");
}

GIBBS_EXPORT int gibbs_rmsnorm_rows_add(float* x, const void* in, int parts, long part_stride, const float* gain, float eps, int dtype,
                                        int n, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(x && in && n >= 0 && hidden > 0 && parts >= 1, "rmsnorm_rows_add: bad sizes n=%d hidden=%d parts=%d", n, hidden, parts);
  if (n == 0) return 0;
  if ((dtype == GIBBS_F32 && launch_rows_add_norm<float>(x, in, parts, part_stride, gain, eps, nullptr, 0.f, nullptr, n, hidden, stream)) ||
      (dtype == GIBBS_BF16 && launch_rows_add_norm<bf16>(x, in, parts, part_stride, gain, eps, nullptr, 0.f, nullptr, n, hidden, stream)))
    GIBBS_LAUNCH_STATUS("rmsnorm_rows_add");
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  if (dtype == GIBBS_F32)
    rmsnorm_rows_add_kernel<float><<<n, threads, 0, stream>>>(x, in, parts, (size_t)part_stride, gain, eps, hidden);
  else if (dtype == GIBBS_BF16)
    rmsnorm_rows_add_kernel<bf16><<<n, threads, 0, stream>>>(x, in, parts, (size_t)part_stride, gain, eps, hidden);
  else
    return gibbs_fail("rmsnorm_rows_add: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("rmsnorm_rows_add");
}

GIBBS_EXPORT int gibbs_rmsnorm_rows(const void* in, int parts, long part_stride, const float* gain, float eps, void* out, int dtype,
                                    int n, int hidden, hipStream_t stream) {
  GIBBS_REQUIRE(in && out && n >= 0 && hidden > 0 && parts >= 1, "rmsnorm_rows: bad sizes n=%d hidden=%d parts=%d", n, hidden, parts);
  if (n == 0) return 0;
  const int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
  if (dtype == GIBBS_F32)
    rmsnorm_rows_kernel<float><<<n, threads, 0, stream>>>(in, parts, (size_t)part_stride, gain, eps, (float*)out, hidden);
  else if (dtype == GIBBS_BF16)
    rmsnorm_rows_kernel<bf16><<<n, threads, 0, stream>>>(in, parts, (size_t)part_stride, gain, eps, (bf16*)out, hidden);
  else
    return gibbs_fail("rmsnorm_rows: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("rmsnorm_rows");
}
