// Token embedding: x[n, :] = float(table[ids[n], :]) * scale (+ a sinusoidal position vector).  The
// residual stream is float32 whatever the table's type is.
//
// The position vector, when `inv_freq` [hidden / 2] is given: with a_i = p * inv_freq[i], even entries
// 2i take sin(a_i) and odd entries 2i + 1 take cos(a_i), a_i being the float32 product of the float32 position and the
// float32 frequency.  `keep` (optional) receives a second copy of the rows, for a model that adds the
// embedding's output into the stream again later.
#include "common.h"

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ x, bf16* __restrict__ mirror, int hidden, int vocab, float scale,
                             const int* __restrict__ pos, const float* __restrict__ inv_freq, float* __restrict__ keep) {
  const int n = blockIdx.x;
  int id = ids[n];
  // The host checks ids it uploads; a sampled id is < vocab by construction.  Clamp so that
  // a bad id can never read outside the table.
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (size_t)id * hidden;
  float* out = x + (size_t)n * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = to_float(row[i]) * scale;
    if (inv_freq && i / 2 < hidden / 2) {
      const float angle = (float)pos[n] * inv_freq[i / 2];
      v += (i & 1) ? cosf(angle) : sinf(angle);
    }
    out[i] = v;
    if (keep) keep[(size_t)n * hidden + i] = v;
    if (mirror) mirror[(size_t)n * hidden + i] = (bf16)v;
  }
}

// mirror (optional): the same rows rounded to bfloat16, [n, hidden].
GIBBS_EXPORT int gibbs_embed_general(const void* table, int dtype, const int* ids, float* x, void* mirror, int n, int hidden,
                                     int vocab, float scale, const int* pos, const float* inv_freq, float* keep,
                                     hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes n=%d hidden=%d vocab=%d", n, hidden, vocab);
  GIBBS_REQUIRE(!inv_freq || pos, "embed: a position vector needs the rows' positions");
  if (n == 0) return 0;
  const int threads = hidden >= 1024 ? 256 : 64;
  if (dtype == GIBBS_F32)
    embed_kernel<float><<<n, threads, 0, stream>>>((const float*)table, ids, x, (bf16*)mirror, hidden, vocab, scale, pos, inv_freq, keep);
  else if (dtype == GIBBS_BF16)
    embed_kernel<bf16><<<n, threads, 0, stream>>>((const bf16*)table, ids, x, (bf16*)mirror, hidden, vocab, scale, pos, inv_freq, keep);
  else
    return gibbs_fail("embed: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("embed");
}

GIBBS_EXPORT int gibbs_embed(const void* table, int dtype, const int* ids, float* x, void* mirror, int n,
                             int hidden, int vocab, hipStream_t stream) {
  return gibbs_embed_general(table, dtype, ids, x, mirror, n, hidden, vocab, 1.0f, nullptr, nullptr, nullptr, stream);
}

// The model's other end: logits capped in place, v <- cap * tanh(v / cap) (float32).
__global__ void softcap_kernel(float* __restrict__ v, long count, float cap) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) v[i] = cap * tanhf(v[i] / cap);
}
GIBBS_EXPORT int gibbs_softcap_rows(float* v, long count, float cap, hipStream_t stream) {
  GIBBS_REQUIRE(v && count >= 0 && cap > 0.f, "softcap: bad operands count=%ld cap=%g", count, cap);
  if (count == 0) return 0;
  softcap_kernel<<<ceil_div(count, 256), 256, 0, stream>>>(v, count, cap);
  GIBBS_LAUNCH_STATUS("softcap");
}
