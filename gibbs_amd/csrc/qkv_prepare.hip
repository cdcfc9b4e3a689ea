// What an attention with projection biases, a rotation of part of each head, values of a head size of their own
// and value mixing does to a step's projected rows before the scores, in one pass:
//
//   q heads: + bias -> rotation of the first `rot` channels -> back in place
//   k heads: + bias -> the same rotation -> back in place and into page[table[req][pos / ps]][kv head][pos % ps]
//   v heads: + bias -> (value mixing) -> back in place and into their page
//
// Rows are [q: nh*hd | k: nkv*hd | v: nkv*vd]; `bias` (float32, the row's layout) may be null.  Rotation of pair
// (i0, i1) by angle = float(pos) * inv_freq[j] (a float32 product): half-split pairs (j, j + rot/2), interleaved
// pairs (2j, 2j+1); channels beyond `rot` pass.  Cosines and sines come from a table [positions, rot/2] of
// (cos, sin) where it reaches, else from the same functions that filled it.
//
// Value mixing: one layer of a model publishes its values of the step's rows (`keep` [N, nkv * vt], vt the true
// value size: heads may be stored wider, zeros behind their vt channels), and a later layer mixes them into its
// own before they are cached,  v <- (1 - lambda) v + lambda v_published,  lambda one number on the device.  The
// mix is float32 arithmetic (the layer's own value with its bias still unrounded), rounded once.
#include "common.h"
#include "lane8.h"

namespace {
enum { ROPE_HALF_SPLIT = 0, ROPE_INTERLEAVED = 1 };
enum { KEEP_NONE = 0, KEEP_PUBLISH = 1, KEEP_MIX = 2 };

struct QkvPrepareArgs {
  const float* bias;      // [nh*hd + nkv*hd + nkv*vd] or null
  const float* inv_freq;  // [rot / 2] or null: no rotation
  int rot, variant;
  const float2* cs_table;  // [table_len, rot / 2] or null
  int table_len;
  const float* lambda;     // the mixing weight (KEEP_MIX)
  int keep_mode, vt;       // vt: channels of a value head that are published or mixed
  const int* pos;
  const int* row_req;
  const int* table;
  int max_pages, page_size, num_pages;
  int nh, nkv, hd, vd;
  long ld;
};

template <typename T>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(T* __restrict__ rows, T* __restrict__ kpages, T* __restrict__ vpages,
                                                          T* __restrict__ keep, QkvPrepareArgs a) {
  const int n = blockIdx.x;
  const int hs = blockIdx.y * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (hs >= a.nh + 2 * a.nkv) return;
  const bool is_q = hs < a.nh, is_k = !is_q && hs < a.nh + a.nkv;
  const int g = is_q ? hs : (is_k ? hs - a.nh : hs - a.nh - a.nkv);
  const int size = (is_q || is_k) ? a.hd : a.vd;
  const long off = is_q ? (long)g * a.hd : (is_k ? (long)(a.nh + g) * a.hd : (long)(a.nh + a.nkv) * a.hd + (long)g * a.vd);
  T* src = rows + (size_t)n * a.ld + off;
  const float* bias = a.bias ? a.bias + off : nullptr;
  const int p = a.pos[n];
  T* page_dst = nullptr;
  if (!is_q && kpages) {
    const int page = a.table[(size_t)a.row_req[n] * a.max_pages + p / a.page_size];
    if (page >= 0 && page < a.num_pages)   // (the host never asks for another; never write outside the pool)
      page_dst = (is_k ? kpages : vpages) + (((size_t)page * a.nkv + g) * a.page_size + p % a.page_size) * size;
  }
  auto value = [&](int e) -> float { return bias ? to_float(src[e]) + bias[e] : to_float(src[e]); };
  auto put = [&](int e, float v) {
    const T r = from_float<T>(v);
    src[e] = r;
    if (page_dst) page_dst[e] = r;
  };
  if (!is_q && !is_k) {
    const float lam = a.keep_mode == KEEP_MIX ? *a.lambda : 0.f;
    T* kept = a.keep_mode != KEEP_NONE ? keep + ((size_t)n * a.nkv + g) * a.vt : nullptr;
    for (int e = lane; e < size; e += WAVE) {
      float v = value(e);
      if (a.keep_mode == KEEP_MIX && e < a.vt) v = (1.0f - lam) * v + lam * to_float(kept[e]);
      put(e, v);
      if (a.keep_mode == KEEP_PUBLISH && e < a.vt) kept[e] = from_float<T>(v);
    }
    return;
  }
  const int half = a.inv_freq ? a.rot / 2 : 0;
  // a lane reads both channels of its pairs before it writes either
  for (int j = lane; j < half; j += WAVE) {
    const int i0 = a.variant == ROPE_HALF_SPLIT ? j : 2 * j;
    const int i1 = a.variant == ROPE_HALF_SPLIT ? j + half : 2 * j + 1;
    const float x0 = value(i0), x1 = value(i1);
    float c, s;
    if (a.cs_table && p < a.table_len) {
      const float2 cs = a.cs_table[(size_t)p * half + j];
      c = cs.x;
      s = cs.y;
    } else {
      rope_cos_sin((float)p * a.inv_freq[j], &c, &s);
    }
    put(i0, x0 * c - x1 * s);
    put(i1, x1 * c + x0 * s);
  }
  for (int e = 2 * half + lane; e < size; e += WAVE) put(e, value(e));
}
}  // namespace

// keep_mode: 0 none, 1 the values are published into `keep`, 2 `keep` is mixed into the values with *lambda.
GIBBS_EXPORT int gibbs_qkv_prepare(void* rows, long ld, void* kpages, void* vpages, int dtype, const float* bias,
                                   const float* inv_freq, int rot, int variant, const float* cs_table, int table_len,
                                   void* keep, int keep_mode, int vt, const float* lambda, const int* pos, const int* row_req,
                                   const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh, int nkv,
                                   int hd, int vd, hipStream_t stream) {
  GIBBS_REQUIRE(rows && pos && n_rows > 0 && nh > 0 && nkv > 0 && hd > 0 && vd > 0, "qkv_prepare: bad operands rows=%d heads=%d kv=%d", n_rows, nh, nkv);
  GIBBS_REQUIRE(ld >= (long)(nh + nkv) * hd + (long)nkv * vd, "qkv_prepare: rows of %ld values cannot hold q, k and v", ld);
  GIBBS_REQUIRE(!kpages || (vpages && row_req && table && max_pages > 0 && page_size > 0 && num_pages > 0), "qkv_prepare: pages without their table");
  GIBBS_REQUIRE(!inv_freq || (rot > 0 && rot % 2 == 0 && rot <= hd), "qkv_prepare: %d rotated channels of a head of %d", rot, hd);
  GIBBS_REQUIRE(keep_mode == KEEP_NONE || (keep && vt > 0 && vt <= vd && (keep_mode == KEEP_PUBLISH || (keep_mode == KEEP_MIX && lambda))),
                "qkv_prepare: value mixing needs the published values and its weight");
  QkvPrepareArgs a{bias, inv_freq, inv_freq ? rot : 0, variant, (const float2*)cs_table, cs_table && inv_freq ? table_len : 0, lambda, keep_mode, vt,
                   pos, row_req, table, max_pages, page_size, num_pages, nh, nkv, hd, vd, ld};
  const int per_block = 4;
  const dim3 grid(n_rows, ceil_div(nh + 2 * nkv, per_block));
  if (dtype == GIBBS_F32)
    qkv_prepare_kernel<float><<<grid, per_block * WAVE, 0, stream>>>((float*)rows, (float*)kpages, (float*)vpages, (float*)keep, a);
  else if (dtype == GIBBS_BF16)
    qkv_prepare_kernel<bf16><<<grid, per_block * WAVE, 0, stream>>>((bf16*)rows, (bf16*)kpages, (bf16*)vpages, (bf16*)keep, a);
  else
    return gibbs_fail("qkv_prepare: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("qkv_prepare");
}
