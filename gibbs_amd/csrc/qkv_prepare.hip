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
//
// Further options (`gibbs_qkv_prepare_full`): q and k heads divided by their root mean square and multiplied by a gain
// [norm_dim] before the rotation (the mean over the first norm_dim channels of a head, which may be stored wider with
// zeros behind them); values that are the keys as projected (`v_from_k`: rows hold no values, the key's wave writes the
// unnormed, unrotated key into the value page); and values turned by their position over all of their first `v_rot`
// channels, pairs in the same layout, angle float(pos) * v_inv_freq[m], before they are cached.  `gibbs_attention_finish`
// is the other end of that: the heads' outputs turned back by the query's position and multiplied by sigmoid(gate).
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
  const float* q_gain;     // [norm_dim] or null: q heads are RMS-normed with this gain before the rotation
  const float* k_gain;     // the same for k heads
  float qk_eps;
  int norm_dim;            // channels of a head that the norm's mean runs over
  int v_from_k;            // the values are the keys as projected: rows are [q | k | ...], no value heads
  const float* v_inv_freq; // [v_rot / 2] or null: values are turned by their position over their first v_rot channels
  int v_rot;
};

// LPH lanes share a head (16 for heads of up to 128 channels: four heads a wave; else the whole wave).
template <typename T, int LPH>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(T* __restrict__ rows, T* __restrict__ kpages, T* __restrict__ vpages,
                                                          T* __restrict__ keep, QkvPrepareArgs a) {
  constexpr int WAVE = LPH;      // (below, "the wave" is the group of lanes that shares a head)
  const int n = blockIdx.x;
  const int hs = blockIdx.y * (blockDim.x / LPH) + threadIdx.x / LPH;
  const int lane = threadIdx.x % LPH;
  if (hs >= a.nh + (a.v_from_k ? 1 : 2) * a.nkv) return;
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
  auto raw_value = [&](int e) -> float { return bias ? to_float(src[e]) + bias[e] : to_float(src[e]); };
  auto put = [&](int e, float v) {
    const T r = from_float<T>(v);
    src[e] = r;
    if (page_dst) page_dst[e] = r;
  };
  if (is_k && a.v_from_k && vpages) {
    // the value of this position is the key as projected (vd channels of it), before norm and rotation
    const int page = a.table[(size_t)a.row_req[n] * a.max_pages + p / a.page_size];
    if (page >= 0 && page < a.num_pages) {
      T* vdst = vpages + (((size_t)page * a.nkv + g) * a.page_size + p % a.page_size) * a.vd;
      for (int e = lane; e < a.vd; e += WAVE) vdst[e] = from_float<T>(e < a.hd ? raw_value(e) : 0.f);
    }
  }
  if (!is_q && !is_k && a.v_inv_freq) {
    const int vh = a.v_rot / 2;
    for (int j = lane; j < vh; j += WAVE) {
      const int i0 = a.variant == ROPE_HALF_SPLIT ? j : 2 * j;
      const int i1 = a.variant == ROPE_HALF_SPLIT ? j + vh : 2 * j + 1;
      const float x0 = raw_value(i0), x1 = raw_value(i1);
      float c, s;
      rope_cos_sin((float)p * a.v_inv_freq[j], &c, &s);
      put(i0, x0 * c - x1 * s);
      put(i1, x1 * c + x0 * s);
    }
    for (int e = a.v_rot + lane; e < size; e += WAVE) put(e, raw_value(e));
    return;
  }
  // q and k heads: x / sqrt(mean(x^2) + eps) * gain over the head's first norm_dim channels, before the rotation
  const float* gain = is_q ? a.q_gain : (is_k ? a.k_gain : nullptr);
  float inv = 1.0f;
  if (gain) {
    float ss = 0.f;
    for (int e = lane; e < a.norm_dim; e += WAVE) { const float x = raw_value(e); ss = fmaf(x, x, ss); }
    inv = 1.0f / sqrtf((LPH == 64 ? wave_sum(ss) : group_sum<LPH>(ss)) / (float)a.norm_dim + a.qk_eps);
  }
  auto value = [&](int e) -> float { return gain ? (e < a.norm_dim ? raw_value(e) * inv * gain[e] : 0.f) : raw_value(e); };
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

// The same for bfloat16 rows whose sizes are multiples of 8 (heads, values, published values) and whose rotated part is
// a multiple of 16 in half-split pairs: a thread takes 8 neighbouring channels with 16-byte accesses, or, inside the rotated
// part, the 8 channels j .. j + 7 and their partners j + rot/2 ..; the threads are numbered over all (row, item) of the step,
// so that a wave is full whatever the head size.
__device__ __forceinline__ void unpack_bf16x8(const uint4& raw, float* f) { unpack8(raw, f); }
__device__ __forceinline__ uint4 pack_bf16x8(const float* f) {
  union { bf16 h[8]; uint4 u; } o;
#pragma unroll
  for (int i = 0; i < 8; ++i) o.h[i] = (bf16)f[i];
  return o.u;
}
__global__ __launch_bounds__(256) void qkv_prepare_bf16x8_kernel(bf16* __restrict__ rows, bf16* __restrict__ kpages, bf16* __restrict__ vpages,
                                                                 bf16* __restrict__ keep, QkvPrepareArgs a, int n_rows) {
  const int half = a.inv_freq ? a.rot / 2 : 0;
  const int per_qk = half / 8 + (a.hd - 2 * half) / 8, per_v = a.vd / 8;
  const int per_row = (a.nh + a.nkv) * per_qk + a.nkv * per_v;
  const unsigned item = blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= (unsigned)n_rows * (unsigned)per_row) return;
  const int n = (int)(item / (unsigned)per_row);
  int it = (int)(item % (unsigned)per_row);
  const int p = a.pos[n];
  bf16* row = rows + (size_t)n * a.ld;
  const bool is_v = it >= (a.nh + a.nkv) * per_qk;
  int head, sub;
  if (is_v) {
    it -= (a.nh + a.nkv) * per_qk;
    head = it / per_v;
    sub = it % per_v;
  } else {
    head = it / per_qk;
    sub = it % per_qk;
  }
  const bool is_q = !is_v && head < a.nh;
  const int g = is_v ? head : (is_q ? head : head - a.nh);
  const long off = is_v ? (long)(a.nh + a.nkv) * a.hd + (long)g * a.vd : (long)head * a.hd;
  const int size = is_v ? a.vd : a.hd;
  bf16* page_dst = nullptr;
  if (!is_q && kpages) {
    const int page = a.table[(size_t)a.row_req[n] * a.max_pages + p / a.page_size];
    if (page >= 0 && page < a.num_pages)
      page_dst = (is_v ? vpages : kpages) + (((size_t)page * a.nkv + g) * a.page_size + p % a.page_size) * size;
  }
  bf16* src = row + off;
  const float* bias = a.bias ? a.bias + off : nullptr;
  auto load = [&](int e0, float* f) {
    unpack_bf16x8(*(const uint4*)(src + e0), f);
    if (bias) {
      const float4 b0 = *(const float4*)(bias + e0), b1 = *(const float4*)(bias + e0 + 4);
      f[0] += b0.x; f[1] += b0.y; f[2] += b0.z; f[3] += b0.w; f[4] += b1.x; f[5] += b1.y; f[6] += b1.z; f[7] += b1.w;
    }
  };
  auto put = [&](int e0, const float* f) {
    const uint4 r = pack_bf16x8(f);
    *(uint4*)(src + e0) = r;
    if (page_dst) *(uint4*)(page_dst + e0) = r;
  };
  if (is_v) {
    const int e0 = sub * 8;
    float v[8];
    load(e0, v);
    if (a.keep_mode != KEEP_NONE && e0 < a.vt) {
      bf16* kept = keep + ((size_t)n * a.nkv + g) * a.vt + e0;
      if (a.keep_mode == KEEP_MIX) {
        const float lam = *a.lambda;
        float o[8];
        unpack_bf16x8(*(const uint4*)kept, o);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (1.0f - lam) * v[i] + lam * o[i];
      } else {
        *(uint4*)kept = pack_bf16x8(v);
      }
    }
    put(e0, v);
    return;
  }
  if (sub >= half / 8) {   // channels behind the rotated part pass
    const int e0 = 2 * half + (sub - half / 8) * 8;
    float v[8];
    load(e0, v);
    put(e0, v);
    return;
  }
  const int j0 = sub * 8;
  float x0[8], x1[8], y0[8], y1[8];
  load(j0, x0);
  load(j0 + half, x1);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float c, s;
    if (a.cs_table && p < a.table_len) {
      const float2 cs = a.cs_table[(size_t)p * half + j0 + i];
      c = cs.x;
      s = cs.y;
    } else {
      rope_cos_sin((float)p * a.inv_freq[j0 + i], &c, &s);
    }
    y0[i] = x0[i] * c - x1[i] * s;
    y1[i] = x1[i] * c + x0[i] * s;
  }
  put(j0, y0);
  put(j0 + half, y1);
}
// The heads' outputs att [N, nh * vd] (row stride ldo), in place: each head turned back by its row's position over its
// first v_rot channels (pair m by -pos * v_inv_freq[m]; null: not turned), then multiplied element by element with
// sigmoid(gate[n, h * gate_head + c]) (gate rows of stride ld_gate in the same type, c < vt; null: no gate).  float32 arithmetic.
template <typename T>
__global__ __launch_bounds__(256) void attention_finish_kernel(T* __restrict__ att, long ldo, const T* __restrict__ gate, long ld_gate,
                                                               int gate_head, const int* __restrict__ pos, const float* __restrict__ v_inv_freq,
                                                               int v_rot, int variant, int nh, int vd, int vt) {
  const int n = blockIdx.x;
  const int h = blockIdx.y * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (h >= nh) return;
  T* o = att + (size_t)n * ldo + (size_t)h * vd;
  const T* g = gate ? gate + (size_t)n * ld_gate + (size_t)h * gate_head : nullptr;
  auto gated = [&](int e, float v) -> float { return (g && e < vt) ? v / (1.0f + expf(-to_float(g[e]))) : v; };
  const int vh = v_inv_freq ? v_rot / 2 : 0;
  const float p = (float)pos[n];
  for (int j = lane; j < vh; j += WAVE) {
    const int i0 = variant == ROPE_HALF_SPLIT ? j : 2 * j;
    const int i1 = variant == ROPE_HALF_SPLIT ? j + vh : 2 * j + 1;
    const float x0 = to_float(o[i0]), x1 = to_float(o[i1]);
    float c, s;
    rope_cos_sin(p * v_inv_freq[j], &c, &s);
    o[i0] = from_float<T>(gated(i0, x0 * c + x1 * s));      // (the turn by -angle)
    o[i1] = from_float<T>(gated(i1, x1 * c - x0 * s));
  }
  if (g)
    for (int e = 2 * vh + lane; e < vd; e += WAVE) o[e] = from_float<T>(gated(e, to_float(o[e])));
}
}  // namespace

// keep_mode: 0 none, 1 the values are published into `keep`, 2 `keep` is mixed into the values with *lambda.
GIBBS_EXPORT int gibbs_qkv_prepare_full(void* rows, long ld, void* kpages, void* vpages, int dtype, const float* bias,
                                        const float* inv_freq, int rot, int variant, const float* cs_table, int table_len,
                                        void* keep, int keep_mode, int vt, const float* lambda, const int* pos, const int* row_req,
                                        const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh, int nkv,
                                        int hd, int vd, const float* q_gain, const float* k_gain, float qk_eps, int norm_dim,
                                        int v_from_k, const float* v_inv_freq, int v_rot, hipStream_t stream) {
  GIBBS_REQUIRE(rows && pos && n_rows > 0 && nh > 0 && nkv > 0 && hd > 0 && vd > 0, "qkv_prepare: bad operands rows=%d heads=%d kv=%d", n_rows, nh, nkv);
  GIBBS_REQUIRE(ld >= (long)(nh + nkv) * hd + (v_from_k ? 0 : (long)nkv * vd), "qkv_prepare: rows of %ld values cannot hold q, k and v", ld);
  GIBBS_REQUIRE(!kpages || (vpages && row_req && table && max_pages > 0 && page_size > 0 && num_pages > 0), "qkv_prepare: pages without their table");
  GIBBS_REQUIRE(!inv_freq || (rot > 0 && rot % 2 == 0 && rot <= hd), "qkv_prepare: %d rotated channels of a head of %d", rot, hd);
  GIBBS_REQUIRE(keep_mode == KEEP_NONE || (keep && vt > 0 && vt <= vd && (keep_mode == KEEP_PUBLISH || (keep_mode == KEEP_MIX && lambda))),
                "qkv_prepare: value mixing needs the published values and its weight");
  GIBBS_REQUIRE(!(q_gain || k_gain) || (norm_dim > 0 && norm_dim <= hd), "qkv_prepare: a norm over %d channels of a head of %d", norm_dim, hd);
  GIBBS_REQUIRE(!v_from_k || (keep_mode == KEEP_NONE && !v_inv_freq), "qkv_prepare: values that are the keys are neither mixed nor turned");
  GIBBS_REQUIRE(!v_inv_freq || (v_rot > 0 && v_rot % 2 == 0 && v_rot <= vd && keep_mode == KEEP_NONE), "qkv_prepare: %d turned channels of a value head of %d", v_rot, vd);
  QkvPrepareArgs a{bias, inv_freq, inv_freq ? rot : 0, variant, (const float2*)cs_table, cs_table && inv_freq ? table_len : 0, lambda, keep_mode, vt,
                   pos, row_req, table, max_pages, page_size, num_pages, nh, nkv, hd, vd, ld, q_gain, k_gain, qk_eps, norm_dim, v_from_k,
                   v_inv_freq, v_inv_freq ? v_rot : 0};
  const bool plain_options = !q_gain && !k_gain && !v_from_k && !v_inv_freq;
  const bool x8 = plain_options && dtype == GIBBS_BF16 && hd % 8 == 0 && vd % 8 == 0 && ld % 8 == 0 && ((uintptr_t)rows % 16) == 0 && (!inv_freq || (variant == ROPE_HALF_SPLIT && rot % 16 == 0)) &&
                  (!bias || ((uintptr_t)bias % 16) == 0) && (keep_mode == KEEP_NONE || (vt % 8 == 0 && ((uintptr_t)keep % 16) == 0)) &&
                  (!kpages || (((uintptr_t)kpages % 16) == 0 && ((uintptr_t)vpages % 16) == 0));
  if (x8) {
    const int half = a.rot / 2;
    const long items = (long)n_rows * ((long)(nh + nkv) * (half / 8 + (hd - 2 * half) / 8) + (long)nkv * (vd / 8));
    if (items < (1L << 31)) {
      qkv_prepare_bf16x8_kernel<<<ceil_div(items, 256), 256, 0, stream>>>((bf16*)rows, (bf16*)kpages, (bf16*)vpages, (bf16*)keep, a, n_rows);
      GIBBS_LAUNCH_STATUS("qkv_prepare");
    }
  }
  const bool narrow = hd <= 128 && vd <= 128;      // four heads a wave
  const int per_block = narrow ? 16 : 4;
  const dim3 grid(n_rows, ceil_div(nh + 2 * nkv, per_block));
  if (dtype == GIBBS_F32) {
    if (narrow) qkv_prepare_kernel<float, 16><<<grid, 256, 0, stream>>>((float*)rows, (float*)kpages, (float*)vpages, (float*)keep, a);
    else qkv_prepare_kernel<float, 64><<<grid, 256, 0, stream>>>((float*)rows, (float*)kpages, (float*)vpages, (float*)keep, a);
  } else if (dtype == GIBBS_BF16) {
    if (narrow) qkv_prepare_kernel<bf16, 16><<<grid, 256, 0, stream>>>((bf16*)rows, (bf16*)kpages, (bf16*)vpages, (bf16*)keep, a);
    else qkv_prepare_kernel<bf16, 64><<<grid, 256, 0, stream>>>((bf16*)rows, (bf16*)kpages, (bf16*)vpages, (bf16*)keep, a);
  } else
    return gibbs_fail("qkv_prepare: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("qkv_prepare");
}
GIBBS_EXPORT int gibbs_qkv_prepare(void* rows, long ld, void* kpages, void* vpages, int dtype, const float* bias,
                                   const float* inv_freq, int rot, int variant, const float* cs_table, int table_len,
                                   void* keep, int keep_mode, int vt, const float* lambda, const int* pos, const int* row_req,
                                   const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh, int nkv,
                                   int hd, int vd, hipStream_t stream) {
  return gibbs_qkv_prepare_full(rows, ld, kpages, vpages, dtype, bias, inv_freq, rot, variant, cs_table, table_len, keep, keep_mode, vt, lambda,
                                pos, row_req, table, max_pages, page_size, num_pages, n_rows, nh, nkv, hd, vd, nullptr, nullptr, 0.f, 0, 0,
                                nullptr, 0, stream);
}

GIBBS_EXPORT int gibbs_attention_finish(void* att, long ldo, const void* gate, long ld_gate, int gate_head, int dtype, const int* pos,
                                        const float* v_inv_freq, int v_rot, int variant, int n_rows, int nh, int vd, int vt,
                                        hipStream_t stream) {
  GIBBS_REQUIRE(att && n_rows > 0 && nh > 0 && vd > 0 && vt > 0 && vt <= vd && ldo >= (long)nh * vd, "attention_finish: bad operands rows=%d heads=%d vd=%d", n_rows, nh, vd);
  GIBBS_REQUIRE(!v_inv_freq || (pos && v_rot > 0 && v_rot % 2 == 0 && v_rot <= vd), "attention_finish: %d turned channels of a head of %d", v_rot, vd);
  GIBBS_REQUIRE(!gate || (gate_head >= vt && ld_gate >= (long)nh * gate_head), "attention_finish: gate rows too short");
  if (!gate && !v_inv_freq) return 0;
  const int per_block = 4;
  const dim3 grid(n_rows, ceil_div(nh, per_block));
  if (dtype == GIBBS_F32)
    attention_finish_kernel<float><<<grid, per_block * WAVE, 0, stream>>>((float*)att, ldo, (const float*)gate, ld_gate, gate_head, pos, v_inv_freq, v_rot, variant, nh, vd, vt);
  else if (dtype == GIBBS_BF16)
    attention_finish_kernel<bf16><<<grid, per_block * WAVE, 0, stream>>>((bf16*)att, ldo, (const bf16*)gate, ld_gate, gate_head, pos, v_inv_freq, v_rot, variant, nh, vd, vt);
  else
    return gibbs_fail("attention_finish: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("attention_finish");
}
