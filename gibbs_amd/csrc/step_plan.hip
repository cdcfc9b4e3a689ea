// The step of a whole model as one native call.
//
// When a model is bound, its parts are laid down in a plan (step_plan_api.h): norms and bodies (what reads
// normed rows and gives a delta for the residual stream: a mixer or a feed-forward), and a program of
// operations over them that says how every layer arranges its parts.  gibbs_plan_step then runs one ragged
// batch through embedding, the program, the final norm of the wanted rows and the head, choosing for each
// operation the kernel that the step's shape asks for (the few-row weight-streaming products and their
// fused epilogues for steps of decoded tokens, the library's or the tiled product above that, the
// matrix-core attention for prompt portions, the key-splitting one for decoded tokens, the plain kernels
// for float32 and odd sizes) and queueing everything on the caller's stream.  The host does no work per
// kernel beyond this function: a step of a hundred kernels costs it a few tens of microseconds, where a
// launch from an interpreter costs that much for every few kernels.  The reference's step is one native
// call as well (src/model/native.rs:78-83).
//
// This file is the one place where those choices are made.  A caller that runs a kernel by itself asks
// here (gibbs_rule_*, gibbs_linear, gibbs_skinny_residual_routed), and a part run alone (gibbs_plan_body_forward)
// goes through the code that a whole step goes through.
//
// The program is open: the parts that the library brings (RMS norm, gated short convolution, attention
// over the paged cache, gated dense feed-forward) sit beside parts from anywhere else, which are a
// function pointer and a user pointer each; and the arrangement x += mixer(norm(x)); x += ffn(norm(x)) is
// two "half" operations where another arrangement writes norm, body, add and drop operations in its own
// order.  Only a half can take the fused decode kernels (norm, part and residual add in two or three
// kernels), when its norm's gain is folded into the part's matrices and the part has such kernels.
//
// Activations live in a workspace that the caller passes: the same function run "dry" (nothing queued)
// reports the bytes a step needs, so the caller can size the workspace before the real run.  Buffers are
// taken and given back in the order of the code below; kernels run in stream order, so a buffer that
// was given back can be handed out again at once.
#include "common.h"
#include "step_plan_api.h"
#include <map>
#include <memory>
#include <vector>

namespace {
struct Matrix {
  const void* w = nullptr;       // [O, I] row-major in the run's compute type
  const void* packed = nullptr;  // the same in tile order (bfloat16 only), or null
  int O = 0, I = 0;
};

long ceil_div_l(long a, long b) { return (a + b - 1) / b; }

// ------------------------------------------------------------------------------------------------- rules
constexpr int FUSED_ROWS = 64;            // rows that the few-row products (and so the fused decode kernels) take
constexpr int SKINNY_ROWS = 64;           // rows up to which a plain product takes the weight-streaming kernel
constexpr int SKINNY_ROWS_F32_OUT = 48;   // the same for float32 output (the head: it streams faster than the tiled product)
constexpr int ACT_CLAMPED = 4;            // the gated feed-forward's clamped activation (activation.h: ACT_CLAMPED_SWISH)
constexpr int SSD_CHUNKED_ROWS = 256;     // rows of one request from which the state-space rule runs in chunks
constexpr int MATRIX_SLICE_PAGES = 510;   // page ids of a key slice that the decode attention's matrix-core walk keeps in LDS

// Ranges of k that the few-row product is cut into so that at least `want_blocks` workgroups run (a
// workgroup owns `features` output features), each with at least `min_k` of k.
int skinny_splits(int n_out, int inner, int want_blocks = 512, int features = 16, int min_k = 1024) {
  const long blocks = ceil_div_l(n_out, features);
  const long s = std::max<long>(1, std::min<long>(ceil_div_l(want_blocks, blocks), inner / min_k));
  const long per = ceil_div_l(ceil_div_l(inner, s), 128) * 128;
  return (int)ceil_div_l(inner, per);
}

// (key slices per (row, kv head), waves per workgroup) of the decode attention.  Few rows: enough slices to
// give each of the 256 compute units two workgroups of 4 waves, but at least 64 keys to a slice (256 on the
// matrix cores: two tiles of 32 for every wave, and few enough slices for the merge to take them at once).
// Rows and heads that fill the chip by themselves: no slices (a slice costs every wave its own prologue and
// final fold), 8 waves on the vector units, 4 on the matrix cores (measured at batch 1 to 64, 2,048 to 8,192
// keys).  The matrix-core walk keeps the page ids of a whole slice in LDS: caches longer than that are cut
// into as many slices as it takes.  kind: 0 the kernel's choice of walk, 1 vector units, 2 matrix cores.
void decode_splits(int n_rows, int nkv, int group, int max_seq, int hd, int page_size, int kind, int* n_splits, int* waves) {
  kind &= 3;   // (+ 4 only says which kernel merges the slices)
  const bool matrix = kind != 1 && hd > 0 && hd % 16 == 0 && hd <= 128;
  const int gt = group >= 8 ? 8 : (group > 2 ? 4 : group);
  const long per_split = std::max<long>(1, (long)n_rows * nkv * ceil_div_l(group, gt));
  const long least = matrix ? std::max<long>(1, ceil_div_l(max_seq, (long)MATRIX_SLICE_PAGES * page_size - 256)) : 1;
  if (per_split >= 256) {
    *n_splits = (int)least;
    *waves = matrix ? 4 : 8;
    return;
  }
  const long want = ceil_div_l(512, per_split);
  *n_splits = (int)std::max<long>(least, std::min<long>(std::min<long>(want, max_seq / (matrix ? 256 : 64)), 256));
  *waves = 4;
}

// Query tiles of 64 rows that a ragged batch makes (requests' rows do not share tiles).
long prefill_tiles(int rows, int reqs) { return ceil_div_l(rows, 64) + reqs / 2; }
// Slices of the key tiles for the prompt attention: none while the query tiles and heads fill the chip by
// themselves (about three workgroups per compute unit); else enough for eight workgroups per compute unit,
// with at least four tiles of 64 keys to a slice (measured: 512 rows over 7,680 cached keys take 203 us
// whole, 113 us in 4 slices, 94 us in 8).
int prefill_splits(long n_tiles, int nh, int max_seq, int window) {
  const long blocks = std::max<long>(1, n_tiles * nh);
  const long keys = window > 0 ? std::min<long>(max_seq, window + 64) : max_seq;
  if (blocks >= 768 || keys < 8 * 64) return 1;
  return (int)std::max<long>(1, std::min<long>(std::min<long>(ceil_div_l(2048, blocks), keys / 256), 16));
}

// Query heads of a kv head's group that a workgroup of the prompt attention takes (they share its K and V
// tiles).  With one head a workgroup re-reads all keys and values of its rows' past for 64 x 64 scores at a
// time, and from about 4,000 keys a row that traffic, not the arithmetic, bounds the kernel (537 TFLOP/s at
// 8.4 TB/s through L2 and the L1s); more heads a workgroup are fewer, longer workgroups.  Measured at 32 heads
// in groups of 4, head size 64 (us, with 1 / 2 / 4 heads): 2,048 rows 68 / 63 / 63; 4,096 rows 196 / 209 / 203;
// 8,192 rows 577 / 562 / 584; 32,768 rows 8,086 / 7,147 / 6,626; 2,048 rows behind 6,144 keys 281 / 220 / 205;
// 512 rows behind 7,680 keys in 8 slices 80 / 84 / 92.
int prefill_heads(int rows, int reqs, int nh, int nkv, int hd, int max_seq, int n_splits) {
  const int group = nh / std::max(nkv, 1);
  if (hd > 64 || group % 2 || n_splits > 1) return 1;
  const long seen = (long)max_seq - rows / (2 * std::max(reqs, 1));   // keys a row sees on average, if one request has them all
  return (group % 4 == 0 && seen >= 6000) ? 4 : 2;
}

// Which product runs y = x W^T, and in how many float32 partial sums it leaves its result.
enum { LIN_F32, LIN_PLAIN, LIN_SKINNY, LIN_LIBRARY, LIN_TILED };
struct LinearChoice {
  int kernel, splits;
};
LinearChoice choose_linear(bool bf16_run, int n, int O, int I, bool aligned, bool out_f32, bool partial_ok, bool own_gemm) {
  if (!bf16_run) return {LIN_F32, 1};                    // the true 32-bit product, plain FMA in ascending k
  if (!aligned) return {LIN_PLAIN, 1};                   // what the matrix-core kernels refuse
  if (n <= (out_f32 && !partial_ok ? SKINNY_ROWS_F32_OUT : SKINNY_ROWS)) return {LIN_SKINNY, partial_ok ? skinny_splits(O, I) : 1};
  if (!own_gemm && !out_f32 && O % 8 == 0) return {LIN_LIBRARY, 1};    // (the library writes bfloat16 only, in rows of whole 16 bytes)
  return {LIN_TILED, 1};
}
bool aligned_for_matrix_cores(const void* x, long ldx, const void* w, int I) {
  return I % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
}
int run_linear(LinearChoice c, const void* x, long ldx, const Matrix& m, bool use_packed, void* y, int n, bool out_f32,
               hipStream_t stream) {
  const int O = m.O, I = m.I, out_dtype = out_f32 ? GIBBS_F32 : GIBBS_BF16;
  switch (c.kernel) {
    case LIN_F32: return gibbs_gemm_f32((const float*)x, (const float*)m.w, (float*)y, n, O, I, ldx, I, O, stream);
    case LIN_PLAIN: return gibbs_gemm_bf16_plain(x, m.w, y, out_dtype, n, O, I, ldx, I, O, stream);
    case LIN_SKINNY: {
      const bool packed = use_packed && m.packed;
      return gibbs_gemm_skinny(x, packed ? m.packed : m.w, y, c.splits > 1 ? GIBBS_F32 : out_dtype, n, O, I, ldx, packed ? 0 : I, O,
                               c.splits, stream);
    }
    case LIN_LIBRARY: return gibbs_gemm_library(x, m.w, y, n, O, I, ldx, I, O, stream);
    default: return gibbs_gemm_bf16(x, m.w, y, out_dtype, n, O, I, ldx, I, O, stream);
  }
}

// x += y W^T with the mirror kept, for the rows of a fused decode step.  Many rows and a long inner size:
// every workgroup re-reads y, so workgroups take 64 features each and the chip is filled by cutting k
// instead; the float32 partial sums are added to the stream by a second kernel (measured at 33 to 64 rows:
// 17 against 24 us at k = 8192, 12 against 9 at 2048).  Returns the number of partial sums (0: one kernel).
int residual_parts(int n, int O, int I) { return (n > 32 && I >= 4096) ? skinny_splits(O, I, 256, 64, 256) : 0; }
int run_skinny_residual(const void* y, const void* w, long ldw, float* x, void* mirror, int n, int O, int I, float* parts,
                        hipStream_t stream) {
  const int splits = residual_parts(n, O, I);
  if (splits == 0) return gibbs_skinny_residual(y, w, x, mirror, n, O, I, I, ldw, stream);
  if (gibbs_gemm_skinny(y, w, parts, GIBBS_F32, n, O, I, I, ldw, O, splits, stream)) return 1;
  return gibbs_residual_add(x, parts, GIBBS_F32, splits, (long)n * O, mirror, (long)n * O, stream);
}

// ------------------------------------------------------------------------------------------------- the workspace
// First-fit allocator over the workspace with coalescing; in a dry run it only tracks the high-water mark.
struct Arena {
  char* base;
  long size;
  bool dry;
  long peak = 0;
  std::map<long, long> free_ranges;   // offset -> bytes
  std::map<long, long> taken;         // offset -> bytes
  // (a dry run hands out addresses that nothing dereferences, from a base that is aligned like a real one)
  Arena(void* b, long n, bool d) : base(d ? (char*)4096 : (char*)b), size(d ? (1L << 46) : n), dry(d) { free_ranges[0] = size; }
  void* take(long bytes) {
    bytes = (std::max<long>(bytes, 1) + 255) / 256 * 256;
    for (auto it = free_ranges.begin(); it != free_ranges.end(); ++it) {
      if (it->second < bytes) continue;
      const long off = it->first, rest = it->second - bytes;
      free_ranges.erase(it);
      if (rest > 0) free_ranges[off + bytes] = rest;
      taken[off] = bytes;
      peak = std::max(peak, off + bytes);
      return base + off;
    }
    return nullptr;
  }
  void give(void* p) {
    if (!p) return;
    const long off = (char*)p - base;
    auto it = taken.find(off);
    if (it == taken.end()) return;
    long bytes = it->second, start = off;
    taken.erase(it);
    auto next = free_ranges.lower_bound(start);
    if (next != free_ranges.end() && next->first == start + bytes) {
      bytes += next->second;
      next = free_ranges.erase(next);
    }
    if (next != free_ranges.begin()) {
      auto prev = std::prev(next);
      if (prev->first + prev->second == start) {
        start = prev->first;
        bytes += prev->second;
        free_ranges.erase(prev);
      }
    }
    free_ranges[start] = bytes;
  }
};

// A delta that has not been added to the residual stream yet.
struct Pending {
  void* data = nullptr;
  int parts = 0;   // 0: nothing; 1: [N, H] in the activation type; >= 2: float32 partial sums [parts, N, H]
};

struct Plan;

// What the parts need of a running step: its operands, the workspace, and the products.
struct Exec {
  const Plan& p;
  const GibbsStepArgs& a;
  Arena arena;
  bool dry;
  int status = 0;
  int esize;                  // bytes of an activation element
  bool bf16_run;
  bool few_rows;              // a bfloat16 step of so few rows that the weight-streaming products with fused epilogues take it
  bool fused_step;            // and every row is one token of a request of its own (decoded tokens)
  int fused_halves = 0;
  // rows that a body of this step has published for later bodies (an attention's values, for layers that mix them
  // into their own), by key; given back when the step ends
  std::map<int, void*> published;
  // A mixture of experts' weighted sum that has not been written yet: the operation that adds the delta into the stream may
  // sum it on its way (one kernel less, and the sum stays float32); whatever else comes first writes it (`mix_now`).
  struct DeferredMix {
    void* delta = nullptr;      // where the sum goes (null: nothing is deferred)
    void* y = nullptr;          // [places, hidden]: the choices' results
    int* place = nullptr;       // [n, top]
    float* weight = nullptr;    // [n, top]
    void* shared = nullptr;     // [n, hidden] or null
    float* gate = nullptr;      // [n] or null
    int top = 0;
  } deferred;
  void mix_done() {
    give(deferred.shared);
    give(deferred.y);
    give(deferred.place);
    give(deferred.weight);
    give(deferred.gate);
    deferred = DeferredMix{};
  }
  void mix_now();
  Exec(const Plan& plan, const GibbsStepArgs& args);
  void* take(long bytes) {
    void* ptr = arena.take(bytes);
    if (!ptr && !status) status = gibbs_fail("step: the workspace of %ld bytes is too small", a.workspace_bytes);
    return ptr;
  }
  void give(void* ptr) { arena.give(ptr); }
  bool ok() const { return status == 0; }
  const int* table(int group) const { return a.tables[group]; }
  int width(int group) const { return a.widths[group]; }
  // A step of one token per request: row n is request n, and the attention need not look that up (a dependent
  // load less in front of its page ids).
  bool rows_are_requests() const { return a.max_q == 1 && a.n_rows == a.n_req; }

  // y = x @ W^T in the precision of the run.  `out_f32`: float32 output; `partial_ok`: the caller takes
  // float32 partial sums; `use_packed`: the few-row kernel may read the tile-ordered copy.  Returns the
  // buffer ([N, O], or [parts, N, O] float32 with *parts >= 2).
  void* linear(const void* x, const Matrix& m, int n, bool out_f32, bool partial_ok, bool use_packed, int* parts, long ldx = 0);
  void linear_into(const void* x, const Matrix& m, int n, bool out_f32, bool use_packed, void* y);
  // adds what is pending and makes sure the bfloat16 mirror of x exists
  void with_mirror(float* x, Pending& pending, void** mirror);
  // adds what is pending into x
  void settle(float* x, Pending& pending);
  // x += y @ W^T with the mirror kept (the last product of a fused half of a layer)
  void skinny_residual(const void* y, const Matrix& m, float* x, void* mirror);
  void run();
};
// queues a kernel unless this is a dry run or an earlier call failed
#define RUN(e, call)                                            \
  do {                                                          \
    if (!(e).dry && (e).status == 0 && (call)) (e).status = 1;  \
  } while (0)

// ------------------------------------------------------------------------------------------------- parts
struct NormPart {
  virtual ~NormPart() = default;
  // x += pending (if any, when all rows are normed); returns norm(x) of all rows (or of `rows`) in the activation type
  virtual void* run(Exec& e, float* x, Pending& pending, const int* rows, int n_out) const = 0;
  // an RMS norm whose gain is folded into the matrices that follow: the fused kernels do the rest of it
  virtual bool folded_rms(float* eps) const { return false; }
  // the norm of a part's result before it is added (the stream is not touched); gives the delta's buffer back
  virtual Pending run_on(Exec& e, Pending delta) const;
  // x += norm(a part's result) in one pass, where the norm can (else: false, and nothing is done)
  virtual bool add_normed(Exec& e, float* x, Pending delta) const { return false; }
  // the norm of a weighted sum of several residual streams x [streams][N][hidden] (coef null: their plain sum), of all
  // rows or of `rows`; the streams are not touched
  virtual void* run_streams(Exec& e, const float* x, int streams, const float* coef, const int* rows, int n_out) const;
  // a plain RMS norm with its gain (null: none) and eps, for kernels that apply it beside their own work
  virtual bool plain_rms(const float** gain, float* eps) const { return false; }
  // an RMS norm in groups (1: a plain one) with its gain, for the kernel that norms a result into the stream and the
  // stream for the next sublayer in one pass
  virtual bool group_rms(const float** gain, float* eps, int* groups) const { return false; }
  // a norm that the streams' kernels apply themselves: its kind there (0 root mean square, 1 layer norm) and operands
  virtual bool for_streams(int* kind, const float** gain, const float** bias, float* eps) const { return false; }
};

struct Body {
  virtual ~Body() = default;
  virtual Pending general(Exec& e, void* h) const = 0;    // the delta of normed rows h [N, hidden]
  // has fused few-row kernels for its sizes and for this step (single: every row is one token of its own request;
  // a part that works on rows one by one, as a feed-forward does, need not ask for that)
  virtual bool fusable(bool single) const { return false; }
  virtual void fused(Exec& e, float eps, float* x, void* mirror) const {}   // x += body(x / rms(x)), mirror kept
  virtual int cache_group() const { return -1; }
};

// How a sublayer reads and writes several residual streams (hyper-connections): it reads u = sum_s in[s] x_s, and
// writes x_t <- sum_s mix[s][t] x_s + out[t] y for all t at once.
struct Hyper {
  const float* in = nullptr;    // [streams]
  const float* mix = nullptr;   // [streams, streams], indexed [from][to]
  const float* out = nullptr;   // [streams]
};

struct Plan {
  int dtype = GIBBS_BF16;   // activations, matrices and cache pages
  int hidden = 0, vocab = 0;
  const void* table = nullptr;
  int table_dtype = GIBBS_BF16;
  // residual streams: x is [streams][rows][hidden], every stream starting as the embedding's output
  int streams = 1;
  std::vector<Hyper> hypers;
  // tables whose rows are added to the token table's: one over hashed pairs (previous token, token), the row
  // `buckets` for a sequence's first token, and one over positions; the previous token of a request lives in its
  // state slot (prev_state [slots] int32, slot_stride words apart)
  const void* pair_table = nullptr;
  int buckets = 0, mul_prev = 0, mul_cur = 0;
  const void* pos_table = nullptr;
  int pos_len = 0;
  int* prev_state = nullptr;
  long prev_stride = 0;
  bool table_sums() const { return pair_table || pos_table || streams > 1; }
  float embed_scale = 1.0f;            // the table's rows are multiplied by it
  const float* embed_inv_freq = nullptr;   // [hidden / 2]: a sinusoidal position vector is added to the rows
  bool plain_embedding() const { return embed_scale == 1.0f && !embed_inv_freq && !reinjects && !table_sums(); }
  bool reinjects = false;              // the program adds the embedding's output into the stream again
  Matrix head;
  float logit_softcap = 0.f;   // > 0: logits <- cap * tanh(logits / cap)
  int tail = -1;            // the norm in front of the head
  int fused_rows = FUSED_ROWS;   // steps of at most this many decoded tokens take the fused decode kernels
  int own_gemm = 0;         // products above the few-row kernels' range: 0 the library's, 1 the tiled kernel
  std::vector<std::unique_ptr<NormPart>> norms;
  std::vector<std::unique_ptr<Body>> bodies;
  enum { OP_HALF, OP_NORM, OP_BODY, OP_ADD, OP_DROP, OP_NORM_DELTA, OP_REINJECT, OP_ADD_NORMED, OP_STREAMS_NORM, OP_STREAMS_ADD, OP_ROWS };
  struct Op {
    int kind, norm, body, value;   // value: what a body reads, an add adds, a drop drops
    int result;                    // the value that a norm or a body makes
  };
  std::vector<Op> ops;
  int n_values = 0;
  mutable int last_fused = 0;
  bool has_norm(int i) const { return i >= 0 && i < (int)norms.size(); }
  bool has_body(int i) const { return i >= 0 && i < (int)bodies.size(); }
  bool has_hyper(int i) const { return i >= 0 && i < (int)hypers.size(); }
};

Exec::Exec(const Plan& plan, const GibbsStepArgs& args)
    : p(plan), a(args), arena(args.workspace, args.workspace_bytes, args.workspace == nullptr), dry(args.workspace == nullptr) {
  esize = p.dtype == GIBBS_BF16 ? 2 : 4;
  bf16_run = p.dtype == GIBBS_BF16;
  few_rows = bf16_run && a.n_rows <= std::min(p.fused_rows, FUSED_ROWS);
  fused_step = few_rows && a.max_q == 1;
}

void* Exec::linear(const void* x, const Matrix& m, int n, bool out_f32, bool partial_ok, bool use_packed, int* parts, long ldx) {
  if (ldx == 0) ldx = m.I;     // (x may be a slice of wider rows)
  const LinearChoice c = choose_linear(bf16_run, n, m.O, m.I, aligned_for_matrix_cores(x, ldx, m.w, m.I), out_f32, partial_ok, p.own_gemm);
  const long elem = !bf16_run || out_f32 || c.splits > 1 ? 4 : 2;
  void* y = take((long)c.splits * n * m.O * elem);
  RUN(*this, run_linear(c, x, ldx, m, use_packed, y, n, out_f32, a.stream));
  if (parts) *parts = c.splits;
  return y;
}
void Exec::linear_into(const void* x, const Matrix& m, int n, bool out_f32, bool use_packed, void* y) {
  const LinearChoice c = choose_linear(bf16_run, n, m.O, m.I, aligned_for_matrix_cores(x, m.I, m.w, m.I), out_f32, false, p.own_gemm);
  RUN(*this, run_linear(c, x, m.I, m, use_packed, y, n, out_f32, a.stream));
}
void Exec::with_mirror(float* x, Pending& pending, void** mirror) {
  if (pending.parts == 0 && *mirror) return;
  const long count = (long)a.n_rows * p.hidden;
  if (!*mirror) *mirror = take(count * 2);
  RUN(*this, gibbs_residual_add(x, pending.data, pending.parts >= 2 ? GIBBS_F32 : (pending.parts == 1 ? p.dtype : 0),
                                std::max(pending.parts, 1), count, *mirror, count, a.stream));
  give(pending.data);
  pending = Pending{};
}
void Exec::settle(float* x, Pending& pending) {
  if (pending.parts == 0) return;
  const long count = (long)a.n_rows * p.hidden;
  RUN(*this, gibbs_residual_add(x, pending.data, pending.parts >= 2 ? GIBBS_F32 : p.dtype, pending.parts, count, nullptr, count,
                                a.stream));
  give(pending.data);
  pending = Pending{};
}
void Exec::skinny_residual(const void* y, const Matrix& m, float* x, void* mirror) {
  const int n = a.n_rows, splits = residual_parts(n, m.O, m.I);
  float* parts = splits ? (float*)take((long)splits * n * m.O * 4) : nullptr;
  RUN(*this, run_skinny_residual(y, m.packed ? m.packed : m.w, m.packed ? 0 : m.I, x, mirror, n, m.O, m.I, parts, a.stream));
  give(parts);
}

// ---- norms
Pending NormPart::run_on(Exec& e, Pending delta) const {
  if (!e.status) e.status = gibbs_fail("step: this norm cannot be applied to a part's result");
  return delta;
}
void* NormPart::run_streams(Exec& e, const float*, int, const float*, const int*, int) const {
  if (!e.status) e.status = gibbs_fail("step: this norm cannot read several residual streams");
  return nullptr;
}
struct RmsNorm : NormPart {
  const float* gain = nullptr;   // null: folded into the matrices that follow
  float eps = 0.f;
  void* run_streams(Exec& e, const float* x, int streams, const float* coef, const int* rows, int n_out) const override {
    const int H = e.p.hidden;
    void* out = e.take((long)n_out * H * e.esize);
    RUN(e, gibbs_streams_norm(x, streams, (long)e.a.n_rows * H, coef, 0, gain, nullptr, eps, out, e.p.dtype, rows, n_out, H, e.a.stream));
    return out;
  }
  bool for_streams(int* kind, const float** g, const float** b, float* e) const override {
    *kind = 0; *g = gain; *b = nullptr; *e = eps;
    return true;
  }
  void* run(Exec& e, float* x, Pending& pending, const int* rows, int n_out) const override {
    const int H = e.p.hidden;
    void* out = e.take((long)n_out * H * e.esize);
    if (pending.parts >= 2)
      RUN(e, gibbs_add_partials_rmsnorm(x, (const float*)pending.data, pending.parts, (long)e.a.n_rows * H, gain, eps, out, e.p.dtype,
                                        rows, n_out, H, e.a.stream));
    else
      RUN(e, gibbs_add_rmsnorm(x, pending.data, gain, eps, out, e.p.dtype, rows, n_out, H, e.a.stream));
    e.give(pending.data);
    pending = Pending{};
    return out;
  }
  bool folded_rms(float* e) const override {
    *e = eps;
    return gain == nullptr;
  }
  bool plain_rms(const float** g, float* e) const override {
    *g = gain; *e = eps;
    return true;
  }
  bool add_normed(Exec& e, float* x, Pending delta) const override {
    const int N = e.a.n_rows, H = e.p.hidden;
    RUN(e, gibbs_rmsnorm_rows_add(x, delta.data, std::max(delta.parts, 1), (long)N * H, gain, eps, e.p.dtype, N, H, e.a.stream));
    e.give(delta.data);
    return true;
  }
  Pending run_on(Exec& e, Pending delta) const override {
    const int N = e.a.n_rows, H = e.p.hidden;
    Pending out{e.take((long)N * H * e.esize), 1};
    RUN(e, gibbs_rmsnorm_rows(delta.data, std::max(delta.parts, 1), (long)N * H, gain, eps, out.data, e.p.dtype, N, H, e.a.stream));
    e.give(delta.data);
    return out;
  }
};
// RMS norm in `groups` equal consecutive parts of the row, each divided by its own root mean square; the gain over the whole row.
struct GroupRmsNorm : NormPart {
  const float* gain = nullptr;
  float eps = 0.f;
  int groups = 1;
  void* run(Exec& e, float* x, Pending& pending, const int* rows, int n_out) const override {
    const int H = e.p.hidden;
    e.settle(x, pending);
    void* out = e.take((long)n_out * H * e.esize);
    RUN(e, gibbs_group_rmsnorm(x, nullptr, 0, 0, nullptr, 0.f, 0, gain, eps, groups, out, e.p.dtype, rows, n_out, H, e.a.stream));
    return out;
  }
  bool group_rms(const float** g, float* ep, int* gr) const override {
    *g = gain; *ep = eps; *gr = groups;
    return true;
  }
  bool add_normed(Exec& e, float* x, Pending delta) const override {
    const int N = e.a.n_rows, H = e.p.hidden;
    RUN(e, gibbs_group_rmsnorm(x, delta.data, std::max(delta.parts, 1), (long)N * H, gain, eps, groups, nullptr, 0.f, 0, nullptr, e.p.dtype, nullptr,
                               N, H, e.a.stream));
    e.give(delta.data);
    return true;
  }
};
// Layer norm with gain and bias: (x - mean) / sqrt(mean((x - mean)^2) + eps) * gain + bias, all in float32.
struct LayerNorm : NormPart {
  const float* gain = nullptr;
  const float* bias = nullptr;
  float eps = 0.f;
  void* run_streams(Exec& e, const float* x, int streams, const float* coef, const int* rows, int n_out) const override {
    const int H = e.p.hidden;
    void* out = e.take((long)n_out * H * e.esize);
    RUN(e, gibbs_streams_norm(x, streams, (long)e.a.n_rows * H, coef, 1, gain, bias, eps, out, e.p.dtype, rows, n_out, H, e.a.stream));
    return out;
  }
  void* run(Exec& e, float* x, Pending& pending, const int* rows, int n_out) const override {
    e.settle(x, pending);
    return run_streams(e, x, 1, nullptr, rows, n_out);
  }
  bool for_streams(int* kind, const float** g, const float** b, float* e) const override {
    *kind = 1; *g = gain; *b = bias; *e = eps;
    return true;
  }
};
struct HostNorm : NormPart {
  GibbsHostNorm fn = nullptr;
  void* user = nullptr;
  void* run(Exec& e, float* x, Pending& pending, const int* rows, int n_out) const override {
    void* out = e.take((long)n_out * e.p.hidden * e.esize);
    RUN(e, fn(user, &e.a, x, pending.data, pending.parts, rows, n_out, out));
    e.give(pending.data);
    pending = Pending{};
    return out;
  }
};

// ---- gated short convolution
struct ConvBody : Body {
  Matrix in, out;
  const void* in_packed3 = nullptr;   // in-projection packed in three row groups (B, C, x), for the fused kernel
  const float* taps = nullptr;
  const float* bias = nullptr;
  int C = 0, K = 0;
  float* state = nullptr;        // [slots, K - 1, C] float32
  long slot_stride = 0;
  bool fusable(bool single) const override { return single && in.I % 8 == 0 && C % 8 == 0 && K <= 8; }
  void fused(Exec& e, float eps, float* x, void* mirror) const override {
    const int N = e.a.n_rows, H = in.I;
    void* y = e.take((long)N * C * 2);
    RUN(e, gibbs_skinny_conv(mirror, in_packed3 ? in_packed3 : in.w, y, N, C, H, H, in_packed3 ? 0 : H, 1, eps, taps, bias, state,
                             slot_stride, e.a.slot, e.a.ctx, K, e.a.stream));
    e.skinny_residual(y, out, x, mirror);
    e.give(y);
  }
  // the gated convolution of the projected rows [N, 3 C] with the requests' states; gives the rows back
  void* convolve(Exec& e, void* bcx) const {
    const int N = e.a.n_rows;
    void* y = e.take((long)N * C * e.esize);
    // (requests at the head of the batch that bring one row each: all of them in a step of decoded tokens)
    const int lead = e.a.max_q == 1 ? e.a.n_req : e.a.lead_single;
    RUN(e, gibbs_shortconv(bcx, taps, bias, state, slot_stride, e.a.cu, e.a.ctx, e.a.slot, y, e.p.dtype, N, e.a.n_req, lead, C, K, e.a.stream));
    e.give(bcx);
    return y;
  }
  Pending general(Exec& e, void* h) const override {
    const int N = e.a.n_rows;
    void* y = convolve(e, e.linear(h, in, N, false, false, false, nullptr));
    Pending delta;
    delta.data = e.linear(y, out, N, false, true, true, &delta.parts);
    e.give(y);
    return delta;
  }
};

// ---- attention over the paged cache
// What the attention kernels need to know of a mixer whose rows are prepared (normed, rotated, the new keys and
// values in their pages): q [N, nh * hd] (row stride ldq) against keys of head size hd and values of head size vd.
struct PagedAttention {
  void* kpages;
  void* vpages;
  int num_pages, page_size, group;
  int nh, nkv, hd, vd;
  float scale;
  int window;
  const float* slopes;    // a bias on the scores by distance: the plain kernel takes it
  const float* bias;      // [bias_len, nh]
  const float* bias_t;    // the same as [nh, bias_len] divided by the scale: what the matrix-core kernels add to raw scores
  int bias_len;
  const float* sink;      // [nh]: a term exp(sink[h]) in the softmax's denominator without key or value
  int chunk = 0;          // > 0: a row sees the keys of its own stretch of `chunk` positions (counted from 0) instead of a window
  float softcap = 0.f;    // > 0: scores are capped as softcap * tanh(s / softcap)
};
void decode_attention(Exec& e, const PagedAttention& t, const void* q, long ldq, int n_rows, const int* pos, const int* row_req, void* o) {
  int n_splits, waves;
  // (with chunks a row sees at most a chunk's keys: slices are chosen for that many)
  decode_splits(n_rows, t.nkv, t.nh / t.nkv, t.chunk > 0 ? std::min(e.a.max_seq, t.chunk) : e.a.max_seq, t.hd, t.page_size, 0, &n_splits, &waves);
  float* partial = n_splits > 1 ? (float*)e.take(gibbs_attention_decode_workspace(n_rows, t.nh, t.hd, n_splits) * 4) : nullptr;
  RUN(e, gibbs_attention_decode_masked(q, t.kpages, t.vpages, o, partial, pos, row_req, e.table(t.group), e.width(t.group), t.page_size,
                                       t.num_pages, n_rows, t.nh, t.nkv, t.hd, ldq, (long)t.nh * t.hd, t.scale, t.window, n_splits, waves, 0,
                                       e.a.max_seq, t.bias_t, t.bias_len, t.sink, t.chunk, t.softcap, e.a.stream));
  e.give(partial);
}
// attention of prepared rows, whatever the step's rows are; returns [N, nh * vd] (row stride ldo)
void* attend_prepared(Exec& e, const PagedAttention& t, void* raw, long ldq, long ldo) {
  const GibbsStepArgs& a = e.a;
  const int N = a.n_rows;
  const int* table = e.table(t.group);
  const int width = e.width(t.group);
  void* att = e.take((long)N * ldo * e.esize);
  // the matrix-core kernels take rows that are prepared (whatever prepared them), keys and values of one head
  // size, and a bias on the scores as a table over the distance (no slopes)
  const bool matrix_sizes = t.hd % 16 == 0 && t.hd <= 128;
  const bool fast_bf16 = e.bf16_run && !t.slopes && t.vd == t.hd && (!t.bias || (t.bias_t && matrix_sizes)) && (!t.sink || t.scale > 0.f) &&
                         (t.softcap == 0.f || t.scale > 0.f) && ldq % 8 == 0 && ((uintptr_t)raw % 16) == 0;
  if (fast_bf16 && a.max_q > 1 && matrix_sizes) {
    // decoded tokens at the head of the batch (where the scheduler puts them) take the kernel that splits
    // their keys (a row of its own in the matrix-core kernel would walk its cache alone); the rest the
    // matrix-core kernel
    const int lead = a.lead_single >= 2 ? a.lead_single : 0;
    if (lead) decode_attention(e, t, raw, ldq, lead, a.pos, a.row_req, att);
    const int rows = N - lead, reqs = a.n_req - lead;
    const int n_splits = a.max_seq > 0 ? prefill_splits(prefill_tiles(rows, reqs), t.nh, a.max_seq, t.chunk > 0 ? t.chunk : t.window) : 1;
    float* partial = n_splits > 1 ? (float*)e.take(gibbs_attention_decode_workspace(N, t.nh, t.hd, n_splits) * 4) : nullptr;
    RUN(e, gibbs_attention_prefill_masked(raw, t.kpages, t.vpages, att, partial, a.cu + lead, a.ctx + lead, table + (long)lead * width, reqs,
                                          width, t.page_size, t.num_pages, rows, t.nh, t.nkv, t.hd, ldq, ldo, t.scale, t.window, n_splits, lead,
                                          prefill_heads(rows, reqs, t.nh, t.nkv, t.hd, a.max_seq, n_splits), t.bias_t, t.bias_len, t.sink,
                                          t.chunk, t.softcap, a.stream));
    e.give(partial);
  } else if (fast_bf16 && a.max_q == 1 && t.hd % 8 == 0 && t.hd <= 256 && (!t.bias || matrix_sizes)) {
    decode_attention(e, t, raw, ldq, N, a.pos, a.row_req, att);
  } else {
    RUN(e, gibbs_attention_plain_masked(raw, t.kpages, t.vpages, att, e.p.dtype, a.pos, a.row_req, table, width, t.page_size, t.num_pages,
                                        N, t.nh, t.nkv, t.hd, t.vd, ldq, ldo, t.scale, t.window, t.slopes, t.bias, t.bias_len, t.sink, t.chunk,
                                        t.softcap, a.stream));
  }
  return att;
}

struct AttnBody : Body {
  Matrix qkv, out;
  const void* qkv_packed = nullptr;   // for the fused kernel
  int nh = 0, nkv = 0, hd = 0, window = 0;
  float scale = 0.f, qk_eps = 0.f;
  const float* q_gain = nullptr;
  const float* k_gain = nullptr;
  const float* inv_freq = nullptr;
  int rot = 0, variant = 0, table_len = 0;
  const float* cos_sin = nullptr;
  void* kpages = nullptr;
  void* vpages = nullptr;
  int num_pages = 0, page_size = 0, group = 0, owns = 0;
  const float* slopes = nullptr;      // a bias on the scores by distance: the plain kernel takes it
  GibbsHostRows hook = nullptr;       // something else done to q and k rows before k is cached
  void* hook_user = nullptr;
  // what gibbs_plan_attention_extras sets: values of a head size of their own, q and k divided by their root mean
  // square without a gain, a temperature on q that grows with the position, a table of score biases over the distance
  int vd = 0;
  int unit_qk = 0, temp_every = 0;
  int norm_dim = 0;                   // channels of a head that the unit norm's mean runs over (heads may be stored wider, zero-padded)
  float temp_coef = 0.f;
  const float* bias = nullptr;        // [bias_len, nh]
  const float* bias_t = nullptr;      // the same as [nh, bias_len] divided by the scale: what the matrix-core kernels add to raw scores
  int bias_len = 0;
  // what gibbs_plan_attention_projection sets: a bias on the projected rows, a sink in the softmax, values that are
  // published for later layers or mixed with what an earlier layer published (values of their own size with a rotation
  // on q and k come this way too: `general_prep`)
  const float* proj_bias = nullptr;   // [qkv.O] float32
  const float* sink = nullptr;        // [nh]
  int keep_mode = 0, keep_key = -1, vt = 0;
  const float* lambda = nullptr;
  bool general_prep = false;
  // what gibbs_plan_attention_gated sets (on top of the projection options): q and k normed per head with a gain before the
  // rotation; values that are the keys as projected; values turned by their position and the heads' outputs turned back;
  // chunks instead of a window; capped scores; a sigmoid gate on the heads' outputs from nh * vd further projected columns
  const float* prep_q_gain = nullptr;
  const float* prep_k_gain = nullptr;
  float prep_eps = 0.f;
  int prep_norm_dim = 0;
  int v_from_k = 0;
  const float* v_inv_freq = nullptr;
  int v_rot = 0;
  int chunk = 0;
  float softcap = 0.f;
  int gate_off = -1;                  // where the gate's columns start in a projected row (< 0: no gate)
  bool extras() const { return !general_prep && (vd != hd || unit_qk || temp_every > 0 || bias); }
  int cache_group() const override { return group; }
  // the fast kernels know rotations only (or no encoding at all)
  bool fast() const { return !slopes && !hook && !extras() && !general_prep; }
  // what the kernel that takes the raw projection (q/k norm, rotation, cache write and attention in one) needs
  bool raw_ok() const { return fast() && owns && hd % 16 == 0 && hd <= 256 && (!inv_freq || rot % 16 == 0); }
  bool fusable(bool single) const override { return single && raw_ok() && qkv.I % 8 == 0 && (nh * hd) % 8 == 0; }

  // decoded tokens from the raw projection: q/k norm, rotation, the cache write and attention in one kernel
  void* attend_decoded(Exec& e, const void* raw) const {
    const int N = e.a.n_rows;
    int n_splits, waves;
    decode_splits(N, nkv, nh / nkv, e.a.max_seq, hd, page_size, 0, &n_splits, &waves);
    float* partial = n_splits > 1 ? (float*)e.take(gibbs_attention_decode_workspace(N, nh, hd, n_splits) * 4) : nullptr;
    void* o = e.take((long)N * nh * hd * 2);
    RUN(e, gibbs_attention_decode_fused(raw, kpages, vpages, o, partial, q_gain, k_gain, qk_eps, inv_freq, rot, variant, cos_sin,
                                        cos_sin ? table_len : 0, e.a.pos, e.rows_are_requests() ? nullptr : e.a.row_req, e.table(group),
                                        e.width(group), page_size, num_pages, N, nh, nkv, hd, (long)(nh + 2 * nkv) * hd, (long)nh * hd,
                                        scale, window, n_splits, waves, 0, e.a.max_seq, e.a.stream));
    e.give(partial);
    return o;
  }
  void fused(Exec& e, float eps, float* x, void* mirror) const override {
    const int N = e.a.n_rows, H = qkv.I;
    void* raw = e.take((long)N * qkv.O * 2);
    RUN(e, gibbs_skinny_store(mirror, qkv_packed ? qkv_packed : qkv.w, raw, N, qkv.O, H, H, qkv_packed ? 0 : H, qkv.O, 1, eps, e.a.stream));
    void* att = attend_decoded(e, raw);
    e.give(raw);
    e.skinny_residual(att, out, x, mirror);
    e.give(att);
  }
  PagedAttention paged() const {
    return PagedAttention{kpages, vpages, num_pages, page_size, group, nh, nkv, hd, vd, scale, window, slopes, bias, bias_t, bias_len, sink, chunk, softcap};
  }
  // q/k norm, rotation and the cache write of the step's rows (a mixer that reads another's cache writes nothing)
  void prepare_rows(Exec& e, void* raw, long ldq) const {
    const int N = e.a.n_rows, kv = owns ? nkv : 0;
    const int* table = e.table(group);
    const int width = e.width(group);
    if (general_prep) {
      // bias, rotation, value mixing and the cache write in one pass; the values that later layers mix into theirs
      // stay in a buffer of the step
      void* keep = nullptr;
      if (keep_mode == 1) {
        keep = e.take((long)N * nkv * vt * e.esize);
        e.give(e.published[keep_key]);
        e.published[keep_key] = keep;
      } else if (keep_mode == 2) {
        auto it = e.published.find(keep_key);
        if (it == e.published.end() || !it->second) {
          if (!e.status) e.status = gibbs_fail("step: an attention mixes in the values of an earlier layer, and none has published them in this step");
          return;
        }
        keep = it->second;
      }
      RUN(e, gibbs_qkv_prepare_full(raw, ldq, owns ? kpages : nullptr, owns ? vpages : nullptr, e.p.dtype, proj_bias, inv_freq, rot, variant, cos_sin,
                                    table_len, keep, keep_mode, vt, lambda, e.a.pos, e.a.row_req, table, width, page_size, num_pages, N, nh, nkv, hd, vd,
                                    prep_q_gain, prep_k_gain, prep_eps, prep_norm_dim, v_from_k, v_inv_freq, v_rot, e.a.stream));
      return;
    }
    if (extras()) {
      RUN(e, gibbs_qk_unit_kv(raw, ldq, owns ? kpages : nullptr, owns ? vpages : nullptr, e.p.dtype, e.a.pos, e.a.row_req, table, width,
                              page_size, num_pages, N, nh, kv, hd, vd, qk_eps, unit_qk, norm_dim, temp_coef, temp_every, e.a.stream));
      return;
    }
    if (!hook) {
      RUN(e, gibbs_qk_rope_kv(raw, owns ? kpages : nullptr, owns ? vpages : nullptr, e.p.dtype, q_gain, k_gain, qk_eps, inv_freq, rot,
                              variant, cos_sin, cos_sin && inv_freq ? table_len : 0, e.a.pos, e.a.row_req, owns ? table : nullptr,
                              owns ? width : 0, owns ? page_size : 0, owns ? num_pages : 0, N, nh, kv, hd, ldq, e.a.stream));
      return;
    }
    // q/k norm (the kernel norms heads in place when it is given no pages), then the encoding's own doing on
    // the rows, then k and v into their pages
    char* k_rows = (char*)raw + (long)nh * hd * e.esize;
    if (q_gain)
      RUN(e, gibbs_qk_rope_kv(raw, nullptr, nullptr, e.p.dtype, q_gain, nullptr, qk_eps, nullptr, 0, 0, nullptr, 0, e.a.pos, e.a.row_req,
                              nullptr, 0, 0, 0, N, nh, 0, hd, ldq, e.a.stream));
    if (owns && k_gain)
      RUN(e, gibbs_qk_rope_kv(k_rows, nullptr, nullptr, e.p.dtype, k_gain, nullptr, qk_eps, nullptr, 0, 0, nullptr, 0, e.a.pos,
                              e.a.row_req, nullptr, 0, 0, 0, N, kv, 0, hd, ldq, e.a.stream));
    RUN(e, hook(hook_user, &e.a, raw, ldq));
    if (owns)
      RUN(e, gibbs_qk_rope_kv(raw, kpages, vpages, e.p.dtype, nullptr, nullptr, qk_eps, nullptr, 0, 0, nullptr, 0, e.a.pos, e.a.row_req,
                              table, width, page_size, num_pages, N, nh, kv, hd, ldq, e.a.stream));
  }
  // attention of the projected rows raw [N, (nh + 2 kv) hd]: whatever the step's rows are
  void* attend(Exec& e, void* raw) const {
    const GibbsStepArgs& a = e.a;
    const int N = a.n_rows, kv = owns ? nkv : 0;
    const long ldq = general_prep ? qkv.O : (long)(nh + kv) * hd + (long)kv * vd, ldo = (long)nh * vd;
    void* att;
    if (e.bf16_run && a.max_q == 1 && raw_ok()) {
      att = attend_decoded(e, raw);
    } else {
      prepare_rows(e, raw, ldq);
      att = attend_prepared(e, paged(), raw, ldq, ldo);
      // the heads' outputs turned back by the rows' positions, then times the sigmoid of the gate's columns
      if (general_prep && (v_inv_freq || gate_off >= 0))
        RUN(e, gibbs_attention_finish(att, ldo, gate_off >= 0 ? (char*)raw + (long)gate_off * e.esize : nullptr, ldq, vd, e.p.dtype, a.pos, v_inv_freq,
                                      v_rot, variant, N, nh, vd, vt > 0 ? vt : vd, a.stream));
    }
    return att;
  }
  Pending general(Exec& e, void* h) const override {
    const int N = e.a.n_rows;
    void* raw = e.linear(h, qkv, N, false, false, false, nullptr);
    void* att = attend(e, raw);
    e.give(raw);
    Pending delta;
    delta.data = e.linear(att, out, N, false, true, true, &delta.parts);
    e.give(att);
    return delta;
  }
};

// ---- gated dense feed-forward
struct GluBody : Body {
  Matrix gate_up, down;
  const void* gate_up_packed2 = nullptr;   // gate and up packed as two row groups, for the fused kernel
  int F = 0, act = 0;
  // act ACT_CLAMPED: min(gate, limit) * sigmoid(alpha * .) * (clamp(up, -limit, limit) + 1)
  float alpha = 0.f, limit = 0.f;
  bool fusable(bool) const override { return gate_up.I % 8 == 0 && F % 8 == 0; }   // (rows one by one: any few rows)
  void fused(Exec& e, float eps, float* x, void* mirror) const override {
    const int N = e.a.n_rows, H = gate_up.I;
    void* y = e.take((long)N * F * 2);
    RUN(e, gibbs_skinny_glu_general(mirror, gate_up_packed2 ? gate_up_packed2 : gate_up.w, y, N, F, H, H, gate_up_packed2 ? 0 : H, F, 1, eps,
                                    act, alpha, limit, e.a.stream));
    e.skinny_residual(y, down, x, mirror);
    e.give(y);
  }
  Pending general(Exec& e, void* h) const override {
    const int N = e.a.n_rows;
    void* y = e.take((long)N * F * e.esize);
    if (e.few_rows && fusable(false)) {
      // few rows: the gated product is the few-row kernel's epilogue (gate and up stay float32 until the product)
      RUN(e, gibbs_skinny_glu_general(h, gate_up_packed2 ? gate_up_packed2 : gate_up.w, y, N, F, gate_up.I, gate_up.I, gate_up_packed2 ? 0 : gate_up.I, F,
                                      0, 0.f, act, alpha, limit, e.a.stream));
    } else {
      void* gu = e.linear(h, gate_up, N, false, false, false, nullptr);
      if (act == ACT_CLAMPED)
        RUN(e, gibbs_glu_clamped(gu, y, e.p.dtype, N, F, alpha, limit, e.a.stream));
      else
        RUN(e, gibbs_glu(gu, y, e.p.dtype, N, F, act, e.a.stream));
      e.give(gu);
    }
    Pending delta;
    delta.data = e.linear(y, down, N, false, true, true, &delta.parts);
    e.give(y);
    return delta;
  }
};

// ---- a short causal convolution beside the identity on rows that a mixer is about to read: h <- h + conv(h)
struct ConvInputBody : Body {
  const float* taps = nullptr;   // [hidden, K], the last one the current token's
  int K = 0;
  float* state = nullptr;        // [slots][K - 1][hidden] float32: the requests' last K - 1 rows
  long slot_stride = 0;
  Pending general(Exec& e, void* h) const override {
    const GibbsStepArgs& a = e.a;
    const int N = a.n_rows, W = e.p.hidden;
    Pending out{e.take((long)N * W * e.esize), 1};
    RUN(e, gibbs_causal_conv(h, W, e.p.dtype, taps, nullptr, state, slot_stride, a.row_req, a.cu, a.slot, out.data, 0, W, N, a.n_req, W, K, 0, 1, 1,
                             a.max_q == 1, a.stream));
    return out;
  }
};

// ---- state-space mixer (a decayed outer-product state per head, one decay per head and token)
// One product gives [z: inner | x: inner | B: G D | C: G D | dt: H] of the normed rows (inner = H V, D the state size); x, B and
// C pass a short causal convolution with bias and silu; dt = softplus(dt + dt_bias); per head, with S [D, V] from zero,
// S = exp(-exp(A_log) dt) S + B (dt x)';  y = S' C + skip x;  then y silu(z), normed in groups, times a gain, projected back.
struct SsdBody : Body {
  Matrix in, out;
  int H = 0, V = 0, D = 0, G = 0, K = 0, norm_groups = 1;
  const float* taps = nullptr;       // [inner + 2 G D, K]
  const float* conv_bias = nullptr;  // [inner + 2 G D] or null
  const float* dt_bias = nullptr;    // [H]
  const float* a_log = nullptr;      // [H]
  const float* skip = nullptr;       // [H]
  const float* gain = nullptr;       // [inner]
  float* conv_state = nullptr;       // [slots][K - 1][inner + 2 G D]
  float* rule_state = nullptr;       // [slots][H][D][V]
  long slot_stride = 0;
  float eps = 0.f;
  Pending general(Exec& e, void* h) const override {
    const GibbsStepArgs& a = e.a;
    const int N = a.n_rows, inner = H * V, C = inner + 2 * G * D;
    char* raw = (char*)e.linear(h, in, N, false, false, false, nullptr);
    float* xbc = (float*)e.take((long)N * C * 4);
    RUN(e, gibbs_causal_conv(raw + (long)inner * e.esize, in.O, e.p.dtype, taps, conv_bias, conv_state, slot_stride, a.row_req, a.cu, a.slot, xbc, 1, C,
                             N, a.n_req, C, K, 1, 0, 1, a.max_q == 1, a.stream));
    // one request's long portion takes the rule in chunks (matrix products over 64 tokens at a time; it agrees with the walk
    // to rounding); everything else walks token by token
    const long chunk_floats = (a.n_req == 1 && N >= SSD_CHUNKED_ROWS && C % 4 == 0 && (G * D) % 4 == 0) ? gibbs_ssd_chunked_workspace(N, H, D, V) : 0;
    float* decay = (float*)e.take((long)N * H * 4);
    float* log_decay = chunk_floats ? (float*)e.take((long)N * H * 4) : nullptr;
    float* xdt = (float*)e.take((long)N * inner * 4);
    RUN(e, gibbs_ssd_prep(xbc, C, raw + (long)(inner + C) * e.esize, in.O, e.p.dtype, dt_bias, a_log, decay, log_decay, xdt, N, H, V, a.stream));
    float* o = (float*)e.take((long)N * inner * 4);
    if (chunk_floats) {
      float* work = (float*)e.take(chunk_floats * 4);
      RUN(e, gibbs_ssd_chunked(xbc + inner + (long)G * D, xbc + inner, C, xdt, inner, log_decay, rule_state, slot_stride, a.slot, o, work, N, H, G, D, V,
                               a.stream));
      e.give(work);
      e.give(log_decay);
    } else if (a.max_q == 1 && a.n_rows == a.n_req) {
      // one token per request: the kernel that streams the state in whole rows (the walk's arithmetic for the state itself)
      RUN(e, gibbs_ssd_step(xbc + inner + (long)G * D, xbc + inner, C, xdt, inner, decay, rule_state, slot_stride, a.slot, o, a.n_req, H, G, D, V, a.stream));
    } else {
      RUN(e, gibbs_ssd_rule(xbc + inner + (long)G * D, xbc + inner, C, xdt, inner, decay, rule_state, slot_stride, a.cu, a.slot, o, a.n_req, H, G, D, V,
                            a.stream));
    }
    e.give(decay);
    e.give(xdt);
    void* y = e.take((long)N * inner * e.esize);
    RUN(e, gibbs_gated_group_norm(o, xbc, C, skip, V, raw, in.O, gain, eps, norm_groups, y, e.p.dtype, N, inner, a.stream));
    e.give(o);
    e.give(xbc);
    e.give(raw);
    Pending delta;
    delta.data = e.linear(y, out, N, false, true, true, &delta.parts);
    e.give(y);
    return delta;
  }
};

// ---- gated delta rule with short convolutions
// One product gives [q | k | v | b | a | g] of the normed rows (segments start at multiples of 8 values); q, k, v
// pass a short causal convolution and silu; q and k become unit vectors; the rule runs over the requests' states
// S [heads, D, V]; each head's read-out is divided by its root mean square, multiplied by a gain and a gate, and
// projected back.  The decay is one per head (a: heads values) or one per head and key channel (a: a low-rank
// pair, a1 inside the product and a2 after it); the gate is silu of a full projection or sigmoid of a low-rank pair.
struct DeltaBody : Body {
  Matrix in, out, a2, g2;            // a2 / g2: the second matrices of the low-rank pairs (w null: none)
  int H = 0, G = 0, D = 0, V = 0, K = 0;
  int off_b = 0, off_a = 0, off_g = 0;   // where b, a (or a1) and g (or g1) start in a projected row
  const float* taps = nullptr;       // [2 G D + H V, K]
  const float* dt_bias = nullptr;
  const float* a_log = nullptr;
  const float* gain = nullptr;       // [V]
  float* conv_state = nullptr;       // [slots][K - 1][2 G D + H V]
  float* rule_state = nullptr;       // [slots][H][D][V]
  long slot_stride = 0;
  float eps = 0.f, unit_eps = 0.f, q_scale = 0.f;
  Pending general(Exec& e, void* h) const override {
    const GibbsStepArgs& a = e.a;
    const int N = a.n_rows, C = 2 * G * D + H * V;
    const bool channel = a2.w != nullptr;
    char* raw = (char*)e.linear(h, in, N, false, false, false, nullptr);
    float* qkv = (float*)e.take((long)N * C * 4);
    RUN(e, gibbs_causal_conv_silu(raw, in.O, e.p.dtype, taps, conv_state, slot_stride, a.row_req, a.cu, a.slot, qkv, N, a.n_req, C, K, 1,
                                  a.max_q == 1, a.stream));
    float* a_channel = channel ? (float*)e.linear(raw + (long)off_a * e.esize, a2, N, true, false, false, nullptr, in.O) : nullptr;
    float* beta = (float*)e.take((long)N * H * 4);
    float* decay = (float*)e.take((long)N * H * (channel ? D : 1) * 4);
    RUN(e, gibbs_delta_prep(qkv, qkv + (long)G * D, C, raw + (long)off_b * e.esize, raw + (long)off_a * e.esize, in.O, e.p.dtype, a_channel,
                            dt_bias, a_log, beta, decay, N, G, H, D, q_scale, unit_eps, a.stream));
    e.give(a_channel);
    float* o = (float*)e.take((long)N * H * V * 4);
    RUN(e, gibbs_delta_rule(qkv, qkv + (long)G * D, C, qkv + 2L * G * D, C, beta, decay, channel, rule_state, slot_stride, a.cu, a.slot, o,
                            a.n_req, H, G, D, V, a.stream));
    e.give(qkv);
    e.give(beta);
    e.give(decay);
    void* gate = g2.w ? e.linear(raw + (long)off_g * e.esize, g2, N, false, false, false, nullptr, in.O) : nullptr;
    void* y = e.take((long)N * H * V * e.esize);
    RUN(e, gibbs_head_norm_gate(o, gain, V, gate ? gate : raw + (long)off_g * e.esize, gate ? (long)H * V : in.O, y, e.p.dtype, N, H, V, eps,
                                g2.w ? 1 : 0, a.stream));
    e.give(gate);
    e.give(o);
    e.give(raw);
    Pending delta;
    delta.data = e.linear(y, out, N, false, true, true, &delta.parts);
    e.give(y);
    return delta;
  }
};

// ---- time mixing with a decayed outer-product state
// Each of r, k, v, g, w reads its own mix of the row and the row before it, h + (h' - h) mu_s; the decay is
// decay = exp(-exp(z)), z = w0 + W2 tanh(W1 mix_w); the rule runs over the requests' states S [heads, D, D]; each head's
// read-out is divided by its root mean square, multiplied by a gain and silu(g), and projected back.
struct TimeMixBody : Body {
  Matrix wr, wk, wv, wg, w1, w2, out;
  int H = 0, D = 0;
  const float* mu = nullptr;         // [5, hidden]: r, k, v, g, w
  const float* w0 = nullptr;         // [H D]
  const float* bonus = nullptr;      // [H, D]
  const float* gain = nullptr;       // [H D]
  float* shift_state = nullptr;      // [slots][hidden]: the previous token's normed row
  float* rule_state = nullptr;       // [slots][H][D][D]
  long slot_stride = 0;
  float eps = 0.f;
  Pending general(Exec& e, void* h) const override {
    const GibbsStepArgs& a = e.a;
    const int N = a.n_rows, W = e.p.hidden, C = H * D;
    char* mixes = (char*)e.take(5L * N * W * e.esize);
    RUN(e, gibbs_token_shift(h, e.p.dtype, mu, 5, shift_state, slot_stride, a.row_req, a.cu, a.slot, mixes, N, a.n_req, W, 1, a.max_q == 1,
                             a.stream));
    const long one = (long)N * W * e.esize;
    void* r = e.linear(mixes, wr, N, false, false, false, nullptr);
    void* k = e.linear(mixes + one, wk, N, false, false, false, nullptr);
    void* v = e.linear(mixes + 2 * one, wv, N, false, false, false, nullptr);
    void* g = e.linear(mixes + 3 * one, wg, N, false, false, false, nullptr);
    float* z = (float*)e.linear(mixes + 4 * one, w1, N, true, false, false, nullptr);
    e.give(mixes);
    void* t = e.take((long)N * w1.O * e.esize);
    RUN(e, gibbs_tanh_rows(z, t, e.p.dtype, (long)N * w1.O, a.stream));
    e.give(z);
    float* w = (float*)e.linear(t, w2, N, true, false, false, nullptr);
    e.give(t);
    RUN(e, gibbs_double_exp_decay(w, w0, (long)N * C, C, a.stream));
    float* o = (float*)e.take((long)N * C * 4);
    RUN(e, gibbs_decayed_outer_rule(r, k, v, e.p.dtype, w, bonus, rule_state, slot_stride, a.cu, a.slot, o, a.n_req, H, D, a.stream));
    e.give(r);
    e.give(k);
    e.give(v);
    e.give(w);
    void* y = e.take((long)N * C * e.esize);
    RUN(e, gibbs_head_norm_gate(o, gain, C, g, C, y, e.p.dtype, N, H, D, eps, 0, a.stream));
    e.give(o);
    e.give(g);
    Pending delta;
    delta.data = e.linear(y, out, N, false, true, true, &delta.parts);
    e.give(y);
    return delta;
  }
};

// ---- latent attention
// Keys and values of all heads come from one small latent per token: c = rms_norm(W_dkv h)[:rank] and a rotated key part
// k_r = rotate(W_dkv h)[rank : rank + rot] that all heads share; only [c | k_r] is cached, one row per token.  Head i's key is
// [W_uk,i c | k_r], its value W_uv,i c, its query [q_i (dim) | rotate(q_r,i) (rot)], with q = W_uq rms_norm(W_dq h) (or W_q h).
// The scores and the weighted values are taken on the cached rows themselves: q_i . W_uk,i c = (W_uk,i^T q_i) . c, so
// the queries become [W_uk,i^T q_i | rotate(q_r,i)] (rank + rot entries) and every head attends over the same rows
// (one kv head of size rank + rot whose values are the rows again); the weighted sum of the latents then goes
// through W_uv,i.  Softmax over a window, optionally with a sink per head; optionally a sigmoid gate on the heads'
// outputs from the mixer's input; the out-projection.
// One product gives [q or W_dq h | W_dkv h | gate] of the normed rows (segments start at multiples of 8 values).
struct LatentBody : Body {
  Matrix in, uq, out;                 // uq.w null: queries come straight from `in`
  const void* uk_t = nullptr;         // [heads][rank][dim]: W_uk of every head, transposed
  const void* uv = nullptr;           // [heads][vdim][rank]
  const float* q_gain = nullptr;      // [q_rank], or null: folded into W_uq's columns
  const float* kv_gain = nullptr;     // [rank]
  const float* sink = nullptr;        // [heads] or null
  const float* inv_freq = nullptr;    // [rot_dims / 2]
  int H = 0, D = 0, R = 0, V = 0, C = 0, q_rank = 0, rot_dims = 0, variant = 0, window = 0;
  int off_kv = 0, off_g = -1;         // where W_dkv h and the gate start in a projected row (off_g < 0: no gate)
  float scale = 0.f, eps = 0.f;
  void* pages = nullptr;              // [num_pages, 1, page_size, rank + rot]
  int num_pages = 0, page_size = 0, group = 0;
  int cache_group() const override { return group; }
  Pending general(Exec& e, void* h) const override {
    const GibbsStepArgs& a = e.a;
    const int N = a.n_rows, L = C + R;
    char* raw = (char*)e.linear(h, in, N, false, false, false, nullptr);
    void* q = raw;
    long ld_q = in.O;
    if (uq.w && e.few_rows && !q_gain && q_rank % 8 == 0 && in.O % 8 == 0 && ((uintptr_t)raw % 16) == 0 && ((uintptr_t)uq.w % 16) == 0) {
      // few rows, the latent's gain folded into W_uq: the product divides by the root mean square of the rows it reads
      // (the few-row kernel's prologue, as in the other models' fused decode products)
      q = e.take((long)N * uq.O * 2);
      RUN(e, gibbs_skinny_store(raw, uq.w, q, N, uq.O, q_rank, in.O, q_rank, uq.O, 1, eps, a.stream));
      ld_q = uq.O;
    } else if (uq.w) {
      void* cq = e.take((long)N * q_rank * e.esize);
      RUN(e, gibbs_rms_rows_ld(raw, in.O, q_gain, eps, cq, q_rank, e.p.dtype, N, q_rank, a.stream));
      q = e.linear(cq, uq, N, false, false, false, nullptr);
      ld_q = uq.O;
      e.give(cq);
    }
    void* q_lat = e.take((long)N * H * L * e.esize);
    RUN(e, gibbs_latent_prepare(raw + (long)off_kv * e.esize, in.O, q, ld_q, q_lat, (long)H * L, pages, e.p.dtype, kv_gain, eps, inv_freq,
                                rot_dims, variant, a.pos, a.row_req, e.table(group), e.width(group), page_size, num_pages, N, H, D, R, C,
                                a.stream));
    RUN(e, gibbs_gemm_heads(q, ld_q, D + R, uk_t, (long)C * D, D, q_lat, (long)H * L, L, e.p.dtype, N, C, D, H, a.stream));
    if (uq.w) e.give(q);
    const PagedAttention t{pages, pages, num_pages, page_size, group, H, 1, L, L, scale, window, nullptr, nullptr, nullptr, 0, sink};
    void* att = attend_prepared(e, t, q_lat, (long)H * L, (long)H * L);
    e.give(q_lat);
    void* o = e.take((long)N * H * V * e.esize);
    // (the gate multiplies the values' up-projection as it is stored)
    RUN(e, gibbs_gemm_heads_gated(att, (long)H * L, L, uv, (long)V * C, C, o, (long)H * V, V, off_g >= 0 ? raw + (long)off_g * e.esize : nullptr,
                                  in.O, V, e.p.dtype, N, V, C, H, a.stream));
    e.give(att);
    e.give(raw);
    Pending delta;
    delta.data = e.linear(o, out, N, false, true, true, &delta.parts);
    e.give(o);
    return delta;
  }
};

// ---- dense feed-forward without a gate: down(act(up h)), act a polynomial of row-normed powers
struct MlpBody : Body {
  Matrix up, down;
  int F = 0;
  const float* coef = nullptr;        // [4] on the device: a, b, c, e of a N(z) + b N(z^2) + c N(z^3) + e
  float eps = 0.f;
  Pending general(Exec& e, void* h) const override {
    const int N = e.a.n_rows;
    void* z = e.linear(h, up, N, false, false, false, nullptr);
    void* y = e.take((long)N * F * e.esize);
    RUN(e, gibbs_poly_norm(z, y, e.p.dtype, coef, eps, N, F, e.a.stream));
    e.give(z);
    Pending delta;
    delta.data = e.linear(y, down, N, false, true, true, &delta.parts);
    e.give(y);
    return delta;
  }
};

// ---- mixture of experts
// A router picks `top` of E gated feed-forwards for every row (logits and weights in float32, the weights a softmax over the
// chosen logits alone); the row's result is the weighted sum of theirs, plus a shared expert's times sigmoid(w_sg . h) where
// the layer has one.  The rows' (row, choice) pairs are sorted by expert on the device and the experts' products run over
// tiles of pairs that belong to one expert each (moe.hip); the host sees no count, so a step is still one queue of kernels.
struct MoeBody : Body {
  const float* router = nullptr;        // [E, hidden] float32
  const float* router_bias = nullptr;   // [E] or null
  const void* gate = nullptr;           // [E, F, hidden]
  const void* up = nullptr;             // [E, F, hidden]
  const void* down = nullptr;           // [E, hidden, F]
  int E = 0, top = 0, F = 0, act = 0;
  Matrix shared_gate_up, shared_down;   // the shared expert (w null: none): [2 SF, hidden], [hidden, SF]
  int SF = 0, shared_act = 0;
  const float* shared_gate = nullptr;   // [hidden] float32, or null: the shared expert is added as it is
  // mode 1: scores by a softmax over all router outputs, the choice by score + router_bias, weights the chosen scores over
  // their sum; the router's last `identity` outputs are experts without matrices whose result is the row itself
  int mode = 0, identity = 0;
  Pending general(Exec& e, void* h) const override {
    const int N = e.a.n_rows, W = e.p.hidden, pairs = N * top;
    const int bm = gibbs_moe_tile(pairs, E);
    const long cap = gibbs_moe_capacity(pairs, E, bm);
    int* chosen = (int*)e.take((long)pairs * 4);
    float* weight = (float*)e.take((long)pairs * 4);
    float* sgate = shared_gate ? (float*)e.take((long)N * 4) : nullptr;
    RUN(e, gibbs_moe_route_mode(h, W, e.p.dtype, router, router_bias, shared_gate, chosen, weight, sgate, N, W, E + identity, top, mode, e.a.stream));
    int* sorted = (int*)e.take(cap * 4);
    int* place = (int*)e.take((long)pairs * 4);
    int* tile_expert = (int*)e.take(cap / bm * 4);
    RUN(e, gibbs_moe_group(chosen, pairs, E, bm, sorted, place, tile_expert, cap, e.a.stream));
    e.give(chosen);
    void* mid = e.take(cap * F * e.esize);
    RUN(e, gibbs_moe_gemm(h, W, top, sorted, tile_expert, cap, bm, gate, up, mid, F, e.p.dtype, F, W, act, e.a.stream));
    void* y = e.take(cap * W * e.esize);
    RUN(e, gibbs_moe_gemm(mid, F, 0, sorted, tile_expert, cap, bm, down, nullptr, y, W, e.p.dtype, W, F, 0, e.a.stream));
    e.give(mid);
    e.give(sorted);
    e.give(tile_expert);
    void* shared = nullptr;
    if (shared_gate_up.w) {
      void* sy = e.take((long)N * SF * e.esize);
      if (e.few_rows && W % 8 == 0 && SF % 8 == 0) {
        RUN(e, gibbs_skinny_glu_general(h, shared_gate_up.w, sy, N, SF, W, W, W, SF, 0, 0.f, shared_act, 0.f, 0.f, e.a.stream));
      } else {
        void* gu = e.linear(h, shared_gate_up, N, false, false, false, nullptr);
        RUN(e, gibbs_glu(gu, sy, e.p.dtype, N, SF, shared_act, e.a.stream));
        e.give(gu);
      }
      shared = e.linear(sy, shared_down, N, false, false, false, nullptr);
      e.give(sy);
    }
    Pending delta{e.take((long)N * W * e.esize), 1};
    e.mix_now();      // (an earlier sum that nothing has taken yet)
    if (identity > 0) {
      // (the sum reads the rows themselves for the identity experts: it is taken now, while they are there)
      RUN(e, gibbs_moe_combine_self(y, place, weight, shared, sgate, h, delta.data, e.p.dtype, N, top, W, e.a.stream));
      e.give(shared); e.give(y); e.give(place); e.give(weight); e.give(sgate);
      return delta;
    }
    e.deferred.delta = delta.data;
    e.deferred.y = y; e.deferred.place = place; e.deferred.weight = weight; e.deferred.shared = shared; e.deferred.gate = sgate;
    e.deferred.top = top;
    return delta;
  }
};

// ---- a body from elsewhere
struct HostBody : Body {
  GibbsHostBody fn = nullptr;
  void* user = nullptr;
  int group = -1;
  int cache_group() const override { return group; }
  Pending general(Exec& e, void* h) const override {
    Pending delta;
    delta.data = e.take((long)e.a.n_rows * e.p.hidden * e.esize);
    delta.parts = 1;
    RUN(e, fn(user, &e.a, h, delta.data));
    return delta;
  }
};

// ------------------------------------------------------------------------------------------------- the step
void Exec::mix_now() {
  if (!deferred.delta) return;
  RUN(*this, gibbs_moe_combine(deferred.y, deferred.place, deferred.weight, deferred.shared, deferred.gate, deferred.delta, p.dtype, a.n_rows,
                               deferred.top, p.hidden, a.stream));
  mix_done();
}

void Exec::run() {
  const int N = a.n_rows, H = p.hidden;
  float* x = a.x_in;
  void* mirror = few_rows ? a.mirror_in : nullptr;
  float* embedded = nullptr;     // the embedding's output, for a program that adds it again
  const int S = p.streams;
  if (!x && p.table_sums()) {
    // the token table's row plus the pair table's and the position table's, into every stream; then the requests' last
    // tokens go to their slots, for the first row of their next portion
    x = (float*)take((long)S * N * H * 4);
    mirror = nullptr;
    RUN(*this, gibbs_embed_tables(p.table, p.pair_table, p.pos_table, p.table_dtype, a.ids, a.pos, a.row_req, a.cu, a.slot, p.prev_state,
                                  p.prev_stride, x, S, N, H, p.vocab, p.buckets, p.mul_prev, p.mul_cur, p.pos_len, a.stream));
    if (p.pair_table) RUN(*this, gibbs_store_last_token(a.ids, a.cu, a.slot, p.prev_state, p.prev_stride, a.n_req, a.stream));
  } else if (!x) {
    x = (float*)take((long)N * H * 4);
    mirror = few_rows ? take((long)N * H * 2) : nullptr;
    if (p.reinjects) embedded = (float*)take((long)N * H * 4);
    RUN(*this, gibbs_embed_general(p.table, p.table_dtype, a.ids, x, mirror, N, H, p.vocab, p.embed_scale, a.pos, p.embed_inv_freq,
                                   embedded, a.stream));
  }
  Pending pending;
  std::vector<void*> rows(p.n_values, nullptr);       // normed rows by value
  std::vector<Pending> deltas(p.n_values);           // deltas by value
  const bool whole = a.n_ops == 0;
  const int first = whole ? 0 : a.first_op, last = whole ? (int)p.ops.size() : a.first_op + a.n_ops;
  for (int i = first; i < last && ok(); ++i) {
    const Plan::Op& op = p.ops[i];
    if (deferred.delta && op.kind != Plan::OP_ADD_NORMED && !(op.kind == Plan::OP_DROP && deltas[op.value].data != deferred.delta)) mix_now();
    switch (op.kind) {
      case Plan::OP_HALF: {
        const NormPart& n = *p.norms[op.norm];
        const Body& b = *p.bodies[op.body];
        float eps = 0.f;
        if (few_rows && b.fusable(fused_step) && n.folded_rms(&eps)) {
          with_mirror(x, pending, &mirror);
          b.fused(*this, eps, x, mirror);
          ++fused_halves;
        } else {
          void* h = n.run(*this, x, pending, nullptr, N);
          pending = b.general(*this, h);
          give(h);
          give(mirror);
          mirror = nullptr;
        }
        break;
      }
      case Plan::OP_NORM:
        rows[op.result] = p.norms[op.norm]->run(*this, x, pending, nullptr, N);
        give(mirror);      // (x has taken what was pending: its mirror is stale)
        mirror = nullptr;
        break;
      case Plan::OP_BODY:
        deltas[op.result] = p.bodies[op.body]->general(*this, rows[op.value]);
        break;
      case Plan::OP_ROWS: {
        // a body whose result is read as rows by the next body (a filter on what a mixer reads), not added to the stream
        Pending made = p.bodies[op.body]->general(*this, rows[op.value]);
        if (made.parts != 1 && !status) status = gibbs_fail("step: a body whose result is read as rows must give whole rows");
        rows[op.result] = made.data;
        break;
      }
      case Plan::OP_ADD:
        settle(x, pending);
        pending = deltas[op.value];
        deltas[op.value] = Pending{};
        break;
      case Plan::OP_NORM_DELTA:
        deltas[op.result] = p.norms[op.norm]->run_on(*this, deltas[op.value]);
        deltas[op.value] = Pending{};
        break;
      case Plan::OP_ADD_NORMED: {
        // x += norm(delta) and the norm of the new x that the next operation asks for, in one kernel: a sublayer's
        // boundary (both norms plain RMS norms, nothing pending, sizes that the kernel takes)
        const Plan::Op* next = i + 1 < last && p.ops[i + 1].kind == Plan::OP_NORM ? &p.ops[i + 1] : nullptr;
        const float *gain_d = nullptr, *gain_n = nullptr;
        float eps_d = 0.f, eps_n = 0.f;
        Pending& d = deltas[op.value];
        if (next && pending.parts == 0 && d.data && p.norms[op.norm]->plain_rms(&gain_d, &eps_d) && p.norms[next->norm]->plain_rms(&gain_n, &eps_n)) {
          void* out = take((long)N * H * esize);
          int fused = -1;
          const bool mixed = deferred.delta && deferred.delta == d.data;
          if (!dry && status == 0) {
            fused = mixed ? gibbs_rmsnorm_rows_mix_add_norm(x, deferred.y, deferred.place, deferred.weight, deferred.top, deferred.shared, deferred.gate,
                                                            gain_d, eps_d, gain_n, eps_n, out, p.dtype, N, H, a.stream)
                          : gibbs_rmsnorm_rows_add_norm(x, d.data, std::max(d.parts, 1), (long)N * H, gain_d, eps_d, gain_n, eps_n, out, p.dtype, N, H, a.stream);
            if (fused > 0) status = 1;
          } else if (H % 4 == 0 && H <= 16384) {
            fused = 0;      // (a dry run: the same buffers as the real one will take)
          }
          if (fused == 0 && mixed) mix_done();
          if (fused == 0) {
            give(d.data);
            d = Pending{};
            give(mirror);
            mirror = nullptr;
            rows[next->result] = out;
            ++i;
            break;
          }
          give(out);
        }
        mix_now();
        {
          // the same boundary for RMS norms in groups: x += norm(delta) and the norm of the new x in one kernel
          const float *gd = nullptr, *gn = nullptr;
          float ed = 0.f, en = 0.f;
          int grd = 0, grn = 0;
          Pending& dd = deltas[op.value];
          if (next && pending.parts == 0 && dd.data && p.norms[op.norm]->group_rms(&gd, &ed, &grd) && p.norms[next->norm]->group_rms(&gn, &en, &grn)) {
            void* out = take((long)N * H * esize);
            RUN(*this, gibbs_group_rmsnorm(x, dd.data, std::max(dd.parts, 1), (long)N * H, gd, ed, grd, gn, en, grn, out, p.dtype, nullptr, N, H, a.stream));
            give(dd.data);
            dd = Pending{};
            give(mirror);
            mirror = nullptr;
            rows[next->result] = out;
            ++i;
            break;
          }
        }
        // (what is pending stays pending: additions into x commute, and the next norm still takes it on its way)
        if (p.norms[op.norm]->add_normed(*this, x, deltas[op.value])) {
          deltas[op.value] = Pending{};
          give(mirror);
          mirror = nullptr;
        } else {
          settle(x, pending);
          pending = p.norms[op.norm]->run_on(*this, deltas[op.value]);
          deltas[op.value] = Pending{};
        }
        break;
      }
      case Plan::OP_REINJECT:
        settle(x, pending);
        if (!embedded) { if (!status) status = gibbs_fail("step: the embedding's output is added again, but the caller brought the rows"); break; }
        RUN(*this, gibbs_residual_add(x, embedded, GIBBS_F32, 1, (long)N * H, nullptr, (long)N * H, a.stream));
        give(mirror);
        mirror = nullptr;
        break;
      case Plan::OP_STREAMS_NORM:
        rows[op.result] = p.norms[op.norm]->run_streams(*this, x, S, p.hypers[op.body].in, nullptr, N);
        break;
      case Plan::OP_STREAMS_ADD: {
        // the streams are written and, where the next operation reads them for a norm that the kernel knows, read in the
        // same pass (the rows are in registers already: a sublayer's boundary is one kernel, not two)
        const Hyper& hc = p.hypers[op.body];
        Pending& d = deltas[op.value];
        const Plan::Op* next = i + 1 < last && p.ops[i + 1].kind == Plan::OP_STREAMS_NORM ? &p.ops[i + 1] : nullptr;
        int kind = 0;
        const float *gain = nullptr, *bias = nullptr;
        float eps = 0.f;
        if (next && !p.norms[next->norm]->for_streams(&kind, &gain, &bias, &eps)) next = nullptr;
        void* out = next ? take((long)N * H * esize) : nullptr;
        RUN(*this, gibbs_streams_write_norm(x, S, (long)N * H, hc.mix, hc.out, d.data, d.parts >= 2 ? GIBBS_F32 : p.dtype, std::max(d.parts, 1),
                                            (long)N * H, N, H, next ? p.hypers[next->body].in : nullptr, kind, gain, bias, eps, out, p.dtype,
                                            a.stream));
        give(d.data);
        d = Pending{};
        if (next) {
          rows[next->result] = out;
          ++i;
        }
        break;
      }
      case Plan::OP_DROP:
        give(rows[op.value]);
        give(deltas[op.value].data);
        rows[op.value] = nullptr;
        deltas[op.value] = Pending{};
        break;
    }
  }
  mix_now();
  if (whole && a.n_logits > 0 && ok()) {
    // (several streams: the model's output is their sum)
    void* h = S > 1 ? p.norms[p.tail]->run_streams(*this, x, S, nullptr, a.logit_rows, a.n_logits)
                    : p.norms[p.tail]->run(*this, x, pending, a.logit_rows, a.n_logits);
    linear_into(h, p.head, a.n_logits, true, true, a.logits);   // the head: float32 logits straight into the caller's buffer
    if (p.logit_softcap > 0.f) RUN(*this, gibbs_softcap_rows(a.logits, (long)a.n_logits * p.vocab, p.logit_softcap, a.stream));
    give(h);
  }
  if (a.settle) settle(x, pending);
  give(pending.data);
  for (void* r : rows) give(r);
  for (Pending& d : deltas) give(d.data);
  give(mirror);      // (buffers of the caller's are not the arena's: giving them back does nothing)
  for (auto& kv : published) give(kv.second);
  published.clear();
  give(embedded);
  give(x);
}

int check_args(const Plan* p, const GibbsStepArgs* a, bool whole_step) {
  GIBBS_REQUIRE(p && a, "step: no plan or no operands");
  GIBBS_REQUIRE(a->n_rows > 0 && a->n_req >= 0 && a->n_logits >= 0, "step: bad sizes rows=%d requests=%d wanted=%d", a->n_rows, a->n_req, a->n_logits);
  GIBBS_REQUIRE(a->workspace == nullptr || (a->workspace_bytes > 0 && ((uintptr_t)a->workspace % 256) == 0), "step: the workspace is empty or not 256-byte aligned");
  if (!whole_step) return 0;
  GIBBS_REQUIRE(a->n_req > 0 && a->max_q >= 1, "step: bad sizes rows=%d requests=%d", a->n_rows, a->n_req);
  GIBBS_REQUIRE(a->lead_single >= 0 && a->lead_single <= a->n_req, "step: %d leading decoded tokens among %d requests", a->lead_single, a->n_req);
  GIBBS_REQUIRE(a->first_op >= 0 && a->n_ops >= 0 && a->first_op + a->n_ops <= (int)p->ops.size(), "step: operations %d .. %d of %d", a->first_op, a->first_op + a->n_ops, (int)p->ops.size());
  GIBBS_REQUIRE(a->x_in || p->table, "step: the plan has no token table and the caller brought no rows");
  GIBBS_REQUIRE(!a->x_in || !p->reinjects || a->n_ops, "step: this model adds its embedding's output again: the step embeds its rows itself");
  if (a->n_ops == 0 && a->n_logits > 0) {
    GIBBS_REQUIRE(p->has_norm(p->tail) && p->head.w, "step: logits are wanted and the plan has no final norm or no head");
    GIBBS_REQUIRE(a->workspace == nullptr || a->logits, "step: logits are wanted and there is no buffer for them");
  }
  GIBBS_REQUIRE(!p->table_sums() || (p->embed_scale == 1.0f && !p->embed_inv_freq && !p->reinjects), "step: an embedding with a pair or position table, or several streams, takes no scale, sinusoid or second addition");
  GIBBS_REQUIRE(!a->x_in || !p->table_sums() || a->n_ops, "step: this model's embedding is more than the token table's rows: the step embeds its rows itself");
  GIBBS_REQUIRE(!p->pair_table || (p->prev_state && a->slot && a->cu && a->row_req), "step: the pair table needs the requests' slots");
  const int first = a->n_ops ? a->first_op : 0, last = a->n_ops ? a->first_op + a->n_ops : (int)p->ops.size();
  for (int i = first; i < last; ++i) {
    const Plan::Op& op = p->ops[i];
    const bool of_streams = op.kind == Plan::OP_STREAMS_NORM || op.kind == Plan::OP_STREAMS_ADD;
    const bool of_one = op.kind == Plan::OP_HALF || op.kind == Plan::OP_NORM || op.kind == Plan::OP_ADD || op.kind == Plan::OP_ADD_NORMED ||
                        op.kind == Plan::OP_REINJECT;
    GIBBS_REQUIRE(p->streams == 1 || !of_one, "step: operation %d works on one residual stream, the plan has %d", i, p->streams);
    GIBBS_REQUIRE(!of_streams || p->streams <= 8, "step: %d residual streams (1 to 8)", p->streams);
    if (op.kind != Plan::OP_HALF && op.kind != Plan::OP_BODY && op.kind != Plan::OP_ROWS) continue;
    const int g = p->bodies[op.body]->cache_group();
    GIBBS_REQUIRE(g < 0 || (g < a->n_groups && a->tables && a->tables[g] && a->widths[g] > 0), "step: no block table for cache group %d", g);
  }
  return 0;
}

Plan* open_plan(void* plan) {
  if (!plan) gibbs_fail("plan: null");
  return (Plan*)plan;
}
}  // namespace

// ------------------------------------------------------------------------------------------------- building a plan
GIBBS_EXPORT void* gibbs_plan_create(int dtype, int hidden, int vocab, const void* table, int table_dtype, const void* head,
                                     const void* head_packed, int fused_rows, int own_gemm) {
  if ((dtype != GIBBS_BF16 && dtype != GIBBS_F32) || hidden <= 0 || vocab < 0) {
    gibbs_fail("plan: bad model sizes");
    return nullptr;
  }
  if (dtype == GIBBS_BF16 && !own_gemm && gibbs_gemm_library_init()) return nullptr;
  Plan* p = new Plan();
  p->dtype = dtype; p->hidden = hidden; p->vocab = vocab; p->table = table; p->table_dtype = table_dtype;
  p->head.w = head; p->head.packed = head_packed; p->head.O = vocab; p->head.I = hidden;
  p->fused_rows = fused_rows; p->own_gemm = own_gemm;
  return p;
}
GIBBS_EXPORT void gibbs_plan_destroy(void* plan) { delete (Plan*)plan; }

GIBBS_EXPORT int gibbs_plan_norm_rms(void* plan, const float* gain, float eps) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  auto n = std::make_unique<RmsNorm>();
  n->gain = gain; n->eps = eps;
  p->norms.push_back(std::move(n));
  return (int)p->norms.size() - 1;
}
GIBBS_EXPORT int gibbs_plan_norm_host(void* plan, GibbsHostNorm fn, void* user) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!fn) { gibbs_fail("plan: a norm from elsewhere needs its function"); return -1; }
  auto n = std::make_unique<HostNorm>();
  n->fn = fn; n->user = user;
  p->norms.push_back(std::move(n));
  return (int)p->norms.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_conv(void* plan, const void* w_in, const void* p_in3, const void* w_out, const void* p_out,
                                      const float* taps, const float* bias, int C, int K, float* state, long slot_stride) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!(w_in && w_out && taps && state && C > 0 && K >= 2 && slot_stride >= (long)(K - 1) * C)) {
    gibbs_fail("plan: bad short convolution C=%d K=%d", C, K);
    return -1;
  }
  auto c = std::make_unique<ConvBody>();
  c->in = Matrix{w_in, nullptr, 3 * C, p->hidden}; c->in_packed3 = p_in3;
  c->out = Matrix{w_out, p_out, p->hidden, C};
  c->taps = taps; c->bias = bias; c->C = C; c->K = K; c->state = state; c->slot_stride = slot_stride;
  p->bodies.push_back(std::move(c));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_attention(void* plan, const void* w_qkv, const void* p_qkv, const void* w_out, const void* p_out,
                                           int nh, int nkv, int hd, float scale, int window, const float* q_gain,
                                           const float* k_gain, float qk_eps, const float* inv_freq, int rot, int variant,
                                           const float* cos_sin, int table_len, void* kpages, void* vpages, int num_pages,
                                           int page_size, int group, int owns, const float* slopes, GibbsHostRows hook,
                                           void* hook_user) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!(w_qkv && w_out && nh > 0 && nkv > 0 && nh % nkv == 0 && hd > 0 && kpages && vpages && num_pages > 0 && page_size > 0 && group >= 0)) {
    gibbs_fail("plan: bad attention heads=%d kv=%d hd=%d group=%d", nh, nkv, hd, group);
    return -1;
  }
  auto t = std::make_unique<AttnBody>();
  t->qkv = Matrix{w_qkv, nullptr, (nh + (owns ? 2 * nkv : 0)) * hd, p->hidden}; t->qkv_packed = p_qkv;
  t->out = Matrix{w_out, p_out, p->hidden, nh * hd};
  t->nh = nh; t->nkv = nkv; t->hd = hd; t->scale = scale; t->window = window; t->q_gain = q_gain; t->k_gain = k_gain; t->qk_eps = qk_eps;
  t->inv_freq = inv_freq; t->rot = inv_freq ? rot : 0; t->variant = variant; t->cos_sin = cos_sin; t->table_len = table_len;
  t->kpages = kpages; t->vpages = vpages; t->num_pages = num_pages; t->page_size = page_size; t->group = group; t->owns = owns;
  t->slopes = slopes; t->hook = hook; t->hook_user = hook_user; t->vd = hd;
  p->bodies.push_back(std::move(t));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_glu(void* plan, const void* w_gate_up, const void* p_gate_up2, const void* w_down,
                                     const void* p_down, int F, int act) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!(w_gate_up && w_down && F > 0)) {
    gibbs_fail("plan: bad feed-forward width %d", F);
    return -1;
  }
  auto g = std::make_unique<GluBody>();
  g->gate_up = Matrix{w_gate_up, nullptr, 2 * F, p->hidden}; g->gate_up_packed2 = p_gate_up2;
  g->down = Matrix{w_down, p_down, p->hidden, F};
  g->F = F; g->act = act;
  p->bodies.push_back(std::move(g));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_host(void* plan, GibbsHostBody fn, void* user, int group) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!fn) { gibbs_fail("plan: a body from elsewhere needs its function"); return -1; }
  auto b = std::make_unique<HostBody>();
  b->fn = fn; b->user = user; b->group = group;
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_norm_layer(void* plan, const float* gain, const float* bias, float eps) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  auto n = std::make_unique<LayerNorm>();
  n->gain = gain; n->bias = bias; n->eps = eps;
  p->norms.push_back(std::move(n));
  return (int)p->norms.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_latent(void* plan, const GibbsLatentSpec* d) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!d || !(d->w_in && d->w_out && d->w_uk_t && d->w_uv && d->pages && d->heads > 0 && d->dim > 0 && d->rot >= 0 && d->vdim > 0 &&
              d->rank > 0 && d->in_rows > 0 && d->off_kv >= 0 && d->off_kv + d->rank + d->rot <= d->in_rows && d->num_pages > 0 &&
              d->page_size > 0 && d->group >= 0 && d->window >= 0 && (d->rot_dims == 0 || d->inv_freq) && d->rot_dims <= d->rot &&
              (!d->w_uq || d->q_rank > 0) && (d->off_g < 0 || d->off_g + d->heads * d->vdim <= d->in_rows))) {
    gibbs_fail("plan: bad latent attention");
    return -1;
  }
  if (d->rank + d->rot > 512) { gibbs_fail("plan: a cached row of %d values (latent + rotated key part) is more than the attention kernels take (512)", d->rank + d->rot); return -1; }
  auto b = std::make_unique<LatentBody>();
  b->in = Matrix{d->w_in, nullptr, d->in_rows, p->hidden};
  if (d->w_uq) b->uq = Matrix{d->w_uq, nullptr, d->heads * (d->dim + d->rot), d->q_rank};
  b->out = Matrix{d->w_out, nullptr, p->hidden, d->heads * d->vdim};
  b->uk_t = d->w_uk_t; b->uv = d->w_uv; b->q_gain = d->q_gain; b->kv_gain = d->kv_gain; b->sink = d->sink; b->inv_freq = d->inv_freq;
  b->H = d->heads; b->D = d->dim; b->R = d->rot; b->V = d->vdim; b->C = d->rank; b->q_rank = d->q_rank; b->rot_dims = d->rot_dims;
  b->variant = d->variant; b->window = d->window; b->off_kv = d->off_kv; b->off_g = d->off_g; b->scale = d->scale; b->eps = d->eps;
  b->pages = d->pages; b->num_pages = d->num_pages; b->page_size = d->page_size; b->group = d->group;
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_mlp(void* plan, const void* w_up, const void* w_down, int F, const float* coef, float eps) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!(w_up && w_down && coef && F > 0)) { gibbs_fail("plan: bad feed-forward width %d", F); return -1; }
  auto b = std::make_unique<MlpBody>();
  b->up = Matrix{w_up, nullptr, F, p->hidden};
  b->down = Matrix{w_down, nullptr, p->hidden, F};
  b->F = F; b->coef = coef; b->eps = eps;
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_streams(void* plan, int streams) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (streams < 1 || streams > 8) { gibbs_fail("plan: %d residual streams (1 to 8)", streams); return -1; }
  p->streams = streams;
  return 0;
}
GIBBS_EXPORT int gibbs_plan_hyper(void* plan, const float* in, const float* mix, const float* out) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!(in && mix && out)) { gibbs_fail("plan: a hyper-connection needs its three tensors"); return -1; }
  p->hypers.push_back(Hyper{in, mix, out});
  return (int)p->hypers.size() - 1;
}
GIBBS_EXPORT int gibbs_plan_embedding_tables(void* plan, const void* pair_table, int buckets, int mul_prev, int mul_cur,
                                             const void* pos_table, int pos_len, int* prev_state, long prev_stride) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if ((pair_table && (buckets <= 0 || !prev_state || prev_stride <= 0)) || (pos_table && pos_len <= 0)) {
    gibbs_fail("plan: bad embedding tables (buckets %d, positions %d)", buckets, pos_len);
    return -1;
  }
  p->pair_table = pair_table; p->buckets = buckets; p->mul_prev = mul_prev; p->mul_cur = mul_cur;
  p->pos_table = pos_table; p->pos_len = pos_len; p->prev_state = prev_state; p->prev_stride = prev_stride;
  return 0;
}

// ---- more about parts that are there already
GIBBS_EXPORT int gibbs_plan_embedding(void* plan, float scale, const float* inv_freq) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  p->embed_scale = scale; p->embed_inv_freq = inv_freq;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_attention_extras(void* plan, int body, int vd, int unit_qk, int norm_dim, float temp_coef, int temp_every,
                                             const float* bias, const float* bias_t, int bias_len) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  AttnBody* t = p->has_body(body) ? dynamic_cast<AttnBody*>(p->bodies[body].get()) : nullptr;
  if (!t || vd <= 0 || temp_every < 0 || (bias && bias_len <= 0)) { gibbs_fail("plan: body %d is no attention, or bad extras", body); return -1; }
  if (t->inv_freq || t->q_gain || t->k_gain || t->hook || t->slopes || !t->owns) {
    gibbs_fail("plan: an attention with these extras has no rotation, no q/k gains, no hook and no slopes, and owns its pages");
    return -1;
  }
  t->vd = vd; t->unit_qk = unit_qk; t->norm_dim = norm_dim > 0 ? norm_dim : t->hd; t->temp_coef = temp_coef; t->temp_every = temp_every; t->bias = bias; t->bias_t = bias ? bias_t : nullptr; t->bias_len = bias ? bias_len : 0;
  t->qkv.O = (t->nh + t->nkv) * t->hd + t->nkv * vd;
  t->out.I = t->nh * vd;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_attention_projection(void* plan, int body, int vd, const float* bias, const float* sink, int keep_mode,
                                                 int keep_key, int vt, const float* lambda) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  AttnBody* t = p->has_body(body) ? dynamic_cast<AttnBody*>(p->bodies[body].get()) : nullptr;
  if (!t || vd <= 0 || keep_mode < 0 || keep_mode > 2) { gibbs_fail("plan: body %d is no attention, or bad projection options", body); return -1; }
  if (t->q_gain || t->k_gain || t->hook || t->unit_qk || t->temp_every > 0 || !t->owns) {
    gibbs_fail("plan: an attention with projection biases, a sink or value mixing has no q/k norm, no hook and no temperature, and owns its pages");
    return -1;
  }
  if (keep_mode && !(vt > 0 && vt <= vd && keep_key >= 0 && (keep_mode == 1 || lambda))) { gibbs_fail("plan: value mixing needs a key, the values' size and its weight"); return -1; }
  t->general_prep = true;
  t->vd = vd; t->proj_bias = bias; t->sink = sink; t->keep_mode = keep_mode; t->keep_key = keep_key; t->vt = vt; t->lambda = lambda;
  t->qkv.O = (t->nh + t->nkv) * t->hd + t->nkv * vd;
  t->out.I = t->nh * vd;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_attention_gated(void* plan, int body, const float* q_gain, const float* k_gain, float qk_eps, int norm_dim,
                                            int v_from_k, const float* v_inv_freq, int v_rot, int chunk, float softcap, int gate) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  AttnBody* t = p->has_body(body) ? dynamic_cast<AttnBody*>(p->bodies[body].get()) : nullptr;
  if (!t || !t->general_prep || !t->owns) { gibbs_fail("plan: body %d is no attention that owns its pages and takes the projection options", body); return -1; }
  if (((q_gain || k_gain) && !(norm_dim > 0 && norm_dim <= t->hd)) || (v_inv_freq && !(v_rot > 0 && v_rot % 2 == 0 && v_rot <= t->vd)) || chunk < 0 ||
      (chunk > 0 && t->window > 0) || softcap < 0.f || (v_from_k && (t->keep_mode || v_inv_freq || t->vd > t->hd))) {
    gibbs_fail("plan: bad options of a gated attention (norm over %d of %d, %d turned value channels of %d, chunks of %d, window %d)", norm_dim, t->hd, v_rot, t->vd, chunk, t->window);
    return -1;
  }
  t->prep_q_gain = q_gain; t->prep_k_gain = k_gain; t->prep_eps = qk_eps; t->prep_norm_dim = norm_dim; t->v_from_k = v_from_k;
  t->v_inv_freq = v_inv_freq; t->v_rot = v_inv_freq ? v_rot : 0; t->chunk = chunk; t->softcap = softcap;
  int columns = (t->nh + t->nkv) * t->hd + (v_from_k ? 0 : t->nkv * t->vd);
  t->gate_off = gate ? columns : -1;
  if (gate) columns += t->nh * t->vd;
  t->qkv.O = columns;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_norm_group_rms(void* plan, const float* gain, float eps, int groups) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!gain || groups < 1 || p->hidden % groups) { gibbs_fail("plan: an RMS norm in %d parts of a width of %d, or no gain", groups, p->hidden); return -1; }
  auto n = std::make_unique<GroupRmsNorm>();
  n->gain = gain; n->eps = eps; n->groups = groups;
  p->norms.push_back(std::move(n));
  return (int)p->norms.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_conv_input(void* plan, const float* taps, int K, float* state, long slot_stride) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!(taps && state && K >= 1 && slot_stride >= (long)(K - 1) * p->hidden)) { gibbs_fail("plan: bad input convolution K=%d", K); return -1; }
  auto b = std::make_unique<ConvInputBody>();
  b->taps = taps; b->K = K; b->state = state; b->slot_stride = slot_stride;
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_ssd(void* plan, const GibbsSsdSpec* d) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!d || !(d->w_in && d->w_out && d->taps && d->dt_bias && d->a_log && d->skip && d->gain && d->conv_state && d->rule_state && d->heads > 0 &&
              d->groups > 0 && d->heads % d->groups == 0 && d->state > 0 && d->state <= 256 && d->vdim > 0 && d->taps_per_channel >= 1 &&
              d->norm_groups > 0 && (d->heads * d->vdim) % d->norm_groups == 0)) {
    gibbs_fail("plan: bad state-space mixer");
    return -1;
  }
  const int inner = d->heads * d->vdim, C = inner + 2 * d->groups * d->state;
  if (d->slot_stride < (long)d->heads * d->state * d->vdim || d->slot_stride < (long)(d->taps_per_channel - 1) * C) {
    gibbs_fail("plan: a state slot of %ld floats is too small for the state-space mixer", d->slot_stride);
    return -1;
  }
  auto b = std::make_unique<SsdBody>();
  b->in = Matrix{d->w_in, nullptr, inner + C + d->heads, p->hidden};
  b->out = Matrix{d->w_out, nullptr, p->hidden, inner};
  b->H = d->heads; b->V = d->vdim; b->D = d->state; b->G = d->groups; b->K = d->taps_per_channel; b->norm_groups = d->norm_groups;
  b->taps = d->taps; b->conv_bias = d->conv_bias; b->dt_bias = d->dt_bias; b->a_log = d->a_log; b->skip = d->skip; b->gain = d->gain;
  b->conv_state = d->conv_state; b->rule_state = d->rule_state; b->slot_stride = d->slot_stride; b->eps = d->eps;
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_logit_softcap(void* plan, float cap) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!(cap >= 0.f)) { gibbs_fail("plan: logits capped at %g", cap); return -1; }
  p->logit_softcap = cap;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_moe_scores(void* plan, int body, int mode, int identity) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  MoeBody* m = p->has_body(body) ? dynamic_cast<MoeBody*>(p->bodies[body].get()) : nullptr;
  if (!m || (mode != 0 && mode != 1) || identity < 0 || m->E + identity > 1024 || m->top > m->E + identity) { gibbs_fail("plan: body %d is no mixture of experts, or bad router options", body); return -1; }
  m->mode = mode; m->identity = identity;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_body_moe(void* plan, const GibbsMoeSpec* d) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!d || !(d->router && d->gate && d->up && d->down && d->experts > 0 && d->experts <= 1024 && d->top > 0 && d->top <= 1024 && d->F > 0 &&
              d->act >= 0 && d->act < 4 && (!d->shared_gate_up || (d->shared_down && d->shared_F > 0 && d->shared_act >= 0 && d->shared_act < 4)) &&
              (!d->shared_gate || d->shared_gate_up))) {
    gibbs_fail("plan: bad mixture of experts");
    return -1;
  }
  auto b = std::make_unique<MoeBody>();
  b->router = d->router; b->router_bias = d->router_bias; b->gate = d->gate; b->up = d->up; b->down = d->down;
  b->E = d->experts; b->top = d->top; b->F = d->F; b->act = d->act;
  if (d->shared_gate_up) {
    b->shared_gate_up = Matrix{d->shared_gate_up, nullptr, 2 * d->shared_F, p->hidden};
    b->shared_down = Matrix{d->shared_down, nullptr, p->hidden, d->shared_F};
    b->SF = d->shared_F; b->shared_act = d->shared_act; b->shared_gate = d->shared_gate;
  }
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_glu_clamped(void* plan, int body, float alpha, float limit) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  GluBody* g = p->has_body(body) ? dynamic_cast<GluBody*>(p->bodies[body].get()) : nullptr;
  if (!g || !(limit > 0.f)) { gibbs_fail("plan: body %d is no gated feed-forward, or its limit is not positive", body); return -1; }
  g->act = ACT_CLAMPED; g->alpha = alpha; g->limit = limit;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_body_delta(void* plan, const GibbsDeltaSpec* d) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!d || !(d->w_in && d->w_out && d->taps && d->dt_bias && d->a_log && d->gain && d->conv_state && d->rule_state && d->heads > 0 &&
              d->kv_heads > 0 && d->heads % d->kv_heads == 0 && d->dim > 0 && d->dim <= 256 && d->vdim > 0 && d->taps_per_channel >= 1 &&
              d->in_rows > 0 && d->off_b >= 0 && d->off_a >= 0 && d->off_g >= 0 && (!d->w_a2 || d->a_rank > 0) && (!d->w_g2 || d->g_rank > 0))) {
    gibbs_fail("plan: bad delta-rule mixer");
    return -1;
  }
  const int C = 2 * d->kv_heads * d->dim + d->heads * d->vdim;
  if (d->slot_stride < (long)d->heads * d->dim * d->vdim || d->slot_stride < (long)(d->taps_per_channel - 1) * C) {
    gibbs_fail("plan: a state slot of %ld floats is too small for the delta-rule mixer", d->slot_stride);
    return -1;
  }
  auto b = std::make_unique<DeltaBody>();
  b->in = Matrix{d->w_in, nullptr, d->in_rows, p->hidden};
  b->out = Matrix{d->w_out, nullptr, p->hidden, d->heads * d->vdim};
  if (d->w_a2) b->a2 = Matrix{d->w_a2, nullptr, d->heads * d->dim, d->a_rank};
  if (d->w_g2) b->g2 = Matrix{d->w_g2, nullptr, d->heads * d->vdim, d->g_rank};
  b->H = d->heads; b->G = d->kv_heads; b->D = d->dim; b->V = d->vdim; b->K = d->taps_per_channel;
  b->off_b = d->off_b; b->off_a = d->off_a; b->off_g = d->off_g;
  b->taps = d->taps; b->dt_bias = d->dt_bias; b->a_log = d->a_log; b->gain = d->gain;
  b->conv_state = d->conv_state; b->rule_state = d->rule_state; b->slot_stride = d->slot_stride;
  b->eps = d->eps; b->unit_eps = d->unit_eps; b->q_scale = d->q_scale;
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

GIBBS_EXPORT int gibbs_plan_body_time_mix(void* plan, const GibbsTimeMixSpec* d) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!d || !(d->w_r && d->w_k && d->w_v && d->w_g && d->w_1 && d->w_2 && d->w_out && d->mu && d->w0 && d->bonus && d->gain &&
              d->shift_state && d->rule_state && d->heads > 0 && d->dim > 0 && d->dim <= 256 && d->rank > 0)) {
    gibbs_fail("plan: bad time-mixing mixer");
    return -1;
  }
  if (d->slot_stride < (long)d->heads * d->dim * d->dim || d->slot_stride < p->hidden) {
    gibbs_fail("plan: a state slot of %ld floats is too small for the time-mixing mixer", d->slot_stride);
    return -1;
  }
  const int C = d->heads * d->dim, W = p->hidden;
  auto b = std::make_unique<TimeMixBody>();
  b->wr = Matrix{d->w_r, nullptr, C, W}; b->wk = Matrix{d->w_k, nullptr, C, W}; b->wv = Matrix{d->w_v, nullptr, C, W};
  b->wg = Matrix{d->w_g, nullptr, C, W}; b->w1 = Matrix{d->w_1, nullptr, d->rank, W}; b->w2 = Matrix{d->w_2, nullptr, C, d->rank};
  b->out = Matrix{d->w_out, nullptr, W, C};
  b->H = d->heads; b->D = d->dim; b->mu = d->mu; b->w0 = d->w0; b->bonus = d->bonus; b->gain = d->gain;
  b->shift_state = d->shift_state; b->rule_state = d->rule_state; b->slot_stride = d->slot_stride; b->eps = d->eps;
  p->bodies.push_back(std::move(b));
  return (int)p->bodies.size() - 1;
}

// ---- the program
namespace {
int append(Plan* p, int kind, int norm, int body, int value, bool makes_value) {
  Plan::Op op{kind, norm, body, value, makes_value ? p->n_values++ : -1};
  p->ops.push_back(op);
  return makes_value ? op.result : (int)p->ops.size() - 1;
}
bool known_value(const Plan* p, int v) { return v >= 0 && v < p->n_values; }
}  // namespace

GIBBS_EXPORT int gibbs_plan_op_half(void* plan, int norm, int body) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_norm(norm) || !p->has_body(body)) { gibbs_fail("plan: a half of norm %d and body %d: no such part", norm, body); return -1; }
  return append(p, Plan::OP_HALF, norm, body, -1, false);
}
GIBBS_EXPORT int gibbs_plan_op_norm(void* plan, int norm) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_norm(norm)) { gibbs_fail("plan: no norm %d", norm); return -1; }
  return append(p, Plan::OP_NORM, norm, -1, -1, true);
}
GIBBS_EXPORT int gibbs_plan_op_rows(void* plan, int body, int value) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_body(body) || !known_value(p, value)) { gibbs_fail("plan: body %d of value %d: no such part or value", body, value); return -1; }
  return append(p, Plan::OP_ROWS, -1, body, value, true);
}
GIBBS_EXPORT int gibbs_plan_op_body(void* plan, int body, int value) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_body(body) || !known_value(p, value)) { gibbs_fail("plan: body %d of value %d: no such part or value", body, value); return -1; }
  return append(p, Plan::OP_BODY, -1, body, value, true);
}
GIBBS_EXPORT int gibbs_plan_op_add(void* plan, int value) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!known_value(p, value)) { gibbs_fail("plan: no value %d to add", value); return -1; }
  return append(p, Plan::OP_ADD, -1, -1, value, false);
}
GIBBS_EXPORT int gibbs_plan_op_drop(void* plan, int value) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!known_value(p, value)) { gibbs_fail("plan: no value %d to drop", value); return -1; }
  return append(p, Plan::OP_DROP, -1, -1, value, false);
}
GIBBS_EXPORT int gibbs_plan_op_norm_delta(void* plan, int norm, int value) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_norm(norm) || !known_value(p, value)) { gibbs_fail("plan: norm %d of value %d: no such part or value", norm, value); return -1; }
  return append(p, Plan::OP_NORM_DELTA, norm, -1, value, true);
}
GIBBS_EXPORT int gibbs_plan_op_add_normed(void* plan, int norm, int value) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_norm(norm) || !known_value(p, value)) { gibbs_fail("plan: norm %d of value %d: no such part or value", norm, value); return -1; }
  return append(p, Plan::OP_ADD_NORMED, norm, -1, value, false);
}
GIBBS_EXPORT int gibbs_plan_op_streams_norm(void* plan, int norm, int hyper) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_norm(norm) || !p->has_hyper(hyper)) { gibbs_fail("plan: norm %d of hyper-connection %d: no such part", norm, hyper); return -1; }
  return append(p, Plan::OP_STREAMS_NORM, norm, hyper, -1, true);
}
GIBBS_EXPORT int gibbs_plan_op_streams_add(void* plan, int hyper, int value) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_hyper(hyper) || !known_value(p, value)) { gibbs_fail("plan: hyper-connection %d of value %d: no such part or value", hyper, value); return -1; }
  return append(p, Plan::OP_STREAMS_ADD, -1, hyper, value, false);
}
GIBBS_EXPORT int gibbs_plan_op_reinject(void* plan) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  p->reinjects = true;
  return append(p, Plan::OP_REINJECT, -1, -1, -1, false);
}
GIBBS_EXPORT int gibbs_plan_tail(void* plan, int norm) {
  Plan* p = open_plan(plan);
  if (!p) return -1;
  if (!p->has_norm(norm)) { gibbs_fail("plan: no norm %d for the tail", norm); return -1; }
  p->tail = norm;
  return 0;
}
GIBBS_EXPORT int gibbs_plan_op_count(const void* plan) { return plan ? (int)((const Plan*)plan)->ops.size() : 0; }

// ------------------------------------------------------------------------------------------------- running it
// Bytes of workspace that this step needs (its operands as for gibbs_plan_step; nothing is queued).
GIBBS_EXPORT long gibbs_plan_workspace(const void* plan, const GibbsStepArgs* args) {
  if (check_args((const Plan*)plan, args, true)) return -1;
  GibbsStepArgs dry = *args;
  dry.workspace = nullptr;
  Exec e(*(const Plan*)plan, dry);
  e.run();
  return e.status ? -1 : e.arena.peak;
}

// Queues the whole step on args->stream; logits of the wanted rows land in args->logits.
GIBBS_EXPORT int gibbs_plan_step(const void* plan, const GibbsStepArgs* args) {
  if (check_args((const Plan*)plan, args, true)) return 1;
  GIBBS_REQUIRE(args->workspace, "step: no workspace");
  Exec e(*(const Plan*)plan, *args);
  e.run();
  ((const Plan*)plan)->last_fused = e.fused_halves;
  return e.status;
}
GIBBS_EXPORT int gibbs_plan_last_fused(const void* plan) { return plan ? ((const Plan*)plan)->last_fused : 0; }

GIBBS_EXPORT long gibbs_plan_body_forward(const void* plan, int body, const GibbsStepArgs* args, const void* h, long* out_offset,
                                          int* parts) {
  const Plan* p = (const Plan*)plan;
  if (check_args(p, args, false)) return -1;
  if (!p->has_body(body)) return gibbs_fail("plan: no body %d", body), -1;
  const int g = p->bodies[body]->cache_group();
  if (g >= 0 && !(g < args->n_groups && args->tables && args->tables[g] && args->widths[g] > 0)) return gibbs_fail("body: no block table for cache group %d", g), -1;
  Exec e(*p, *args);
  Pending delta = p->bodies[body]->general(e, (void*)h);
  e.mix_now();
  if (e.status) return -1;
  if (e.dry) return e.arena.peak;
  *out_offset = (char*)delta.data - (char*)args->workspace;
  *parts = delta.parts;
  return 0;
}
GIBBS_EXPORT long gibbs_plan_norm_forward(const void* plan, int norm, const GibbsStepArgs* args, float* x, const void* delta,
                                          int delta_parts, const int* rows, int n_out, long* out_offset) {
  const Plan* p = (const Plan*)plan;
  if (check_args(p, args, false)) return -1;
  if (!p->has_norm(norm)) return gibbs_fail("plan: no norm %d", norm), -1;
  Exec e(*p, *args);
  Pending pending{(void*)delta, delta ? std::max(delta_parts, 1) : 0};
  void* out = p->norms[norm]->run(e, x, pending, rows, n_out);
  if (e.status) return -1;
  if (e.dry) return e.arena.peak;
  *out_offset = (char*)out - (char*)args->workspace;
  return 0;
}

// ------------------------------------------------------------------------------------------------- the rules, for callers of single kernels
GIBBS_EXPORT int gibbs_rule_skinny_splits(int n_out, int inner, int want_blocks, int features, int min_k) {
  return skinny_splits(n_out, inner, want_blocks > 0 ? want_blocks : 512, features > 0 ? features : 16, min_k > 0 ? min_k : 1024);
}
GIBBS_EXPORT void gibbs_rule_decode_splits(int n_rows, int nkv, int group, int max_seq, int hd, int page_size, int kind,
                                           int* n_splits, int* waves) {
  decode_splits(n_rows, nkv, group, max_seq, hd, page_size, kind, n_splits, waves);
}
GIBBS_EXPORT int gibbs_rule_prefill_splits(long n_tiles, int nh, int max_seq, int window) {
  return prefill_splits(n_tiles, nh, max_seq, window);
}
GIBBS_EXPORT long gibbs_rule_prefill_tiles(int rows, int reqs) { return prefill_tiles(rows, reqs); }
GIBBS_EXPORT int gibbs_rule_prefill_heads(int rows, int reqs, int nh, int nkv, int hd, int max_seq, int n_splits) {
  return prefill_heads(rows, reqs, nh, nkv, hd, max_seq, n_splits);
}
GIBBS_EXPORT int gibbs_rule_fused_rows(void) { return FUSED_ROWS; }

GIBBS_EXPORT int gibbs_linear_splits(int dtype, int n, int O, int I, long ldx, const void* x, const void* w, int out_f32,
                                     int partial_ok, int own_gemm) {
  return choose_linear(dtype == GIBBS_BF16, n, O, I, aligned_for_matrix_cores(x, ldx, w, I), out_f32, partial_ok, own_gemm).splits;
}
GIBBS_EXPORT int gibbs_linear(const void* x, long ldx, const void* w, const void* packed, void* y, int dtype, int n, int O,
                              int I, int out_f32, int partial_ok, int own_gemm, hipStream_t stream) {
  GIBBS_REQUIRE(x && w && y && n > 0 && O > 0 && I > 0 && ldx >= I, "linear: bad operands n=%d O=%d I=%d", n, O, I);
  GIBBS_REQUIRE(dtype == GIBBS_BF16 || (dtype == GIBBS_F32 && out_f32), "linear: the float32 path writes float32");
  const LinearChoice c = choose_linear(dtype == GIBBS_BF16, n, O, I, aligned_for_matrix_cores(x, ldx, w, I), out_f32, partial_ok, own_gemm);
  if (c.kernel == LIN_LIBRARY && gibbs_gemm_library_init()) return 1;
  return run_linear(c, x, ldx, Matrix{w, packed, O, I}, true, y, n, out_f32, stream);
}

GIBBS_EXPORT long gibbs_skinny_residual_workspace(int n, int O, int I) { return (long)residual_parts(n, O, I) * n * O; }
GIBBS_EXPORT int gibbs_skinny_residual_routed(const void* y, const void* w, long ldw, float* x, void* mirror, int n, int O, int I,
                                              float* workspace, hipStream_t stream) {
  GIBBS_REQUIRE(residual_parts(n, O, I) == 0 || workspace, "skinny_residual: these sizes leave partial sums and there is no workspace for them");
  return run_skinny_residual(y, w, ldw, x, mirror, n, O, I, workspace, stream);
}
