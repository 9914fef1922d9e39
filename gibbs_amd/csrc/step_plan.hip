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
  if (!own_gemm && !out_f32) return {LIN_LIBRARY, 1};    // (the library writes bfloat16 only)
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
  void* linear(const void* x, const Matrix& m, int n, bool out_f32, bool partial_ok, bool use_packed, int* parts);
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

struct Plan {
  int dtype = GIBBS_BF16;   // activations, matrices and cache pages
  int hidden = 0, vocab = 0;
  const void* table = nullptr;
  int table_dtype = GIBBS_BF16;
  Matrix head;
  int tail = -1;            // the norm in front of the head
  int fused_rows = FUSED_ROWS;   // steps of at most this many decoded tokens take the fused decode kernels
  int own_gemm = 0;         // products above the few-row kernels' range: 0 the library's, 1 the tiled kernel
  std::vector<std::unique_ptr<NormPart>> norms;
  std::vector<std::unique_ptr<Body>> bodies;
  enum { OP_HALF, OP_NORM, OP_BODY, OP_ADD, OP_DROP };
  struct Op {
    int kind, norm, body, value;   // value: what a body reads, an add adds, a drop drops
    int result;                    // the value that a norm or a body makes
  };
  std::vector<Op> ops;
  int n_values = 0;
  mutable int last_fused = 0;
  bool has_norm(int i) const { return i >= 0 && i < (int)norms.size(); }
  bool has_body(int i) const { return i >= 0 && i < (int)bodies.size(); }
};

Exec::Exec(const Plan& plan, const GibbsStepArgs& args)
    : p(plan), a(args), arena(args.workspace, args.workspace_bytes, args.workspace == nullptr), dry(args.workspace == nullptr) {
  esize = p.dtype == GIBBS_BF16 ? 2 : 4;
  bf16_run = p.dtype == GIBBS_BF16;
  few_rows = bf16_run && a.n_rows <= std::min(p.fused_rows, FUSED_ROWS);
  fused_step = few_rows && a.max_q == 1;
}

void* Exec::linear(const void* x, const Matrix& m, int n, bool out_f32, bool partial_ok, bool use_packed, int* parts) {
  const LinearChoice c = choose_linear(bf16_run, n, m.O, m.I, aligned_for_matrix_cores(x, m.I, m.w, m.I), out_f32, partial_ok, p.own_gemm);
  const long elem = !bf16_run || out_f32 || c.splits > 1 ? 4 : 2;
  void* y = take((long)c.splits * n * m.O * elem);
  RUN(*this, run_linear(c, x, m.I, m, use_packed, y, n, out_f32, a.stream));
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
struct RmsNorm : NormPart {
  const float* gain = nullptr;   // null: folded into the matrices that follow
  float eps = 0.f;
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
  int cache_group() const override { return group; }
  bool fast() const { return !slopes && !hook; }   // the fast kernels know rotations only (or no encoding at all)
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
  void decode_attention(Exec& e, const void* q, long ldq, int n_rows, const int* pos, const int* row_req, void* o) const {
    int n_splits, waves;
    decode_splits(n_rows, nkv, nh / nkv, e.a.max_seq, hd, page_size, 0, &n_splits, &waves);
    float* partial = n_splits > 1 ? (float*)e.take(gibbs_attention_decode_workspace(n_rows, nh, hd, n_splits) * 4) : nullptr;
    RUN(e, gibbs_attention_decode(q, kpages, vpages, o, partial, pos, row_req, e.table(group), e.width(group), page_size, num_pages,
                                  n_rows, nh, nkv, hd, ldq, (long)nh * hd, scale, window, n_splits, waves, 0, e.a.max_seq, e.a.stream));
    e.give(partial);
  }
  // q/k norm, rotation and the cache write of the step's rows (a mixer that reads another's cache writes nothing)
  void prepare_rows(Exec& e, void* raw, long ldq) const {
    const int N = e.a.n_rows, kv = owns ? nkv : 0;
    const int* table = e.table(group);
    const int width = e.width(group);
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
    const long ldq = (long)(nh + 2 * kv) * hd, ldo = (long)nh * hd;
    void* att;
    if (e.bf16_run && a.max_q == 1 && raw_ok()) {
      att = attend_decoded(e, raw);
    } else {
      prepare_rows(e, raw, ldq);
      const int* table = e.table(group);
      const int width = e.width(group);
      att = e.take((long)N * ldo * e.esize);
      const bool fast_bf16 = e.bf16_run && !slopes;   // (the fast kernels take no score bias)
      if (fast_bf16 && a.max_q > 1 && hd % 16 == 0 && hd <= 128) {
        // decoded tokens at the head of the batch (where the scheduler puts them) take the kernel that splits
        // their keys (a row of its own in the matrix-core kernel would walk its cache alone); the rest the
        // matrix-core kernel
        const int lead = a.lead_single >= 2 ? a.lead_single : 0;
        if (lead) decode_attention(e, raw, ldq, lead, a.pos, a.row_req, att);
        const int rows = N - lead, reqs = a.n_req - lead;
        const int n_splits = a.max_seq > 0 ? prefill_splits(prefill_tiles(rows, reqs), nh, a.max_seq, window) : 1;
        float* partial = n_splits > 1 ? (float*)e.take(gibbs_attention_decode_workspace(N, nh, hd, n_splits) * 4) : nullptr;
        RUN(e, gibbs_attention_prefill(raw, kpages, vpages, att, partial, a.cu + lead, a.ctx + lead, table + (long)lead * width, reqs,
                                       width, page_size, num_pages, rows, nh, nkv, hd, ldq, ldo, scale, window, n_splits, lead,
                                       prefill_heads(rows, reqs, nh, nkv, hd, a.max_seq, n_splits), a.stream));
        e.give(partial);
      } else if (fast_bf16 && a.max_q == 1 && hd % 8 == 0) {
        decode_attention(e, raw, ldq, N, a.pos, a.row_req, att);
      } else {
        RUN(e, gibbs_attention_plain(raw, kpages, vpages, att, e.p.dtype, a.pos, a.row_req, table, width, page_size, num_pages, N, nh,
                                     nkv, hd, ldq, ldo, scale, window, slopes, a.stream));
      }
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
  bool fusable(bool) const override { return gate_up.I % 8 == 0 && F % 8 == 0; }   // (rows one by one: any few rows)
  void fused(Exec& e, float eps, float* x, void* mirror) const override {
    const int N = e.a.n_rows, H = gate_up.I;
    void* y = e.take((long)N * F * 2);
    RUN(e, gibbs_skinny_glu(mirror, gate_up_packed2 ? gate_up_packed2 : gate_up.w, y, N, F, H, H, gate_up_packed2 ? 0 : H, F, 1, eps, act,
                            e.a.stream));
    e.skinny_residual(y, down, x, mirror);
    e.give(y);
  }
  Pending general(Exec& e, void* h) const override {
    const int N = e.a.n_rows;
    void* gu = e.linear(h, gate_up, N, false, false, false, nullptr);
    void* y = e.take((long)N * F * e.esize);
    RUN(e, gibbs_glu(gu, y, e.p.dtype, N, F, act, e.a.stream));
    e.give(gu);
    Pending delta;
    delta.data = e.linear(y, down, N, false, true, true, &delta.parts);
    e.give(y);
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
void Exec::run() {
  const int N = a.n_rows, H = p.hidden;
  float* x = a.x_in;
  void* mirror = few_rows ? a.mirror_in : nullptr;
  if (!x) {
    x = (float*)take((long)N * H * 4);
    mirror = few_rows ? take((long)N * H * 2) : nullptr;
    RUN(*this, gibbs_embed(p.table, p.table_dtype, a.ids, x, mirror, N, H, p.vocab, a.stream));
  }
  Pending pending;
  std::vector<void*> rows(p.n_values, nullptr);       // normed rows by value
  std::vector<Pending> deltas(p.n_values);           // deltas by value
  const bool whole = a.n_ops == 0;
  const int first = whole ? 0 : a.first_op, last = whole ? (int)p.ops.size() : a.first_op + a.n_ops;
  for (int i = first; i < last && ok(); ++i) {
    const Plan::Op& op = p.ops[i];
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
      case Plan::OP_ADD:
        settle(x, pending);
        pending = deltas[op.value];
        deltas[op.value] = Pending{};
        break;
      case Plan::OP_DROP:
        give(rows[op.value]);
        give(deltas[op.value].data);
        rows[op.value] = nullptr;
        deltas[op.value] = Pending{};
        break;
    }
  }
  if (whole && a.n_logits > 0 && ok()) {
    void* h = p.norms[p.tail]->run(*this, x, pending, a.logit_rows, a.n_logits);
    linear_into(h, p.head, a.n_logits, true, true, a.logits);   // the head: float32 logits straight into the caller's buffer
    give(h);
  }
  if (a.settle) settle(x, pending);
  give(pending.data);
  for (void* r : rows) give(r);
  for (Pending& d : deltas) give(d.data);
  give(mirror);      // (buffers of the caller's are not the arena's: giving them back does nothing)
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
  if (a->n_ops == 0 && a->n_logits > 0) {
    GIBBS_REQUIRE(p->has_norm(p->tail) && p->head.w, "step: logits are wanted and the plan has no final norm or no head");
    GIBBS_REQUIRE(a->workspace == nullptr || a->logits, "step: logits are wanted and there is no buffer for them");
  }
  const int first = a->n_ops ? a->first_op : 0, last = a->n_ops ? a->first_op + a->n_ops : (int)p->ops.size();
  for (int i = first; i < last; ++i) {
    const Plan::Op& op = p->ops[i];
    if (op.kind != Plan::OP_HALF && op.kind != Plan::OP_BODY) continue;
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
  t->slopes = slopes; t->hook = hook; t->hook_user = hook_user;
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
