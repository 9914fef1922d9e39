// The step of a whole model as one native call.
//
// When a model is bound, every part that knows how hands its weights, sizes and constants to a plan
// (gibbs_plan_*); gibbs_plan_step then runs one ragged batch through embedding, every run of the layer
// order, the final norm of the wanted rows and the head, choosing for each operation the kernel that the
// step's shape asks for (the few-row weight-streaming products and their fused epilogues for steps of
// decoded tokens, the library's or the tiled product above that, the matrix-core attention for prompt
// portions, the key-splitting one for decoded tokens, the plain kernels for float32 and odd sizes) and
// queueing everything on the caller's stream.  The host does no work per kernel beyond this function:
// a step of a hundred kernels costs it a few tens of microseconds, where a launch from an interpreter
// costs that much for every few kernels.  The reference's step is one native call as well
// (src/model/native.rs:78-83).
//
// Activations live in a workspace that the caller passes: the same function run "dry" (nothing queued)
// reports the bytes a step needs, so the caller can size the workspace before the real run.  Buffers are
// taken and given back in the order of the code below; kernels run in stream order, so a buffer that
// was given back can be handed out again at once.
//
// What is laid down here is the arrangement x += mixer(norm(x)); x += ffn(norm(x)) with an RMS norm, a
// gated short convolution or an attention over the paged cache as mixer and a gated dense feed-forward:
// the parts that the package itself brings.  A model with a part from elsewhere steps through the
// interpreter, part by part, over the same kernels.
#include "common.h"
#include "kernels.h"
#include <map>
#include <vector>

namespace {
constexpr int MAX_GROUPS = 8;

struct Matrix {
  const void* w = nullptr;       // [O, I] row-major in the run's compute type
  const void* packed = nullptr;  // the same in tile order (bfloat16 only), or null
  int O = 0, I = 0;
};
struct NormP {
  const float* gain = nullptr;   // null: folded into the matrices that follow
  float eps = 0.f;
};
struct ConvP {
  Matrix in, out;
  const void* in_packed3 = nullptr;   // in-projection packed in three row groups (B, C, x), for the fused kernel
  const float* taps = nullptr;
  const float* bias = nullptr;
  int C = 0, K = 0;
  float* state = nullptr;        // [slots, K - 1, C] float32
  long slot_stride = 0;
  int fusable = 0;
};
struct AttnP {
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
  int num_pages = 0, page_size = 0, group = 0, owns = 0, fusable = 0;
};
struct GluP {
  Matrix gate_up, down;
  const void* gate_up_packed2 = nullptr;   // gate and up packed as two row groups, for the fused kernel
  int F = 0, act = 0, fusable = 0;
};
enum { MIX_NONE = 0, MIX_CONV = 1, MIX_ATTENTION = 2 };
struct BlockP {
  NormP n1, n2;
  int mixer = MIX_NONE;
  ConvP conv;
  AttnP attn;
  GluP glu;
  bool has_glu = false;
};
struct Plan {
  int dtype = GIBBS_BF16;   // activations, matrices and cache pages
  int hidden = 0, vocab = 0;
  const void* table = nullptr;
  int table_dtype = GIBBS_BF16;
  Matrix head;
  NormP final_norm;
  int fused_rows = 64;      // steps of at most this many decoded tokens take the fused decode kernels
  int own_gemm = 0;         // products above the few-row kernels' range: 0 the library's, 1 the tiled kernel
  std::vector<BlockP> blocks;
  bool complete() const {
    for (const BlockP& b : blocks)
      if (b.mixer == MIX_NONE || !b.has_glu) return false;
    return true;
  }
};
}  // namespace

// One step's operands (the caller's integer metadata lives on the device already).
struct GibbsStepArgs {
  const int* ids;          // [n_rows]
  const int* pos;          // [n_rows]
  const int* row_req;      // [n_rows]
  const int* cu;           // [n_req + 1]
  const int* ctx;          // [n_req]
  const int* slot;         // [n_req]
  const int* logit_rows;   // [n_logits]
  const int* tables[MAX_GROUPS];   // per cache group: [n_req, widths[g]]
  int widths[MAX_GROUPS];
  int n_rows, n_req, n_logits, max_q, max_seq, lead_single;
  void* workspace;         // device memory for the step's activations
  long workspace_bytes;
  float* logits;           // [n_logits, vocab] float32 out
  hipStream_t stream;
  // A step that continues a captured decode loop: the rows' embeddings are there already (the end of the
  // previous step wrote them), as the float32 stream x_in [n_rows, hidden] and, for steps that take the fused
  // decode kernels, its bfloat16 mirror.  Null: the step embeds its ids itself.
  float* x_in;
  void* mirror_in;
};

namespace {
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

long ceil_div_l(long a, long b) { return (a + b - 1) / b; }

// Ranges of k that the few-row product is cut into so that at least `want_blocks` workgroups run (a
// workgroup owns `features` output features), each with at least `min_k` of k.
int skinny_splits(int n_out, int inner, int want_blocks = 512, int features = 16, int min_k = 1024) {
  const long blocks = ceil_div_l(n_out, features);
  const long s = std::max<long>(1, std::min<long>(ceil_div_l(want_blocks, blocks), inner / min_k));
  const long per = ceil_div_l(ceil_div_l(inner, s), 128) * 128;
  return (int)ceil_div_l(inner, per);
}

constexpr int MATRIX_SLICE_PAGES = 510;   // page ids of a key slice that the decode attention's matrix-core walk keeps in LDS

// (key slices per (row, kv head), waves per workgroup) of the decode attention: few rows get enough
// slices to give every compute unit two workgroups, but at least 256 keys to a slice on the matrix cores
// (64 on the vector units); rows and heads that fill the chip by themselves get none.
void decode_splits(int n_rows, int nkv, int group, int max_seq, int hd, int page_size, int* n_splits, int* waves) {
  const bool matrix = hd > 0 && hd % 16 == 0 && hd <= 128;
  const int gt = group >= 8 ? 8 : (group > 2 ? 4 : group);
  const long per_split = (long)n_rows * nkv * ceil_div_l(group, gt);
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

// Slices of the key tiles for the prompt attention: none while query tiles and heads fill the chip.
int prefill_splits(long n_tiles, int nh, int max_seq, int window) {
  const long blocks = std::max<long>(1, n_tiles * nh);
  const long keys = window > 0 ? std::min<long>(max_seq, window + 64) : max_seq;
  if (blocks >= 768 || keys < 8 * 64) return 1;
  return (int)std::max<long>(1, std::min<long>(std::min<long>(ceil_div_l(2048, blocks), keys / 256), 16));
}

struct Exec {
  const Plan& p;
  const GibbsStepArgs& a;
  Arena arena;
  bool dry;
  int status = 0;
  int esize;                  // bytes of an activation element
  bool bf16_run, fused_step;
  Exec(const Plan& plan, const GibbsStepArgs& args, bool dry_run)
      : p(plan), a(args), arena(args.workspace, args.workspace_bytes, dry_run), dry(dry_run) {
    esize = p.dtype == GIBBS_BF16 ? 2 : 4;
    bf16_run = p.dtype == GIBBS_BF16;
    fused_step = bf16_run && a.max_q == 1 && a.n_rows <= std::min(p.fused_rows, 64);
  }
  void* take(long bytes) {
    void* ptr = arena.take(bytes);
    if (!ptr && !status) status = gibbs_fail("step: the workspace of %ld bytes is too small", a.workspace_bytes);
    return ptr;
  }
  void give(void* ptr) { arena.give(ptr); }
  bool ok() const { return status == 0; }
// queues a kernel unless this is a dry run or an earlier call failed
#define RUN(call)                    \
  do {                               \
    if (!dry && status == 0 && (call)) status = 1; \
  } while (0)

  // y = x @ W^T in the precision of the run (see ops/linear.py for the choice; `out_f32`: float32 logits).
  // `partial_ok`: the caller takes float32 partial sums; `use_packed`: the few-row kernel may read the
  // tile-ordered copy.  Returns the buffer ([N, O], or [parts, N, O] float32 with *parts >= 2).
  void* linear(const void* x, const Matrix& m, int n, bool out_f32, bool partial_ok, bool use_packed, int* parts) {
    if (parts) *parts = 1;
    const int O = m.O, I = m.I;
    if (!bf16_run) {
      float* y = (float*)take((long)n * O * 4);
      RUN(gibbs_gemm_f32((const float*)x, (const float*)m.w, y, n, O, I, I, I, O, a.stream));
      return y;
    }
    const int out_dtype = out_f32 ? GIBBS_F32 : GIBBS_BF16;
    const long out_bytes = (long)n * O * (out_f32 ? 4 : 2);
    if (I % 8 || ((uintptr_t)x % 16) || ((uintptr_t)m.w % 16)) {
      void* y = take(out_bytes);
      RUN(gibbs_gemm_bf16_plain(x, m.w, y, out_dtype, n, O, I, I, I, O, a.stream));
      return y;
    }
    if (n <= 32) {
      const int splits = partial_ok ? skinny_splits(O, I) : 1;
      const bool packed = use_packed && m.packed;
      void* y = take(splits > 1 ? (long)splits * n * O * 4 : out_bytes);
      RUN(gibbs_gemm_skinny(x, packed ? m.packed : m.w, y, splits > 1 ? GIBBS_F32 : out_dtype, n, O, I, I, packed ? 0 : I, O,
                            splits, a.stream));
      if (parts) *parts = splits;
      return y;
    }
    void* y = take(out_bytes);
    if (!p.own_gemm && !out_f32) RUN(gibbs_gemm_library(x, m.w, y, n, O, I, I, I, O, a.stream));
    else RUN(gibbs_gemm_bf16(x, m.w, y, out_dtype, n, O, I, I, I, O, a.stream));
    return y;
  }

  // x += pending (if any); returns norm(x) of all rows (or of `rows`) in the activation type
  void* norm(float* x, Pending& pending, const NormP& n, const int* rows, int n_out) {
    const int H = p.hidden;
    void* out = take((long)n_out * H * esize);
    if (pending.parts >= 2)
      RUN(gibbs_add_partials_rmsnorm(x, (const float*)pending.data, pending.parts, (long)a.n_rows * H, n.gain, n.eps, out,
                                     p.dtype, rows, n_out, H, a.stream));
    else
      RUN(gibbs_add_rmsnorm(x, pending.data, n.gain, n.eps, out, p.dtype, rows, n_out, H, a.stream));
    give(pending.data);
    pending = Pending{};
    return out;
  }

  // adds what is pending and makes sure the bfloat16 mirror of x exists
  void with_mirror(float* x, Pending& pending, void** mirror) {
    if (pending.parts == 0 && *mirror) return;
    const long count = (long)a.n_rows * p.hidden;
    if (!*mirror) *mirror = take(count * 2);
    RUN(gibbs_residual_add(x, pending.data, pending.parts >= 2 ? GIBBS_F32 : (pending.parts == 1 ? p.dtype : 0),
                           std::max(pending.parts, 1), count, *mirror, count, a.stream));
    give(pending.data);
    pending = Pending{};
  }

  // x += y @ W^T with the mirror kept (the last product of a fused half of a layer)
  void skinny_residual(const void* y, const Matrix& m, float* x, void* mirror) {
    const int n = a.n_rows, O = m.O, I = m.I;
    if (n > 32 && I >= 4096) {
      // many rows, long inner size: workgroups take 64 features each and k is cut to fill the chip; the
      // partial sums are added to the stream by a second kernel
      const int splits = skinny_splits(O, I, 256, 64, 256);
      float* parts = (float*)take((long)splits * n * O * 4);
      RUN(gibbs_gemm_skinny(y, m.packed ? m.packed : m.w, parts, GIBBS_F32, n, O, I, I, m.packed ? 0 : I, O, splits, a.stream));
      RUN(gibbs_residual_add(x, parts, GIBBS_F32, splits, (long)n * O, mirror, (long)n * O, a.stream));
      give(parts);
      return;
    }
    RUN(gibbs_skinny_residual(y, m.packed ? m.packed : m.w, x, mirror, n, O, I, I, m.packed ? 0 : I, a.stream));
  }

  // ------------------------------------------------------------------------------------------- mixers
  void conv_fused(const ConvP& c, const NormP& n, float* x, void* mirror) {
    const int N = a.n_rows, H = p.hidden;
    void* y = take((long)N * c.C * 2);
    const void* w = c.in_packed3 ? c.in_packed3 : c.in.w;
    RUN(gibbs_skinny_conv(mirror, w, y, N, c.C, H, H, c.in_packed3 ? 0 : H, 1, n.eps, c.taps, c.bias, c.state, c.slot_stride,
                          a.slot, a.ctx, c.K, a.stream));
    skinny_residual(y, c.out, x, mirror);
    give(y);
  }
  Pending conv_general(const ConvP& c, void* h) {
    const int N = a.n_rows;
    void* bcx = linear(h, c.in, N, false, false, false, nullptr);
    void* y = take((long)N * c.C * esize);
    RUN(gibbs_shortconv(bcx, c.taps, c.bias, c.state, c.slot_stride, a.cu, a.ctx, a.slot, y, p.dtype, N, a.n_req, c.C, c.K,
                        a.stream));
    give(bcx);
    Pending out;
    out.data = linear(y, c.out, N, false, true, true, &out.parts);
    give(y);
    return out;
  }

  // A step of one token per request: row n is request n, and the attention need not look that up (a dependent
  // load less in front of its page ids).
  bool rows_are_requests() const { return a.max_q == 1 && a.n_rows == a.n_req; }

  // decoded tokens from the raw projection: q/k norm, rotation, the cache write and attention in one kernel
  void* attend_decoded(const AttnP& t, const void* qkv) {
    const int N = a.n_rows;
    int n_splits, waves;
    decode_splits(N, t.nkv, t.nh / t.nkv, a.max_seq, t.hd, t.page_size, &n_splits, &waves);
    float* partial = n_splits > 1 ? (float*)take(gibbs_attention_decode_workspace(N, t.nh, t.hd, n_splits) * 4) : nullptr;
    void* out = take((long)N * t.nh * t.hd * 2);
    RUN(gibbs_attention_decode_fused(qkv, t.kpages, t.vpages, out, partial, t.q_gain, t.k_gain, t.qk_eps, t.inv_freq, t.rot,
                                     t.variant, t.cos_sin, t.cos_sin ? t.table_len : 0, a.pos, rows_are_requests() ? nullptr : a.row_req, a.tables[t.group],
                                     a.widths[t.group], t.page_size, t.num_pages, N, t.nh, t.nkv, t.hd,
                                     (long)(t.nh + 2 * t.nkv) * t.hd, (long)t.nh * t.hd, t.scale, t.window, n_splits, waves, 0,
                                     a.max_seq, a.stream));
    give(partial);
    return out;
  }
  void attention_fused(const AttnP& t, const NormP& n, float* x, void* mirror) {
    const int N = a.n_rows, H = p.hidden;
    void* qkv = take((long)N * t.qkv.O * 2);
    RUN(gibbs_skinny_store(mirror, t.qkv_packed ? t.qkv_packed : t.qkv.w, qkv, N, t.qkv.O, H, H, t.qkv_packed ? 0 : H, t.qkv.O,
                           1, n.eps, a.stream));
    void* att = attend_decoded(t, qkv);
    give(qkv);
    skinny_residual(att, t.out, x, mirror);
    give(att);
  }
  void decode_attention(const AttnP& t, const void* q, long ldq, int n_rows, const int* pos, const int* row_req, void* out) {
    int n_splits, waves;
    decode_splits(n_rows, t.nkv, t.nh / t.nkv, a.max_seq, t.hd, t.page_size, &n_splits, &waves);
    float* partial = n_splits > 1 ? (float*)take(gibbs_attention_decode_workspace(n_rows, t.nh, t.hd, n_splits) * 4) : nullptr;
    RUN(gibbs_attention_decode(q, t.kpages, t.vpages, out, partial, pos, row_req, a.tables[t.group], a.widths[t.group],
                               t.page_size, t.num_pages, n_rows, t.nh, t.nkv, t.hd, ldq, (long)t.nh * t.hd, t.scale, t.window,
                               n_splits, waves, 0, a.max_seq, a.stream));
    give(partial);
  }
  Pending attention_general(const AttnP& t, void* h) {
    const int N = a.n_rows, nkv = t.owns ? t.nkv : 0;
    const long ldq = (long)(t.nh + 2 * nkv) * t.hd, ldo = (long)t.nh * t.hd;
    void* qkv = linear(h, t.qkv, N, false, false, false, nullptr);
    const bool rot16 = !t.inv_freq || t.rot % 16 == 0;
    void* att;
    if (t.owns && bf16_run && a.max_q == 1 && t.hd % 16 == 0 && t.hd <= 256 && rot16) {
      att = attend_decoded(t, qkv);
    } else {
      const int* table = a.tables[t.group];
      const int width = a.widths[t.group];
      RUN(gibbs_qk_rope_kv(qkv, t.owns ? t.kpages : nullptr, t.owns ? t.vpages : nullptr, p.dtype, t.q_gain, t.k_gain, t.qk_eps,
                           t.inv_freq, t.rot, t.variant, t.cos_sin, t.cos_sin && t.inv_freq ? t.table_len : 0, a.pos, a.row_req,
                           t.owns ? table : nullptr, t.owns ? width : 0, t.owns ? t.page_size : 0, t.owns ? t.num_pages : 0, N,
                           t.nh, nkv, t.hd, ldq, a.stream));
      att = take((long)N * ldo * esize);
      if (bf16_run && a.max_q > 1 && t.hd % 16 == 0 && t.hd <= 128) {
        // decoded tokens at the head of the batch (where the scheduler puts them) take the kernel that splits
        // their keys; the rest the matrix-core kernel
        const int lead = a.lead_single >= 2 ? a.lead_single : 0;
        if (lead) decode_attention(t, qkv, ldq, lead, a.pos, a.row_req, att);
        const int rows = N - lead, reqs = a.n_req - lead;
        const int n_splits = a.max_seq > 0 ? prefill_splits(ceil_div_l(rows, 64) + reqs / 2, t.nh, a.max_seq, t.window) : 1;
        float* partial = n_splits > 1 ? (float*)take(gibbs_attention_decode_workspace(N, t.nh, t.hd, n_splits) * 4) : nullptr;
        RUN(gibbs_attention_prefill(qkv, t.kpages, t.vpages, att, partial, a.cu + lead, a.ctx + lead, table + (long)lead * width,
                                    reqs, width, t.page_size, t.num_pages, rows, t.nh, t.nkv, t.hd, ldq, ldo, t.scale, t.window,
                                    n_splits, lead, a.stream));
        give(partial);
      } else if (bf16_run && a.max_q == 1 && t.hd % 8 == 0) {
        decode_attention(t, qkv, ldq, N, a.pos, a.row_req, att);
      } else {
        RUN(gibbs_attention_plain(qkv, t.kpages, t.vpages, att, p.dtype, a.pos, a.row_req, table, width, t.page_size,
                                  t.num_pages, N, t.nh, t.nkv, t.hd, ldq, ldo, t.scale, t.window, nullptr, a.stream));
      }
    }
    give(qkv);
    Pending out;
    out.data = linear(att, t.out, N, false, true, true, &out.parts);
    give(att);
    return out;
  }

  // ------------------------------------------------------------------------------------------- feed-forward
  void glu_fused(const GluP& g, const NormP& n, float* x, void* mirror) {
    const int N = a.n_rows, H = p.hidden;
    void* act = take((long)N * g.F * 2);
    RUN(gibbs_skinny_glu(mirror, g.gate_up_packed2 ? g.gate_up_packed2 : g.gate_up.w, act, N, g.F, H, H,
                         g.gate_up_packed2 ? 0 : H, g.F, 1, n.eps, g.act, a.stream));
    skinny_residual(act, g.down, x, mirror);
    give(act);
  }
  Pending glu_general(const GluP& g, void* h) {
    const int N = a.n_rows;
    void* gu = linear(h, g.gate_up, N, false, false, false, nullptr);
    void* act = take((long)N * g.F * esize);
    RUN(gibbs_glu(gu, act, p.dtype, N, g.F, g.act, a.stream));
    give(gu);
    Pending out;
    out.data = linear(act, g.down, N, false, true, true, &out.parts);
    give(act);
    return out;
  }

  // ------------------------------------------------------------------------------------------- the step
  void run() {
    const int N = a.n_rows, H = p.hidden;
    float* x = a.x_in;
    void* mirror = fused_step ? a.mirror_in : nullptr;
    if (!x) {
      x = (float*)take((long)N * H * 4);
      mirror = fused_step ? take((long)N * H * 2) : nullptr;
      RUN(gibbs_embed(p.table, p.table_dtype, a.ids, x, mirror, N, H, p.vocab, a.stream));
    }
    Pending pending;
    for (const BlockP& b : p.blocks) {
      const bool mixer_fused = fused_step && (b.mixer == MIX_CONV ? b.conv.fusable : b.attn.fusable);
      if (mixer_fused) {
        with_mirror(x, pending, &mirror);
        if (b.mixer == MIX_CONV) conv_fused(b.conv, b.n1, x, mirror);
        else attention_fused(b.attn, b.n1, x, mirror);
      } else {
        void* h = norm(x, pending, b.n1, nullptr, N);
        pending = b.mixer == MIX_CONV ? conv_general(b.conv, h) : attention_general(b.attn, h);
        give(h);
        give(mirror);
        mirror = nullptr;
      }
      if (fused_step && b.glu.fusable) {
        with_mirror(x, pending, &mirror);
        glu_fused(b.glu, b.n2, x, mirror);
      } else {
        void* h = norm(x, pending, b.n2, nullptr, N);
        pending = glu_general(b.glu, h);
        give(h);
        give(mirror);
        mirror = nullptr;
      }
      if (!ok()) return;
    }
    if (a.n_logits > 0) {
      void* h = norm(x, pending, p.final_norm, a.logit_rows, a.n_logits);
      const int M = a.n_logits, V = p.vocab;
      // the head: float32 logits straight into the caller's buffer
      if (!bf16_run) {
        RUN(gibbs_gemm_f32((const float*)h, (const float*)p.head.w, a.logits, M, V, H, H, H, V, a.stream));
      } else if (H % 8 || ((uintptr_t)h % 16) || ((uintptr_t)p.head.w % 16)) {
        RUN(gibbs_gemm_bf16_plain(h, p.head.w, a.logits, GIBBS_F32, M, V, H, H, H, V, a.stream));
      } else if (M <= 48) {   // (see ops/linear.py)
        RUN(gibbs_gemm_skinny(h, p.head.packed ? p.head.packed : p.head.w, a.logits, GIBBS_F32, M, V, H, H,
                              p.head.packed ? 0 : H, V, 1, a.stream));
      } else {
        RUN(gibbs_gemm_bf16(h, p.head.w, a.logits, GIBBS_F32, M, V, H, H, H, V, a.stream));
      }
      give(h);
    }
    give(pending.data);
    give(mirror);      // (buffers of the caller's are not the arena's: giving them back does nothing)
    give(x);
  }
#undef RUN
};

int check_args(const Plan* p, const GibbsStepArgs* a) {
  GIBBS_REQUIRE(p && a, "step: no plan or no operands");
  GIBBS_REQUIRE(p->complete(), "step: the plan has a block without a mixer or a feed-forward");
  GIBBS_REQUIRE(a->n_rows > 0 && a->n_req > 0 && a->n_logits >= 0 && a->max_q >= 1, "step: bad sizes rows=%d requests=%d wanted=%d", a->n_rows, a->n_req, a->n_logits);
  GIBBS_REQUIRE(a->lead_single >= 0 && a->lead_single <= a->n_req, "step: %d leading decoded tokens among %d requests", a->lead_single, a->n_req);
  for (const BlockP& b : p->blocks)
    if (b.mixer == MIX_ATTENTION)
      GIBBS_REQUIRE(a->tables[b.attn.group] && a->widths[b.attn.group] > 0, "step: no block table for cache group %d", b.attn.group);
  return 0;
}
}  // namespace

// ------------------------------------------------------------------------------------------------- building a plan
GIBBS_EXPORT void* gibbs_plan_create(int dtype, int hidden, int vocab, const void* table, int table_dtype, const void* head,
                                     const void* head_packed, const float* final_gain, float final_eps, int fused_rows,
                                     int own_gemm) {
  if ((dtype != GIBBS_BF16 && dtype != GIBBS_F32) || hidden <= 0 || vocab <= 0 || !table || !head) {
    gibbs_fail("plan: bad model sizes or no token table");
    return nullptr;
  }
  if (dtype == GIBBS_BF16 && !own_gemm && gibbs_gemm_library_init()) return nullptr;
  Plan* p = new Plan();
  p->dtype = dtype; p->hidden = hidden; p->vocab = vocab; p->table = table; p->table_dtype = table_dtype;
  p->head.w = head; p->head.packed = head_packed; p->head.O = vocab; p->head.I = hidden;
  p->final_norm = NormP{final_gain, final_eps};
  p->fused_rows = fused_rows; p->own_gemm = own_gemm;
  return p;
}
GIBBS_EXPORT void gibbs_plan_destroy(void* plan) { delete (Plan*)plan; }

// A new block (run of the layer order) with its two norms; its mixer and feed-forward follow.
GIBBS_EXPORT int gibbs_plan_add_block(void* plan, const float* gain1, float eps1, const float* gain2, float eps2) {
  Plan* p = (Plan*)plan;
  GIBBS_REQUIRE(p, "plan: null");
  BlockP b;
  b.n1 = NormP{gain1, eps1};
  b.n2 = NormP{gain2, eps2};
  p->blocks.push_back(b);
  return 0;
}

GIBBS_EXPORT int gibbs_plan_set_conv(void* plan, const void* w_in, const void* p_in3, const void* w_out, const void* p_out,
                                     const float* taps, const float* bias, int C, int K, float* state, long slot_stride,
                                     int fusable) {
  Plan* p = (Plan*)plan;
  GIBBS_REQUIRE(p && !p->blocks.empty() && p->blocks.back().mixer == MIX_NONE, "plan: no open block for a mixer");
  GIBBS_REQUIRE(w_in && w_out && taps && state && C > 0 && K >= 2 && slot_stride >= (long)(K - 1) * C, "plan: bad short convolution C=%d K=%d", C, K);
  BlockP& b = p->blocks.back();
  b.mixer = MIX_CONV;
  ConvP& c = b.conv;
  c.in = Matrix{w_in, nullptr, 3 * C, p->hidden}; c.in_packed3 = p_in3;
  c.out = Matrix{w_out, p_out, p->hidden, C};
  c.taps = taps; c.bias = bias; c.C = C; c.K = K; c.state = state; c.slot_stride = slot_stride; c.fusable = fusable;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_set_attention(void* plan, const void* w_qkv, const void* p_qkv, const void* w_out, const void* p_out,
                                          int nh, int nkv, int hd, float scale, int window, const float* q_gain,
                                          const float* k_gain, float qk_eps, const float* inv_freq, int rot, int variant,
                                          const float* cos_sin, int table_len, void* kpages, void* vpages, int num_pages,
                                          int page_size, int group, int owns, int fusable) {
  Plan* p = (Plan*)plan;
  GIBBS_REQUIRE(p && !p->blocks.empty() && p->blocks.back().mixer == MIX_NONE, "plan: no open block for a mixer");
  GIBBS_REQUIRE(w_qkv && w_out && nh > 0 && nkv > 0 && nh % nkv == 0 && hd > 0 && kpages && vpages && num_pages > 0 && page_size > 0,
                "plan: bad attention heads=%d kv=%d hd=%d", nh, nkv, hd);
  GIBBS_REQUIRE(group >= 0 && group < MAX_GROUPS, "plan: cache group %d beyond %d", group, MAX_GROUPS);
  BlockP& b = p->blocks.back();
  b.mixer = MIX_ATTENTION;
  AttnP& t = b.attn;
  t.qkv = Matrix{w_qkv, nullptr, (nh + (owns ? 2 * nkv : 0)) * hd, p->hidden}; t.qkv_packed = p_qkv;
  t.out = Matrix{w_out, p_out, p->hidden, nh * hd};
  t.nh = nh; t.nkv = nkv; t.hd = hd; t.scale = scale; t.window = window; t.q_gain = q_gain; t.k_gain = k_gain; t.qk_eps = qk_eps;
  t.inv_freq = inv_freq; t.rot = inv_freq ? rot : 0; t.variant = variant; t.cos_sin = cos_sin; t.table_len = table_len;
  t.kpages = kpages; t.vpages = vpages; t.num_pages = num_pages; t.page_size = page_size; t.group = group; t.owns = owns;
  t.fusable = fusable;
  return 0;
}

GIBBS_EXPORT int gibbs_plan_set_glu(void* plan, const void* w_gate_up, const void* p_gate_up2, const void* w_down,
                                    const void* p_down, int F, int act, int fusable) {
  Plan* p = (Plan*)plan;
  GIBBS_REQUIRE(p && !p->blocks.empty() && !p->blocks.back().has_glu, "plan: no open block for a feed-forward");
  GIBBS_REQUIRE(w_gate_up && w_down && F > 0, "plan: bad feed-forward width %d", F);
  BlockP& b = p->blocks.back();
  GluP& g = b.glu;
  g.gate_up = Matrix{w_gate_up, nullptr, 2 * F, p->hidden}; g.gate_up_packed2 = p_gate_up2;
  g.down = Matrix{w_down, p_down, p->hidden, F};
  g.F = F; g.act = act; g.fusable = fusable;
  b.has_glu = true;
  return 0;
}

// ------------------------------------------------------------------------------------------------- running it
// Bytes of workspace that this step needs (its operands as for gibbs_plan_step; nothing is queued).
GIBBS_EXPORT long gibbs_plan_workspace(const void* plan, const GibbsStepArgs* args) {
  if (check_args((const Plan*)plan, args)) return -1;
  Exec e(*(const Plan*)plan, *args, true);
  e.run();
  return e.status ? -1 : e.arena.peak;
}

// Queues the whole step on args->stream; logits of the wanted rows land in args->logits.
GIBBS_EXPORT int gibbs_plan_step(const void* plan, const GibbsStepArgs* args) {
  if (check_args((const Plan*)plan, args)) return 1;
  GIBBS_REQUIRE(args->workspace && args->workspace_bytes > 0 && ((uintptr_t)args->workspace % 256) == 0, "step: no workspace (or not 256-byte aligned)");
  GIBBS_REQUIRE(args->n_logits == 0 || args->logits, "step: logits are wanted and there is no buffer for them");
  Exec e(*(const Plan*)plan, *args, false);
  e.run();
  return e.status;
}
