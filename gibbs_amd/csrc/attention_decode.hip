// Decode attention over prepared queries (rotated, normed q; the cache already holds the new key).
// The kernel and its launcher are in attention_decode.h.
#include "attention_decode.h"

// Floats of workspace that n_splits > 1 needs.
GIBBS_EXPORT long gibbs_attention_decode_workspace(int n_rows, int nh, int hd, int n_splits) {
  return n_splits > 1 ? (long)n_rows * nh * n_splits * (hd + 2) : 0;
}

// q: [N, >= nh*hd] bfloat16 (row stride ldq); pages: [num_pages, nkv, page_size, hd] bfloat16;
// out: [N, nh*hd] bfloat16 (row stride ldo); partial: workspace (see above) or null with n_splits 1.
// kind: 0 choose, 1 vector units, 2 matrix cores; max_keys: a bound on the keys of any row (0: the block table's width).
GIBBS_EXPORT int gibbs_attention_decode(const void* q, const void* kpages, const void* vpages, void* out, float* partial,
                                        const int* pos, const int* row_req, const int* table, int max_pages,
                                        int page_size, int num_pages, int n_rows, int nh, int nkv, int hd, long ldq,
                                        long ldo, float scale, int window, int n_splits, int waves, int kind, int max_keys, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention_decode: bad sizes rows=%d heads=%d kv=%d hd=%d", n_rows, nh, nkv, hd);
  GIBBS_REQUIRE(nh % nkv == 0, "attention_decode: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd % 8 == 0 && hd <= 256, "attention_decode: head size %d must be a multiple of 8 up to 256", hd);
  GIBBS_REQUIRE(ldq % 8 == 0 && ((uintptr_t)q % 16) == 0, "attention_decode: q rows must be 16-byte aligned");
  GIBBS_REQUIRE(ldq >= (long)nh * hd && ldo >= (long)nh * hd, "attention_decode: row strides shorter than heads * hd");
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_decode: bad cache geometry");
  GIBBS_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || partial), "attention_decode: %d key slices need a workspace", n_splits);
  if (n_rows == 0) return 0;
  DecodeArgs a{};
  a.pos = pos; a.row_req = row_req; a.table = table; a.max_pages = max_pages; a.page_size = page_size;
  a.num_pages = num_pages; a.nh = nh; a.nkv = nkv; a.hd = hd; a.ldq = ldq; a.ldo = ldo; a.scale = scale;
  a.window = window; a.n_splits = n_splits;
  // the kernel only reads the pages here
  return run_decode<false>((const bf16*)q, (bf16*)kpages, (bf16*)vpages, (bf16*)out, partial, a, n_rows, waves, kind, max_keys, stream);
}

