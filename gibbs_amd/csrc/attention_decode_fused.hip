// Decode attention straight from the raw fused q, k, v projection: q/k norm, rotation and the write of
// the new key and value to their pages happen in the attention kernel.  The kernel and its launcher are
// in attention_decode.h.
#include "attention_decode.h"

// qkv: [N, ld] bfloat16, raw projection (q heads, k heads, v heads) of N decoded tokens, one per request.
GIBBS_EXPORT int gibbs_attention_decode_fused(const void* qkv, void* kpages, void* vpages, void* out, float* partial,
                                              const float* q_gain, const float* k_gain, float eps,
                                              const float* inv_freq, int rot, int variant, const float* cs_table,
                                              int table_len, const int* pos, const int* row_req, const int* table, int max_pages, int page_size,
                                              int num_pages, int n_rows, int nh, int nkv, int hd, long ld, long ldo,
                                              float scale, int window, int n_splits, int waves, int kind, int max_keys, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention_decode_fused: bad sizes rows=%d heads=%d kv=%d hd=%d", n_rows, nh, nkv, hd);
  GIBBS_REQUIRE(nh % nkv == 0, "attention_decode_fused: %d heads are not a multiple of %d kv heads", nh, nkv);
  GIBBS_REQUIRE(hd % 16 == 0 && hd <= 256, "attention_decode_fused: head size %d must be a multiple of 16 up to 256", hd);
  GIBBS_REQUIRE(ld % 8 == 0 && ((uintptr_t)qkv % 16) == 0 && ld >= (long)(nh + 2 * nkv) * hd, "attention_decode_fused: qkv rows must be 16-byte aligned and hold q, k and v");
  GIBBS_REQUIRE(ldo >= (long)nh * hd, "attention_decode_fused: output rows shorter than heads * hd");
  GIBBS_REQUIRE(!inv_freq || (rot > 0 && rot % 16 == 0 && rot <= hd), "attention_decode_fused: rotary_dim %d must be a multiple of 16 within the head size %d", rot, hd);
  GIBBS_REQUIRE(variant == 0 || variant == 1, "attention_decode_fused: unknown rotation variant %d", variant);
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0, "attention_decode_fused: bad cache geometry");
  GIBBS_REQUIRE(n_splits >= 1 && n_splits <= 65535 && (n_splits == 1 || partial), "attention_decode_fused: %d key slices need a workspace", n_splits);
  if (n_rows == 0) return 0;
  DecodeArgs a{};
  a.pos = pos; a.row_req = row_req; a.table = table; a.max_pages = max_pages; a.page_size = page_size;
  a.num_pages = num_pages; a.nh = nh; a.nkv = nkv; a.hd = hd; a.ldq = ld; a.ldo = ldo; a.scale = scale;
  a.window = window; a.n_splits = n_splits;
  a.q_gain = q_gain; a.k_gain = k_gain; a.eps = eps; a.inv_freq = inv_freq; a.rot = rot; a.variant = variant;
  a.cs_table = (const float2*)cs_table; a.table_len = cs_table ? table_len : 0;
  return run_decode<true>((const bf16*)qkv, (bf16*)kpages, (bf16*)vpages, (bf16*)out, partial, a, n_rows, waves, kind, max_keys, stream);
}
