// Decode attention over prepared queries (rotated, normed q; the cache already holds the new key).
// The kernel and its launcher are in attention_decode.h.
#include "attention_decode.h"
#include "attention_decode_api.h"
#include <mutex>

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


// ---------------------------------------------------------------------------------------------
// The entry point that allocates nothing: the slices' partial results live in a file-scope device
// array.  In host code the array's name is a stand-in, not a device address: the address on each
// GPU is asked for once, with that GPU current, and only that pointer is ever handed to a kernel.
constexpr long STATIC_FLOATS = 2l << 20;
constexpr int STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) float g_slices_scratch[STATIC_FLOATS];
static float* g_slices_ptr[STATIC_MAX_DEVICES];
static std::mutex g_slices_lock;

GIBBS_EXPORT long gibbs_attention_decode_static_capacity(void) { return STATIC_FLOATS; }

// The current GPU's copy of the array (null after gibbs_fail).
static float* slices_scratch_of_current_device() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) {
    gibbs_fail("attention_decode_static: no current GPU among the first %d (%s)", STATIC_MAX_DEVICES, hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(g_slices_lock);
  if (!g_slices_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_slices_scratch));
    if (e != hipSuccess || !p) {
      gibbs_fail("attention_decode_static: the address of the scratch array on GPU %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_slices_ptr[dev] = (float*)p;
  }
  return g_slices_ptr[dev];
}

GIBBS_EXPORT int gibbs_attention_decode_static(const void* q, const void* kpages, const void* vpages, void* out,
                                               const int* pos, const int* row_req, const int* table, int max_pages,
                                               int page_size, int num_pages, int n_rows, int nh, int nkv, int hd,
                                               long ldq, long ldo, float scale, int window, int n_splits, int waves,
                                               int kind, int max_keys, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && hd > 0 && n_splits >= 1, "attention_decode_static: bad sizes rows=%d heads=%d hd=%d slices=%d", n_rows, nh, hd, n_splits);
  const long need = gibbs_attention_decode_workspace(n_rows, nh, hd, n_splits);
  GIBBS_REQUIRE(need <= STATIC_FLOATS, "attention_decode_static: %d rows x %d heads x %d slices of head size %d need %ld floats of scratch, the array holds %ld", n_rows, nh, n_splits, hd, need, STATIC_FLOATS);
  float* partial = nullptr;
  if (n_splits > 1) {
    partial = slices_scratch_of_current_device();
    if (!partial) return 1;
  }
  return gibbs_attention_decode(q, kpages, vpages, out, partial, pos, row_req, table, max_pages, page_size, num_pages,
                                n_rows, nh, nkv, hd, ldq, ldo, scale, window, n_splits, waves, kind, max_keys, stream);
}
