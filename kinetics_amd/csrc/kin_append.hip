// Paged KV append with per-page mean-key maintenance, and the bulk mean-key
// builder.  Both are byte movers: one 64-lane wave moves one 256-byte head row
// per instruction (4 bytes per lane), so every access is a full-row burst.
#include "kin_common.h"

namespace kin {

struct AppendParams {
  const uint32_t* k;  // [batch, Hkv, 64] dwords (2 bf16 each)
  const uint32_t* v;
  uint32_t* kv_cache;
  uint32_t* kbar;  // may be null
  const int32_t* page_indices;
  const int32_t* page_indptr;
  const int32_t* last_page_len;
  int batch, num_kv_heads, kbar_pages;
  int64_t num_pages;
};

// Mean of the kPageSize key rows of one page for one head, for this lane's
// two columns.  `krow` points at slot 0 of the page's K plane for that head
// (in dwords); `row_stride` is in dwords.  Sum order is slot 0,1,...,15.
__device__ __forceinline__ uint32_t page_mean_dword(const uint32_t* krow, int row_stride, int lane) {
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int t = 0; t < kPageSize; ++t) {
    const uint32_t w = krow[(int64_t)t * row_stride + lane];
    s0 += bf16_lo(w);
    s1 += bf16_hi(w);
  }
  const float inv = 1.0f / kPageSize;
  return f32_to_bf16(s0 * inv) | (f32_to_bf16(s1 * inv) << 16);
}

// grid = ceil(batch*Hkv / 4) blocks of 256 threads; one wave per (sequence, head).
__global__ __launch_bounds__(256) void append_kernel(AppendParams p) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= p.batch * p.num_kv_heads) return;
  const int b = item / p.num_kv_heads, h = item - b * p.num_kv_heads;
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  if (n_pages <= 0) return;
  const int pos = p.last_page_len[b] - 1;
  const int64_t pid = p.page_indices[e - 1];
  // Metadata outside its contract would write outside the cache: skip the row.
  if (pos < 0 || pos >= kPageSize || pid < 0 || pid >= p.num_pages) return;

  const int row_stride = p.num_kv_heads * (kHeadDim / 2);           // dwords per token row
  const int64_t page_dwords = 2LL * kPageSize * row_stride;          // K plane + V plane
  uint32_t* kplane = p.kv_cache + pid * page_dwords + h * (kHeadDim / 2);
  uint32_t* vplane = kplane + (int64_t)kPageSize * row_stride;
  const int64_t src = (int64_t)item * (kHeadDim / 2) + lane;
  const uint32_t kw = p.k[src];
  const uint32_t vw = p.v[src];
  kplane[(int64_t)pos * row_stride + lane] = kw;
  vplane[(int64_t)pos * row_stride + lane] = vw;

  if (p.kbar != nullptr && pos == kPageSize - 1 && n_pages - 1 < p.kbar_pages) {
    // The page is now full.  Rows 0..14 come from the cache, row 15 is the one
    // just written (taken from the register so the result does not depend on
    // store visibility).
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int t = 0; t < kPageSize - 1; ++t) {
      const uint32_t w = kplane[(int64_t)t * row_stride + lane];
      s0 += bf16_lo(w);
      s1 += bf16_hi(w);
    }
    s0 += bf16_lo(kw);
    s1 += bf16_hi(kw);
    const float inv = 1.0f / kPageSize;
    const uint32_t m = f32_to_bf16(s0 * inv) | (f32_to_bf16(s1 * inv) << 16);
    p.kbar[(((int64_t)b * p.kbar_pages + (n_pages - 1)) * p.num_kv_heads + h) * (kHeadDim / 2) + lane] = m;
  }
}

// grid = batch * Hkv * ceil(kbar_pages / 4) blocks (flat, so it is not bound by
// the 65535 limit of grid.y); one wave per (sequence, head, logical page).
__global__ __launch_bounds__(256) void build_kbar_kernel(AppendParams p, int page_blocks) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x / page_blocks;
  const int page = (blockIdx.x - item * page_blocks) * 4 + (threadIdx.x >> 6);
  const int b = item / p.num_kv_heads, h = item - b * p.num_kv_heads;
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  if (n_pages <= 0) return;
  const int n_full = (p.last_page_len[b] >= kPageSize) ? n_pages : n_pages - 1;
  if (page >= n_full || page >= p.kbar_pages) return;
  const int64_t pid = p.page_indices[s + page];
  if (pid < 0 || pid >= p.num_pages) return;
  const int row_stride = p.num_kv_heads * (kHeadDim / 2);
  const int64_t page_dwords = 2LL * kPageSize * row_stride;
  const uint32_t* kplane = p.kv_cache + pid * page_dwords + h * (kHeadDim / 2);
  const uint32_t m = page_mean_dword(kplane, row_stride, lane);
  p.kbar[(((int64_t)b * p.kbar_pages + page) * p.num_kv_heads + h) * (kHeadDim / 2) + lane] = m;
}

static int check_append_args(const char* fn, const void* kv_cache, const void* page_indices,
                             const void* page_indptr, const void* last_page_len, int batch, int num_kv_heads,
                             int head_dim, int page_size, int64_t num_pages, int kbar_pages, bool has_kbar) {
  if (!kv_cache || !page_indices || !page_indptr || !last_page_len)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_common_dims(fn, batch, num_kv_heads, num_kv_heads, head_dim, page_size);
  if (st) return st;
  if (num_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_pages=%lld must be >= 1", fn, (long long)num_pages);
  if (has_kbar && kbar_pages < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: kbar_pages=%d must be >= 1 when kbar is given", fn, kbar_pages);
  if (!aligned16(kv_cache)) return fail(KIN_ERR_MISALIGNED, "%s: kv_cache is not 16-byte aligned", fn);
  return KIN_OK;
}

}  // namespace kin

extern "C" {

int kin_append_paged_kv(const kin_bf16_t* k, const kin_bf16_t* v, kin_bf16_t* kv_cache, kin_bf16_t* kbar,
                        const int32_t* page_indices, const int32_t* page_indptr, const int32_t* last_page_len,
                        int batch, int num_kv_heads, int head_dim, int page_size, int64_t num_pages,
                        int kbar_pages, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_append_paged_kv";
  if (!k || !v) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_append_args(fn, kv_cache, page_indices, page_indptr, last_page_len, batch, num_kv_heads,
                             head_dim, page_size, num_pages, kbar_pages, kbar != nullptr);
  if (st) return st;
  if (!aligned16(k) || !aligned16(v) || (kbar && !aligned16(kbar)))
    return fail(KIN_ERR_MISALIGNED, "%s: k, v and kbar must be 16-byte aligned", fn);
  if (batch == 0) return KIN_OK;
  AppendParams p;
  p.k = reinterpret_cast<const uint32_t*>(k);
  p.v = reinterpret_cast<const uint32_t*>(v);
  p.kv_cache = reinterpret_cast<uint32_t*>(kv_cache);
  p.kbar = reinterpret_cast<uint32_t*>(kbar);
  p.page_indices = page_indices;
  p.page_indptr = page_indptr;
  p.last_page_len = last_page_len;
  p.batch = batch;
  p.num_kv_heads = num_kv_heads;
  p.kbar_pages = kbar_pages;
  p.num_pages = num_pages;
  const int64_t items = (int64_t)batch * num_kv_heads;
  const unsigned blocks = (unsigned)((items + 3) / 4);
  append_kernel<<<blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(p);
  return check_hip(hipGetLastError(), "append_kernel launch");
}

int kin_build_kbar(const kin_bf16_t* kv_cache, kin_bf16_t* kbar, const int32_t* page_indices,
                   const int32_t* page_indptr, const int32_t* last_page_len, int batch, int num_kv_heads,
                   int head_dim, int page_size, int64_t num_pages, int kbar_pages, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_build_kbar";
  if (!kbar) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_append_args(fn, kv_cache, page_indices, page_indptr, last_page_len, batch, num_kv_heads,
                             head_dim, page_size, num_pages, kbar_pages, true);
  if (st) return st;
  if (!aligned16(kbar)) return fail(KIN_ERR_MISALIGNED, "%s: kbar must be 16-byte aligned", fn);
  if (batch == 0) return KIN_OK;
  const int64_t items = (int64_t)batch * num_kv_heads;
  const int page_blocks = (kbar_pages + 3) / 4;
  if (items * page_blocks > 0x7fffffffLL)
    return fail(KIN_ERR_UNSUPPORTED, "%s: batch*num_kv_heads*kbar_pages too large for one launch", fn);
  AppendParams p;
  p.k = nullptr;
  p.v = nullptr;
  p.kv_cache = const_cast<uint32_t*>(reinterpret_cast<const uint32_t*>(kv_cache));
  p.kbar = reinterpret_cast<uint32_t*>(kbar);
  p.page_indices = page_indices;
  p.page_indptr = page_indptr;
  p.last_page_len = last_page_len;
  p.batch = batch;
  p.num_kv_heads = num_kv_heads;
  p.kbar_pages = kbar_pages;
  p.num_pages = num_pages;
  build_kbar_kernel<<<(unsigned)(items * page_blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(p, page_blocks);
  return check_hip(hipGetLastError(), "build_kbar_kernel launch");
}

}  // extern "C"
