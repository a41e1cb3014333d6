// Paged KV append with per-page mean-key maintenance, and the bulk mean-key
// builder.  Both are byte movers: one 64-lane wave moves one 256-byte head row
// per instruction (4 bytes per lane), so every access is a full-row burst.
#include "kin_append.h"

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

// grid = ceil(batch*Hkv / 4) blocks of 256 threads; one wave per (sequence, head).
__global__ __launch_bounds__(256) void append_kernel(AppendParams p) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= p.batch * p.num_kv_heads) return;
  const int b = item / p.num_kv_heads, h = item - b * p.num_kv_heads;
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  if (n_pages <= 0) return;
  uint32_t* kbar_row = p.kbar ? p.kbar + (((int64_t)b * p.kbar_pages + (n_pages - 1)) * p.num_kv_heads + h) * (kHeadDim / 2)
                              : nullptr;
  append_token_row(p.k + (int64_t)item * (kHeadDim / 2), p.v + (int64_t)item * (kHeadDim / 2), p.kv_cache, kbar_row,
                   p.page_indices[e - 1], p.last_page_len[b], n_pages, p.kbar_pages, h, p.num_kv_heads, p.num_pages, lane);
}

// grid = batch * Hkv * ceil(kbar_pages / 16) blocks (flat, so it is not bound by
// the 65535 limit of grid.y); 16 lanes per (sequence, head, logical page), a lane
// owns 8 columns of all 16 key rows: 16 loads of 16 B in flight per lane, and the
// same fp32 sum in slot order that page_mean_dword() makes, so a page's mean key
// is bit-identical whether it is built here or by the append that fills the page.
__global__ __launch_bounds__(256) void build_kbar_kernel(AppendParams p, int page_blocks) {
  const int sub = threadIdx.x >> 4, c16 = threadIdx.x & 15;
  const int item = blockIdx.x / page_blocks;
  const int page = (blockIdx.x - item * page_blocks) * 16 + sub;
  const int b = item / p.num_kv_heads, h = item - b * p.num_kv_heads;
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  if (n_pages <= 0) return;
  const int n_full = (p.last_page_len[b] >= kPageSize) ? n_pages : n_pages - 1;
  if (page >= n_full || page >= p.kbar_pages) return;
  const int64_t pid = p.page_indices[s + page];
  if (pid < 0 || pid >= p.num_pages) return;
  const int row_stride = p.num_kv_heads * (kHeadDim / 2);  // dwords per token row
  const int64_t page_dwords = 2LL * kPageSize * row_stride;
  const u32x4* kplane = reinterpret_cast<const u32x4*>(p.kv_cache + pid * page_dwords + h * (kHeadDim / 2)) + c16;
  u32x4 x[kPageSize];
#pragma unroll
  for (int t = 0; t < kPageSize; ++t) x[t] = __builtin_nontemporal_load(kplane + (int64_t)t * (row_stride / 4));
  float acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = 0.f;
#pragma unroll
  for (int t = 0; t < kPageSize; ++t) {
    acc[0] += bf16_lo(x[t].x); acc[1] += bf16_hi(x[t].x);
    acc[2] += bf16_lo(x[t].y); acc[3] += bf16_hi(x[t].y);
    acc[4] += bf16_lo(x[t].z); acc[5] += bf16_hi(x[t].z);
    acc[6] += bf16_lo(x[t].w); acc[7] += bf16_hi(x[t].w);
  }
  const float inv = 1.0f / kPageSize;
  u32x4 m;
  m.x = f32_to_bf16(acc[0] * inv) | (f32_to_bf16(acc[1] * inv) << 16);
  m.y = f32_to_bf16(acc[2] * inv) | (f32_to_bf16(acc[3] * inv) << 16);
  m.z = f32_to_bf16(acc[4] * inv) | (f32_to_bf16(acc[5] * inv) << 16);
  m.w = f32_to_bf16(acc[6] * inv) | (f32_to_bf16(acc[7] * inv) << 16);
  reinterpret_cast<u32x4*>(p.kbar + (((int64_t)b * p.kbar_pages + page) * p.num_kv_heads + h) * (kHeadDim / 2))[c16] = m;
}

// ---- ragged multi-token append ------------------------------------------------
struct RaggedAppendParams {
  const uint32_t* k;  // [nnz, Hkv, 64] dwords
  const uint32_t* v;
  const int32_t* append_indptr;  // [batch + 1]
  uint32_t* kv_cache;
  uint32_t* kbar;  // may be null
  const int32_t* page_indices;
  const int32_t* page_indptr;
  const int32_t* last_page_len;
  int batch, num_kv_heads, kbar_pages;
  int64_t nnz;
  int64_t num_pages;
};

// Sequence that owns appended row `row`: the last b with append_indptr[b] <= row.
__device__ __forceinline__ int owner_of_row(const int32_t* indptr, int batch, int64_t row) {
  int lo = 0, hi = batch;  // invariant: indptr[lo] <= row < indptr[hi] for a well-formed indptr
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)indptr[mid] <= row) lo = mid; else hi = mid;
  }
  return lo;
}

// grid = ceil(nnz*Hkv / 4) blocks of 256 threads; one wave per (appended row, head).
// The page table describes the cache after the append: row i of sequence b's n_b
// new rows lands at token position kv_len_b - n_b + i.
__global__ __launch_bounds__(256) void append_ragged_kernel(RaggedAppendParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= p.nnz * p.num_kv_heads) return;
  const int64_t row = item / p.num_kv_heads;
  const int h = (int)(item - row * p.num_kv_heads);
  const int b = owner_of_row(p.append_indptr, p.batch, row);
  const int a0 = p.append_indptr[b], a1 = p.append_indptr[b + 1];
  if (row < a0 || row >= a1) return;  // malformed indptr
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  const int last = p.last_page_len[b];
  if (n_pages <= 0 || last < 1 || last > kPageSize) return;
  const int64_t kv_len = (int64_t)(n_pages - 1) * kPageSize + last;
  const int64_t pos = kv_len - (a1 - a0) + (row - a0);
  if (pos < 0) return;  // more rows than the sequence holds: out of contract
  const int64_t pid = p.page_indices[s + (int)(pos / kPageSize)];
  if (pid < 0 || pid >= p.num_pages) return;
  const int slot = (int)(pos % kPageSize);
  const int row_stride = p.num_kv_heads * (kHeadDim / 2);
  const int64_t page_dwords = 2LL * kPageSize * row_stride;
  uint32_t* kplane = p.kv_cache + pid * page_dwords + h * (kHeadDim / 2);
  uint32_t* vplane = kplane + (int64_t)kPageSize * row_stride;
  const int64_t src = item * (kHeadDim / 2) + lane;
  kplane[(int64_t)slot * row_stride + lane] = p.k[src];
  vplane[(int64_t)slot * row_stride + lane] = p.v[src];
}

// Mean keys of the pages an append completed.  grid = batch*Hkv*page_blocks blocks;
// one wave per (sequence, head, j-th page touched by the append).  Runs after
// append_ragged_kernel on the same stream.
__global__ __launch_bounds__(256) void refresh_kbar_kernel(RaggedAppendParams p, int page_blocks) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x / page_blocks;
  const int j = (blockIdx.x - item * page_blocks) * 4 + (threadIdx.x >> 6);
  const int b = item / p.num_kv_heads, h = item - b * p.num_kv_heads;
  const int n_new = p.append_indptr[b + 1] - p.append_indptr[b];
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  const int last = p.last_page_len[b];
  if (n_new <= 0 || n_pages <= 0 || last < 1 || last > kPageSize) return;
  const int64_t kv_len = (int64_t)(n_pages - 1) * kPageSize + last;
  const int64_t first_pos = kv_len - n_new;
  if (first_pos < 0) return;
  const int64_t page = first_pos / kPageSize + j;         // j-th page the append wrote into
  if (page >= kv_len / kPageSize || page >= p.kbar_pages) return;  // not full (or no slot for its mean key)
  const int64_t pid = p.page_indices[s + (int)page];
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
  const int page_blocks = (kbar_pages + 15) / 16;
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

int kin_append_paged_kv_ragged(const kin_bf16_t* k, const kin_bf16_t* v, const int32_t* append_indptr,
                               kin_bf16_t* kv_cache, kin_bf16_t* kbar, const int32_t* page_indices,
                               const int32_t* page_indptr, const int32_t* last_page_len, int batch, int64_t nnz,
                               int max_append_len, int num_kv_heads, int head_dim, int page_size,
                               int64_t num_pages, int kbar_pages, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_append_paged_kv_ragged";
  if (!k || !v || !append_indptr) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_append_args(fn, kv_cache, page_indices, page_indptr, last_page_len, batch, num_kv_heads,
                             head_dim, page_size, num_pages, kbar_pages, kbar != nullptr);
  if (st) return st;
  if (nnz < 0 || max_append_len < 0 || max_append_len > nnz)
    return fail(KIN_ERR_BAD_SHAPE, "%s: nnz=%lld and max_append_len=%d must satisfy 0 <= max_append_len <= nnz", fn,
                (long long)nnz, max_append_len);
  if (!aligned16(k) || !aligned16(v) || (kbar && !aligned16(kbar)))
    return fail(KIN_ERR_MISALIGNED, "%s: k, v and kbar must be 16-byte aligned", fn);
  if (batch == 0 || nnz == 0) return KIN_OK;
  const int64_t items = nnz * num_kv_heads;
  const int64_t blocks = (items + 3) / 4;
  // pages one sequence's append can touch: a partial page in front plus the pages its rows fill
  const int page_blocks = ((max_append_len + kPageSize - 1) / kPageSize + 1 + 3) / 4;
  const int64_t lists = (int64_t)batch * num_kv_heads;
  if (blocks > 0x7fffffffLL || lists * page_blocks > 0x7fffffffLL)
    return fail(KIN_ERR_UNSUPPORTED, "%s: problem too large for one launch", fn);
  RaggedAppendParams p;
  p.k = reinterpret_cast<const uint32_t*>(k);
  p.v = reinterpret_cast<const uint32_t*>(v);
  p.append_indptr = append_indptr;
  p.kv_cache = reinterpret_cast<uint32_t*>(kv_cache);
  p.kbar = reinterpret_cast<uint32_t*>(kbar);
  p.page_indices = page_indices;
  p.page_indptr = page_indptr;
  p.last_page_len = last_page_len;
  p.batch = batch;
  p.num_kv_heads = num_kv_heads;
  p.kbar_pages = kbar_pages;
  p.nnz = nnz;
  p.num_pages = num_pages;
  hipStream_t s = static_cast<hipStream_t>(stream);
  append_ragged_kernel<<<(unsigned)blocks, 256, 0, s>>>(p);
  st = check_hip(hipGetLastError(), "append_ragged_kernel launch");
  if (st || !kbar) return st;
  refresh_kbar_kernel<<<(unsigned)(lists * page_blocks), 256, 0, s>>>(p, page_blocks);
  return check_hip(hipGetLastError(), "refresh_kbar_kernel launch");
}

}  // extern "C"
