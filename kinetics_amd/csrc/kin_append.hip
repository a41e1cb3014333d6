// Paged KV append with per-page mean-key maintenance (one token per sequence, or
// a ragged run of tokens per sequence), and the bulk mean-key builder.  All are
// byte movers.
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
  int batch, num_kv_heads, kbar_pages, page_size;
  int head_dim;  // 128 or 64: these kernels move bytes and take it at run time
  int64_t num_pages;
  const int32_t* slot_ids;  // kbar row block of each sequence (null: the sequence's own index)
  int num_slots;
};

// grid = ceil(batch*Hkv / 4) blocks of 256 threads; one wave per (sequence, head).
template <bool F16>
__global__ __launch_bounds__(256) void append_kernel(AppendParams p) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= p.batch * p.num_kv_heads) return;
  const int b = item / p.num_kv_heads, h = item - b * p.num_kv_heads;
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  if (n_pages <= 0) return;
  const int kb = kbar_block_of(p.slot_ids, p.num_slots, b);
  const int row_dwords = p.head_dim / 2;
  uint32_t* kbar_row = (p.kbar && kb >= 0) ? p.kbar + kbar_row_index(kb, h, n_pages - 1, p.num_kv_heads, p.kbar_pages) * row_dwords
                                           : nullptr;
  const uint32_t* k_row = p.k + (int64_t)item * row_dwords;
  const uint32_t* v_row = p.v + (int64_t)item * row_dwords;
  if (p.head_dim == kHeadDimSmall)
    append_token_row<F16, kHeadDimSmall>(k_row, v_row, p.kv_cache, kbar_row, p.page_indices[e - 1], p.last_page_len[b], n_pages,
                                         p.kbar_pages, h, p.num_kv_heads, p.num_pages, lane, p.page_size);
  else
    append_token_row<F16, kHeadDim>(k_row, v_row, p.kv_cache, kbar_row, p.page_indices[e - 1], p.last_page_len[b], n_pages,
                                    p.kbar_pages, h, p.num_kv_heads, p.num_pages, lane, p.page_size);
}

// grid = batch * Hkv * page_blocks blocks (flat, so it is not bound by
// the 65535 limit of grid.y); head_dim / 8 lanes (16 or 8) per (sequence, head, logical page), so a
// block covers 16 or 32 pages; a lane
// owns 8 columns of all 16 key rows: 16 loads of 16 B in flight per lane, and the
// same fp32 sum in slot order that page_mean_dword() makes, so a page's mean key
// is bit-identical whether it is built here or by the append that fills the page.
template <bool F16>
__global__ __launch_bounds__(256) void build_kbar_kernel(AppendParams p, int page_blocks) {
  const int lpp = p.head_dim / 8;  // lanes per page = 16-byte chunks of a head row
  const int sub = threadIdx.x / lpp, c16 = threadIdx.x - sub * lpp;
  const int item = blockIdx.x / page_blocks;
  const int page = (blockIdx.x - item * page_blocks) * (256 / lpp) + sub;
  const int b = item / p.num_kv_heads, h = item - b * p.num_kv_heads;
  const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
  const int n_pages = e - s;
  if (n_pages <= 0) return;
  const int n_full = (p.last_page_len[b] >= p.page_size) ? n_pages : n_pages - 1;
  if (page >= n_full || page >= p.kbar_pages) return;
  const int64_t pid = p.page_indices[s + page];
  if (pid < 0 || pid >= p.num_pages) return;
  const int kb = kbar_block_of(p.slot_ids, p.num_slots, b);
  if (kb < 0) return;
  const int row_stride = p.num_kv_heads * (p.head_dim / 2);  // dwords per token row
  const int64_t page_dwords = 2LL * p.page_size * row_stride;
  const u32x4* kplane = reinterpret_cast<const u32x4*>(p.kv_cache + pid * page_dwords + h * (p.head_dim / 2)) + c16;
  const u32x4 m = page_mean_16B<F16>(kplane, row_stride / 4, p.page_size);
  // Streaming store: the mean keys are not read again by this launch.  (Stores that leave the caches while the
  // read stream is saturated cost about five times their bytes: 2.1 GB of them take the config-1 build from
  // 4.95 to 6.97 ms with a plain store, 6.55 ms with this one; writing them in 64 KiB bursts changes nothing.)
  __builtin_nontemporal_store(m, reinterpret_cast<u32x4*>(p.kbar + kbar_row_index(kb, h, page, p.num_kv_heads, p.kbar_pages) * (p.head_dim / 2)) + c16);
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
  int batch, num_kv_heads, kbar_pages, page_size;
  int head_dim;  // 128 or 64
  int64_t nnz;
  int64_t num_pages;
  const int32_t* slot_ids;  // kbar row block of each sequence (null: the sequence's own index)
  int num_slots;
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

constexpr int kRaggedRows = 32;  // appended token rows one workgroup moves

// grid = ceil(nnz / kRaggedRows) blocks of 256 threads.  A token's K row over all
// heads is one contiguous run of Hkv * head_dim * 2 bytes in k[] and in its page slot (and
// likewise V), so the workgroup's rows are moved as 16-byte chunks, several in
// flight per thread; where each row goes is worked out once per row (threads
// 0..31) and handed over in LDS.  The page table describes the cache after the
// append: row i of sequence b's n_b new rows lands at token position
// kv_len_b - n_b + i.
__global__ __launch_bounds__(256) void append_ragged_kernel(RaggedAppendParams p) {
  __shared__ int64_t dst16[kRaggedRows];  // K destination of the row in 16-byte units, -1: skip
  const int tid = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * kRaggedRows;
  const int rows_here = (int)min((int64_t)kRaggedRows, p.nnz - row0);
  const int cpr = p.num_kv_heads * (p.head_dim / 8);  // 16-byte chunks per token row (all heads)
  const int P = p.page_size;
  if (tid < kRaggedRows) {
    int64_t dst = -1;
    const int64_t row = row0 + tid;
    if (tid < rows_here) {
      const int b = owner_of_row(p.append_indptr, p.batch, row);
      const int a0 = p.append_indptr[b], a1 = p.append_indptr[b + 1];
      const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
      const int n_pages = e - s;
      const int last = p.last_page_len[b];
      // rows outside their sequence's range (malformed indptr) or contract are skipped
      if (row >= a0 && row < a1 && n_pages > 0 && last >= 1 && last <= P) {
        const int64_t kv_len = (int64_t)(n_pages - 1) * P + last;
        const int64_t pos = kv_len - (a1 - a0) + (row - a0);
        if (pos >= 0) {
          const int64_t pid = p.page_indices[s + (int)(pos / P)];
          if (pid >= 0 && pid < p.num_pages) dst = (pid * 2 * P + (pos % P)) * cpr;
        }
      }
    }
    dst16[tid] = dst;
  }
  __syncthreads();
  const u32x4* ksrc = reinterpret_cast<const u32x4*>(p.k) + row0 * cpr;
  const u32x4* vsrc = reinterpret_cast<const u32x4*>(p.v) + row0 * cpr;
  u32x4* cache = reinterpret_cast<u32x4*>(p.kv_cache);
  const int64_t v_plane = (int64_t)P * cpr;  // V plane of a page follows its K plane
  const int total = rows_here * cpr;
  constexpr int kU = 4;
  for (int base = tid; base < total; base += 256 * kU) {
    u32x4 kk[kU], vv[kU];
    int64_t d[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const int c = base + u * 256;
      d[u] = -1;
      if (c < total) {
        const int r = c / cpr;
        const int64_t dr = dst16[r];
        if (dr >= 0) d[u] = dr + (c - r * cpr);
        kk[u] = __builtin_nontemporal_load(ksrc + c);
        vv[u] = __builtin_nontemporal_load(vsrc + c);
      }
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (d[u] >= 0) {
        cache[d[u]] = kk[u];
        cache[d[u] + v_plane] = vv[u];
      }
    }
  }
}

// Mean keys of the pages an append completed: the pages that received an appended
// row in their last slot.  Same grid and row bookkeeping as append_ragged_kernel
// (so its cost follows the number of appended rows, whatever their split over the
// sequences); 16 lanes per (completed page, head).  Runs after
// append_ragged_kernel on the same stream.
template <bool F16>
__global__ __launch_bounds__(256) void refresh_kbar_kernel(RaggedAppendParams p) {
  __shared__ int64_t src16[kRaggedRows];  // K plane of the page a row completed, in 16-byte units; -1: none
  __shared__ int64_t dst16[kRaggedRows];  // its mean-key row for head 0, in 16-byte units (head h: + h * kbar_pages rows)
  const int tid = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * kRaggedRows;
  const int rows_here = (int)min((int64_t)kRaggedRows, p.nnz - row0);
  const int cpr = p.num_kv_heads * (p.head_dim / 8);
  const int P = p.page_size;
  if (tid < kRaggedRows) {
    int64_t src = -1, dst = 0;
    const int64_t row = row0 + tid;
    if (tid < rows_here) {
      const int b = owner_of_row(p.append_indptr, p.batch, row);
      const int a0 = p.append_indptr[b], a1 = p.append_indptr[b + 1];
      const int s = p.page_indptr[b], e = p.page_indptr[b + 1];
      const int n_pages = e - s;
      const int last = p.last_page_len[b];
      if (row >= a0 && row < a1 && n_pages > 0 && last >= 1 && last <= P) {
        const int64_t kv_len = (int64_t)(n_pages - 1) * P + last;
        const int64_t pos = kv_len - (a1 - a0) + (row - a0);
        const int64_t page = pos / P;
        if (pos >= 0 && pos % P == P - 1 && page < p.kbar_pages) {
          const int64_t pid = p.page_indices[s + (int)page];
          const int kb = kbar_block_of(p.slot_ids, p.num_slots, b);
          if (pid >= 0 && pid < p.num_pages && kb >= 0) {
            src = pid * 2 * P * cpr;
            dst = kbar_row_index(kb, 0, (int)page, p.num_kv_heads, p.kbar_pages) * (p.head_dim / 8);
          }
        }
      }
    }
    src16[tid] = src;
    dst16[tid] = dst;
  }
  __syncthreads();
  const int lpp = p.head_dim / 8;  // lanes per (completed page, head) = 16-byte chunks of a head row
  const int sub = tid / lpp, c16 = tid - sub * lpp;
  const u32x4* cache = reinterpret_cast<const u32x4*>(p.kv_cache);
  u32x4* kbar = reinterpret_cast<u32x4*>(p.kbar);
  for (int pair = sub; pair < rows_here * p.num_kv_heads; pair += 256 / lpp) {
    const int r = pair / p.num_kv_heads, h = pair - r * p.num_kv_heads;
    const int64_t src = src16[r];
    if (src < 0) continue;
    const u32x4 m = page_mean_16B<F16>(cache + src + h * lpp + c16, cpr, P);
    kbar[dst16[r] + (int64_t)h * p.kbar_pages * lpp + c16] = m;
  }
}

static int check_append_args(const char* fn, const void* kv_cache, const void* page_indices,
                             const void* page_indptr, const void* last_page_len, int batch, int num_kv_heads,
                             int head_dim, int page_size, int64_t num_pages, int kbar_pages, bool has_kbar,
                             const int32_t* slot_ids, int num_slots) {
  if (slot_ids && num_slots < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_slots=%d must be >= 1 when slot_ids is given", fn, num_slots);
  if (!kv_cache || !page_indices || !page_indptr || !last_page_len)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_common_dims(fn, batch, num_kv_heads, num_kv_heads, head_dim, page_size, true);
  if (st) return st;
  if (num_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_pages=%lld must be >= 1", fn, (long long)num_pages);
  if (has_kbar && kbar_pages < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: kbar_pages=%d must be >= 1 when kbar is given", fn, kbar_pages);
  if (!aligned16(kv_cache)) return fail(KIN_ERR_MISALIGNED, "%s: kv_cache is not 16-byte aligned", fn);
  return KIN_OK;
}

}  // namespace kin

extern "C" {

static int append_impl(const char* fn, bool f16, const uint16_t* k, const uint16_t* v, uint16_t* kv_cache, uint16_t* kbar,
                       const int32_t* page_indices, const int32_t* page_indptr, const int32_t* last_page_len,
                       int batch, int num_kv_heads, int head_dim, int page_size, int64_t num_pages,
                       int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  using namespace kin;
  if (!k || !v) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_append_args(fn, kv_cache, page_indices, page_indptr, last_page_len, batch, num_kv_heads,
                             head_dim, page_size, num_pages, kbar_pages, kbar != nullptr, slot_ids, num_slots);
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
  p.page_size = page_size;
  p.head_dim = head_dim;
  p.num_pages = num_pages;
  p.slot_ids = slot_ids;
  p.num_slots = slot_ids ? num_slots : batch;
  const int64_t items = (int64_t)batch * num_kv_heads;
  const unsigned blocks = (unsigned)((items + 3) / 4);
  if (f16) append_kernel<true><<<blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(p);
  else append_kernel<false><<<blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(p);
  return check_hip(hipGetLastError(), "append_kernel launch");
}

int kin_append_paged_kv(const kin_bf16_t* k, const kin_bf16_t* v, kin_bf16_t* kv_cache, kin_bf16_t* kbar,
                        const int32_t* page_indices, const int32_t* page_indptr, const int32_t* last_page_len,
                        int batch, int num_kv_heads, int head_dim, int page_size, int64_t num_pages,
                        int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  return append_impl("kin_append_paged_kv", false, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, batch,
                     num_kv_heads, head_dim, page_size, num_pages, kbar_pages, slot_ids, num_slots, stream);
}

int kin_append_paged_kv_f16(const kin_f16_t* k, const kin_f16_t* v, kin_f16_t* kv_cache, kin_f16_t* kbar,
                            const int32_t* page_indices, const int32_t* page_indptr, const int32_t* last_page_len,
                            int batch, int num_kv_heads, int head_dim, int page_size, int64_t num_pages,
                            int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  return append_impl("kin_append_paged_kv_f16", true, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, batch,
                     num_kv_heads, head_dim, page_size, num_pages, kbar_pages, slot_ids, num_slots, stream);
}

static int build_kbar_impl(const char* fn, bool f16, const uint16_t* kv_cache, uint16_t* kbar, const int32_t* page_indices,
                           const int32_t* page_indptr, const int32_t* last_page_len, int batch, int num_kv_heads,
                           int head_dim, int page_size, int64_t num_pages, int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  using namespace kin;
  if (!kbar) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_append_args(fn, kv_cache, page_indices, page_indptr, last_page_len, batch, num_kv_heads,
                             head_dim, page_size, num_pages, kbar_pages, true, slot_ids, num_slots);
  if (st) return st;
  if (!aligned16(kbar)) return fail(KIN_ERR_MISALIGNED, "%s: kbar must be 16-byte aligned", fn);
  if (batch == 0) return KIN_OK;
  const int64_t items = (int64_t)batch * num_kv_heads;
  const int pages_per_block = 256 / (head_dim / 8);
  const int page_blocks = (kbar_pages + pages_per_block - 1) / pages_per_block;
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
  p.page_size = page_size;
  p.head_dim = head_dim;
  p.num_pages = num_pages;
  p.slot_ids = slot_ids;
  p.num_slots = slot_ids ? num_slots : batch;
  if (f16) build_kbar_kernel<true><<<(unsigned)(items * page_blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(p, page_blocks);
  else build_kbar_kernel<false><<<(unsigned)(items * page_blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(p, page_blocks);
  return check_hip(hipGetLastError(), "build_kbar_kernel launch");
}

int kin_build_kbar(const kin_bf16_t* kv_cache, kin_bf16_t* kbar, const int32_t* page_indices,
                   const int32_t* page_indptr, const int32_t* last_page_len, int batch, int num_kv_heads,
                   int head_dim, int page_size, int64_t num_pages, int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  return build_kbar_impl("kin_build_kbar", false, kv_cache, kbar, page_indices, page_indptr, last_page_len, batch, num_kv_heads,
                         head_dim, page_size, num_pages, kbar_pages, slot_ids, num_slots, stream);
}

int kin_build_kbar_f16(const kin_f16_t* kv_cache, kin_f16_t* kbar, const int32_t* page_indices,
                       const int32_t* page_indptr, const int32_t* last_page_len, int batch, int num_kv_heads,
                       int head_dim, int page_size, int64_t num_pages, int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  return build_kbar_impl("kin_build_kbar_f16", true, kv_cache, kbar, page_indices, page_indptr, last_page_len, batch,
                         num_kv_heads, head_dim, page_size, num_pages, kbar_pages, slot_ids, num_slots, stream);
}

static int append_ragged_impl(const char* fn, bool f16, const uint16_t* k, const uint16_t* v, const int32_t* append_indptr,
                              uint16_t* kv_cache, uint16_t* kbar, const int32_t* page_indices,
                              const int32_t* page_indptr, const int32_t* last_page_len, int batch, int64_t nnz,
                              int max_append_len, int num_kv_heads, int head_dim, int page_size,
                              int64_t num_pages, int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  using namespace kin;
  if (!k || !v || !append_indptr) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_append_args(fn, kv_cache, page_indices, page_indptr, last_page_len, batch, num_kv_heads,
                             head_dim, page_size, num_pages, kbar_pages, kbar != nullptr, slot_ids, num_slots);
  if (st) return st;
  if (nnz < 0 || max_append_len < 0 || max_append_len > nnz)
    return fail(KIN_ERR_BAD_SHAPE, "%s: nnz=%lld and max_append_len=%d must satisfy 0 <= max_append_len <= nnz", fn,
                (long long)nnz, max_append_len);
  if (!aligned16(k) || !aligned16(v) || (kbar && !aligned16(kbar)))
    return fail(KIN_ERR_MISALIGNED, "%s: k, v and kbar must be 16-byte aligned", fn);
  if (batch == 0 || nnz == 0) return KIN_OK;
  const int64_t blocks = (nnz + kRaggedRows - 1) / kRaggedRows;
  if (blocks > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: problem too large for one launch", fn);
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
  p.page_size = page_size;
  p.head_dim = head_dim;
  p.nnz = nnz;
  p.num_pages = num_pages;
  p.slot_ids = slot_ids;
  p.num_slots = slot_ids ? num_slots : batch;
  hipStream_t s = static_cast<hipStream_t>(stream);
  append_ragged_kernel<<<(unsigned)blocks, 256, 0, s>>>(p);
  st = check_hip(hipGetLastError(), "append_ragged_kernel launch");
  if (st || !kbar) return st;
  if (f16) refresh_kbar_kernel<true><<<(unsigned)blocks, 256, 0, s>>>(p);
  else refresh_kbar_kernel<false><<<(unsigned)blocks, 256, 0, s>>>(p);
  return check_hip(hipGetLastError(), "refresh_kbar_kernel launch");
}

int kin_append_paged_kv_ragged(const kin_bf16_t* k, const kin_bf16_t* v, const int32_t* append_indptr,
                               kin_bf16_t* kv_cache, kin_bf16_t* kbar, const int32_t* page_indices,
                               const int32_t* page_indptr, const int32_t* last_page_len, int batch, int64_t nnz,
                               int max_append_len, int num_kv_heads, int head_dim, int page_size,
                               int64_t num_pages, int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  return append_ragged_impl("kin_append_paged_kv_ragged", false, k, v, append_indptr, kv_cache, kbar, page_indices, page_indptr,
                            last_page_len, batch, nnz, max_append_len, num_kv_heads, head_dim, page_size, num_pages,
                            kbar_pages, slot_ids, num_slots, stream);
}

int kin_append_paged_kv_ragged_f16(const kin_f16_t* k, const kin_f16_t* v, const int32_t* append_indptr,
                                   kin_f16_t* kv_cache, kin_f16_t* kbar, const int32_t* page_indices,
                                   const int32_t* page_indptr, const int32_t* last_page_len, int batch, int64_t nnz,
                                   int max_append_len, int num_kv_heads, int head_dim, int page_size,
                                   int64_t num_pages, int kbar_pages, const int32_t* slot_ids, int num_slots, kin_stream_t stream) {
  return append_ragged_impl("kin_append_paged_kv_ragged_f16", true, k, v, append_indptr, kv_cache, kbar, page_indices,
                            page_indptr, last_page_len, batch, nnz, max_append_len, num_kv_heads, head_dim, page_size,
                            num_pages, kbar_pages, slot_ids, num_slots, stream);
}

}  // extern "C"
