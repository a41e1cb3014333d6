// Paged attention for one decode token per sequence (sparse page lists from
// the selector, or the full page table for the dense baseline), plus the
// split-K merge.  One 256-thread workgroup per (sequence, KV head, split); the
// per-list work is attend_list() in kin_attend.h.  HBM-bound: every K/V byte is
// read exactly once.
#include "kin_attend.h"

namespace kin {

struct DecodeParams {
  const uint16_t* q;
  const uint16_t* kv;
  const int32_t* page_ids;       // sel_pages, or page_indices for dense
  const int32_t* list_indptr;    // dense: page_indptr [batch+1]; sparse: null
  const int32_t* list_count;     // sparse: sel_count [batch*Hkv]; dense: null
  const int32_t* last_page_len;  // [batch]
  uint16_t* out;
  float* lse;     // may be null
  float* ws_o;    // [batch*Hq, splits, 128] fp32, splits > 1 only
  float* ws_lse;  // [batch*Hq, splits]      fp32 (log2 domain)
  int batch, num_q_heads, num_kv_heads, group;
  int list_stride, num_splits;
  int first_page_offset;  // padding slots at the start of list entry 0
  int page_size;
  int rotate;  // attend_rotates(lists)
  int64_t num_pages;
  float scale_log2;  // sm_scale * log2(e)
};

template <int NG, bool F16, int HD = kHeadDim>
__global__ __launch_bounds__(256, 2) void paged_decode_kernel(DecodeParams p) {
  constexpr int kRowB = HD * 2;  // bytes of a head row
  __shared__ __attribute__((aligned(16))) unsigned char lds[attend_lds_bytes(4)];
  __shared__ float sm_m[4][4 * NG];
  __shared__ float sm_l[4][4 * NG];

  const int split = blockIdx.y;
  int b, h;
  if (!xcd_list_of(blockIdx.x, p.batch, p.num_kv_heads, b, h)) return;
  const int list = b * p.num_kv_heads + h;
  const int G = p.group;

  const int32_t* __restrict__ pl;
  int n;
  if (p.list_indptr) {
    const int s = p.list_indptr[b];
    pl = p.page_ids + s;
    n = p.list_indptr[b + 1] - s;
  } else {
    pl = p.page_ids + (int64_t)list * p.list_stride;
    n = min(p.list_count[list], p.list_stride);  // a count beyond the row would run into the next list
  }
  n = max(n, 0);
  const int per_split = (n + p.num_splits - 1) / p.num_splits;

  AttendArgs a;
  a.q_bh = p.q + ((int64_t)b * p.num_q_heads + (int64_t)h * G) * HD;
  a.kvb = reinterpret_cast<const char*>(p.kv) + (int64_t)h * kRowB;
  a.row_bytes = p.num_kv_heads * kRowB;
  a.page_bytes = 2 * p.page_size * a.row_bytes;
  a.span = a.page_bytes - h * kRowB;
  a.page_size = p.page_size;
  a.num_pages = p.num_pages;
  a.G = G;
  a.scale_log2 = p.scale_log2;
  a.n = n;
  a.p0 = min(split * per_split, n);
  a.p1 = min(n, a.p0 + per_split);
  a.last_len = p.last_page_len[b];
  a.first_skip = p.first_page_offset;
  a.rotate = p.rotate ? attend_rotation(list, split) : 0u;

  // The list is read-only for the whole kernel; the constant address space
  // makes the uniform id load a scalar one (off the vector-memory counter that
  // the page prefetch relies on).
  const __attribute__((address_space(4))) int32_t* pl_c =
      reinterpret_cast<const __attribute__((address_space(4))) int32_t*>(reinterpret_cast<uintptr_t>(pl));
  const int64_t hq0 = (int64_t)b * p.num_q_heads + (int64_t)h * G;
  attend_list<NG, 4, F16, HD>(
      a, [&](int i) -> int { return pl_c[i]; }, lds, sm_m, sm_l,
      [&](int g, int d, float o, float lse2) {
        const int64_t hq = hq0 + g;
        if (p.num_splits == 1) {
          p.out[hq * HD + d] = (uint16_t)f32_to_elem<F16>(o);
          if (p.lse && d == 0) p.lse[hq] = lse2 * kLn2;
        } else {
          p.ws_o[(hq * p.num_splits + split) * HD + d] = o;
          if (d == 0) p.ws_lse[hq * p.num_splits + split] = lse2;
        }
      });
}

// Split-K merge: one block of head_dim threads per (sequence, query head).
template <bool F16>
__global__ __launch_bounds__(128) void merge_splits_kernel(const float* __restrict__ ws_o,
                                                           const float* __restrict__ ws_lse,
                                                           uint16_t* __restrict__ out, float* __restrict__ lse,
                                                           int num_splits) {
  const int64_t hq = blockIdx.x;
  const int d = threadIdx.x;
  const int hd = blockDim.x;
  const float* l2 = ws_lse + hq * num_splits;
  float mm = kNegInf;
#pragma unroll 8
  for (int s = 0; s < num_splits; ++s) mm = fmaxf(mm, l2[s]);
  const float m_safe = (mm == kNegInf) ? 0.f : mm;
  float num = 0.f, den = 0.f;
#pragma unroll 8
  for (int s = 0; s < num_splits; ++s) {
    const float wgt = fast_exp2(l2[s] - m_safe);
    num += ws_o[(hq * num_splits + s) * hd + d] * wgt;
    den += wgt;
  }
  out[hq * hd + d] = (uint16_t)f32_to_elem<F16>(den > 0.f ? num / den : 0.f);
  if (lse && d == 0) lse[hq] = (den > 0.f) ? (mm + fast_log2(den)) * kLn2 : kNegInf;
}

static int auto_splits(int batch, int num_kv_heads, int max_pages_per_list) {
  // Measured on dense decode (8 to 1024 lists of 65 to 2049 pages, 1 to 24 splits each):
  // up to 256 lists, a little under one workgroup per CU is best (more splits only add
  // partial results and merge work), never below 4 pages -- one per wave -- a split;
  // between 256 and 768 lists long lists gain from splitting (300 lists of 2049
  // pages: 0.94 ms whole, 0.77 ms in four to eight parts; 513 lists: 1.51 ms whole, 1.36
  // in four -- whole lists cannot be balanced over the CUs), shorter ones only just above a
  // multiple of the CUs (below), and from 768 lists on every CU holds its three workgroups anyway.
  const int64_t lists = (int64_t)batch * num_kv_heads;
  if (lists <= 0) return 1;
  int64_t want = 1;
  if (lists <= kNumCus)
    want = (kNumCus - kNumCus / 8 + lists / 2) / lists;
  else if (lists < 3 * kNumCus && max_pages_per_list >= 1024)
    want = (8 * kNumCus + lists - 1) / lists;
  else if (lists < 3 * kNumCus && lists % kNumCus != 0 && lists % kNumCus <= 96 && max_pages_per_list >= 32)
    // A few lists more than a multiple of the CUs: whole lists would leave those few running on a few
    // CUs beside or after the others.  In parts they spread (129-page lists: 264 lists 65 -> 55 us in
    // four parts, 300: 67 -> 58, 352: 73 -> 66 in two, 528: 108 -> 100; 257-page lists of 8 heads:
    // 264 lists 135 -> 108, 300: 138 -> 116, 528: 225 -> 201; 400 and 640 lists: whole lists win).
    want = lists % kNumCus <= 64 ? 4 : 2;
  int64_t cap = max_pages_per_list / 4;
  if (want > cap) want = cap;
  if (want > 64) want = 64;
  if (want < 1) want = 1;
  return (int)want;
}

static size_t workspace_bytes_for(int batch, int num_q_heads, int splits) {
  if (splits <= 1) return 0;
  return (size_t)batch * num_q_heads * splits * (kHeadDim + 1) * sizeof(float);
}

static int launch_decode(const char* fn, DecodeParams& p, int batch, void* workspace, size_t workspace_bytes,
                         int max_pages_per_list, int num_splits, bool f16, int head_dim, hipStream_t stream) {
  int splits = num_splits > 0 ? num_splits : auto_splits(batch, p.num_kv_heads, max_pages_per_list);
  if (splits > 65535) return fail(KIN_ERR_BAD_SHAPE, "%s: num_splits=%d exceeds 65535", fn, splits);
  p.num_splits = splits;
  if (splits > 1) {
    const size_t need = workspace_bytes_for(batch, p.num_q_heads, splits);
    if (!workspace || workspace_bytes < need)
      return fail(KIN_ERR_WORKSPACE, "%s: %d splits need %zu workspace bytes, got %zu", fn, splits, need,
                  workspace ? workspace_bytes : (size_t)0);
    if (!aligned16(workspace)) return fail(KIN_ERR_MISALIGNED, "%s: workspace must be 16-byte aligned", fn);
    p.ws_o = static_cast<float*>(workspace);
    p.ws_lse = p.ws_o + (size_t)batch * p.num_q_heads * splits * head_dim;
  } else {
    p.ws_o = nullptr;
    p.ws_lse = nullptr;
  }
  const int64_t lists = xcd_grid_size(batch, p.num_kv_heads);
  if (lists > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: batch*num_kv_heads too large", fn);
  p.batch = batch;
  p.rotate = attend_rotates((int64_t)batch * p.num_kv_heads) ? 1 : 0;
  dim3 grid((unsigned)lists, (unsigned)splits);
  if (head_dim == kHeadDimSmall) {
    if (p.group <= 4) {
      if (f16) paged_decode_kernel<1, true, kHeadDimSmall><<<grid, 256, 0, stream>>>(p);
      else paged_decode_kernel<1, false, kHeadDimSmall><<<grid, 256, 0, stream>>>(p);
    } else {
      if (f16) paged_decode_kernel<4, true, kHeadDimSmall><<<grid, 256, 0, stream>>>(p);
      else paged_decode_kernel<4, false, kHeadDimSmall><<<grid, 256, 0, stream>>>(p);
    }
  } else if (p.group <= 4) {
    if (f16) paged_decode_kernel<1, true><<<grid, 256, 0, stream>>>(p);
    else paged_decode_kernel<1, false><<<grid, 256, 0, stream>>>(p);
  } else {
    if (f16) paged_decode_kernel<4, true><<<grid, 256, 0, stream>>>(p);
    else paged_decode_kernel<4, false><<<grid, 256, 0, stream>>>(p);
  }
  int st = check_hip(hipGetLastError(), "paged_decode_kernel launch");
  if (st) return st;
  if (splits > 1) {
    const unsigned mgrid = (unsigned)((int64_t)batch * p.num_q_heads);
    if (f16) merge_splits_kernel<true><<<mgrid, head_dim, 0, stream>>>(p.ws_o, p.ws_lse, p.out, p.lse, splits);
    else merge_splits_kernel<false><<<mgrid, head_dim, 0, stream>>>(p.ws_o, p.ws_lse, p.out, p.lse, splits);
    st = check_hip(hipGetLastError(), "merge_splits_kernel launch");
  }
  return st;
}

static int check_decode_args(const char* fn, const void* q, const void* kv_cache, const void* last_page_len,
                             const void* out, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                             int page_size, int64_t num_pages, int first_page_offset, int num_splits) {
  if (!q || !kv_cache || !last_page_len || !out) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_common_dims(fn, batch, num_q_heads, num_kv_heads, head_dim, page_size, true);
  if (st) return st;
  st = check_first_page_offset(fn, first_page_offset, page_size);
  if (st) return st;
  if (num_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_pages=%lld must be >= 1", fn, (long long)num_pages);
  if (num_splits < 0) return fail(KIN_ERR_BAD_SHAPE, "%s: num_splits=%d is negative", fn, num_splits);
  if (!aligned16(q) || !aligned16(kv_cache) || !aligned16(out))
    return fail(KIN_ERR_MISALIGNED, "%s: q, kv_cache and out must be 16-byte aligned", fn);
  return KIN_OK;
}

}  // namespace kin

extern "C" {

int kin_decode_auto_splits(int batch, int num_kv_heads, int max_pages_per_list) {
  return kin::auto_splits(batch, num_kv_heads, max_pages_per_list);
}

size_t kin_decode_workspace_bytes(int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                  int max_pages_per_list, int num_splits) {
  (void)head_dim;
  if (batch <= 0 || num_q_heads <= 0 || num_kv_heads <= 0) return 0;
  const int splits = num_splits > 0 ? num_splits : kin::auto_splits(batch, num_kv_heads, max_pages_per_list);
  return kin::workspace_bytes_for(batch, num_q_heads, splits);
}

static int sparse_decode_impl(const char* fn, bool f16, const uint16_t* q, const uint16_t* kv_cache, const int32_t* sel_pages,
                              const int32_t* sel_count, const int32_t* last_page_len, uint16_t* out, float* lse,
                              void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                              int head_dim, int page_size, int64_t num_pages, int sel_stride, int first_page_offset,
                              float sm_scale, int num_splits, kin_stream_t stream) {
  using namespace kin;
  if (!sel_pages || !sel_count) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_decode_args(fn, q, kv_cache, last_page_len, out, batch, num_q_heads, num_kv_heads, head_dim,
                             page_size, num_pages, first_page_offset, num_splits);
  if (st) return st;
  if (sel_stride < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: sel_stride=%d must be >= 1", fn, sel_stride);
  if (batch == 0) return KIN_OK;
  DecodeParams p;
  p.q = q;
  p.kv = kv_cache;
  p.page_ids = sel_pages;
  p.list_indptr = nullptr;
  p.list_count = sel_count;
  p.last_page_len = last_page_len;
  p.out = out;
  p.lse = lse;
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.group = num_q_heads / num_kv_heads;
  p.list_stride = sel_stride;
  p.num_pages = num_pages;
  p.first_page_offset = first_page_offset;
  p.page_size = page_size;
  const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim);
  p.scale_log2 = scale * 1.4426950408889634f;
  return launch_decode(fn, p, batch, workspace, workspace_bytes, sel_stride, num_splits, f16, head_dim,
                       static_cast<hipStream_t>(stream));
}

static int dense_decode_impl(const char* fn, bool f16, const uint16_t* q, const uint16_t* kv_cache, const int32_t* page_indices,
                             const int32_t* page_indptr, const int32_t* last_page_len, uint16_t* out, float* lse,
                             void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                             int head_dim, int page_size, int64_t num_pages, int max_pages_per_seq,
                             int first_page_offset, float sm_scale, int num_splits, kin_stream_t stream) {
  using namespace kin;
  if (!page_indices || !page_indptr) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_decode_args(fn, q, kv_cache, last_page_len, out, batch, num_q_heads, num_kv_heads, head_dim,
                             page_size, num_pages, first_page_offset, num_splits);
  if (st) return st;
  if (max_pages_per_seq < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: max_pages_per_seq=%d must be >= 1", fn, max_pages_per_seq);
  if (batch == 0) return KIN_OK;
  DecodeParams p;
  p.q = q;
  p.kv = kv_cache;
  p.page_ids = page_indices;
  p.list_indptr = page_indptr;
  p.list_count = nullptr;
  p.last_page_len = last_page_len;
  p.out = out;
  p.lse = lse;
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.group = num_q_heads / num_kv_heads;
  p.list_stride = 0;
  p.num_pages = num_pages;
  p.first_page_offset = first_page_offset;
  p.page_size = page_size;
  const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim);
  p.scale_log2 = scale * 1.4426950408889634f;
  return launch_decode(fn, p, batch, workspace, workspace_bytes, max_pages_per_seq, num_splits, f16, head_dim,
                       static_cast<hipStream_t>(stream));
}

#define KIN_SPARSE_DECODE_ARGS                                                                                         \
  sel_pages, sel_count, last_page_len, out, lse, workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim, \
      page_size, num_pages, sel_stride, first_page_offset, sm_scale, num_splits, stream

int kin_sparse_paged_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache, const int32_t* sel_pages,
                            const int32_t* sel_count, const int32_t* last_page_len, kin_bf16_t* out, float* lse,
                            void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                            int head_dim, int page_size, int64_t num_pages, int sel_stride, int first_page_offset,
                            float sm_scale, int num_splits, kin_stream_t stream) {
  return sparse_decode_impl("kin_sparse_paged_decode", false, q, kv_cache, KIN_SPARSE_DECODE_ARGS);
}

int kin_sparse_paged_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache, const int32_t* sel_pages,
                                const int32_t* sel_count, const int32_t* last_page_len, kin_f16_t* out, float* lse,
                                void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                                int head_dim, int page_size, int64_t num_pages, int sel_stride, int first_page_offset,
                                float sm_scale, int num_splits, kin_stream_t stream) {
  return sparse_decode_impl("kin_sparse_paged_decode_f16", true, q, kv_cache, KIN_SPARSE_DECODE_ARGS);
}

#define KIN_DENSE_DECODE_ARGS                                                                                             \
  page_indices, page_indptr, last_page_len, out, lse, workspace, workspace_bytes, batch, num_q_heads, num_kv_heads, head_dim, \
      page_size, num_pages, max_pages_per_seq, first_page_offset, sm_scale, num_splits, stream

int kin_dense_paged_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache, const int32_t* page_indices,
                           const int32_t* page_indptr, const int32_t* last_page_len, kin_bf16_t* out, float* lse,
                           void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                           int head_dim, int page_size, int64_t num_pages, int max_pages_per_seq,
                           int first_page_offset, float sm_scale, int num_splits, kin_stream_t stream) {
  return dense_decode_impl("kin_dense_paged_decode", false, q, kv_cache, KIN_DENSE_DECODE_ARGS);
}

int kin_dense_paged_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache, const int32_t* page_indices,
                               const int32_t* page_indptr, const int32_t* last_page_len, kin_f16_t* out, float* lse,
                               void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                               int head_dim, int page_size, int64_t num_pages, int max_pages_per_seq,
                               int first_page_offset, float sm_scale, int num_splits, kin_stream_t stream) {
  return dense_decode_impl("kin_dense_paged_decode_f16", true, q, kv_cache, KIN_DENSE_DECODE_ARGS);
}

}  // extern "C"
