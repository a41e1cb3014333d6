// Stand-alone page scoring + top-k page selection kernel: one 256-thread
// workgroup per (sequence, KV head) runs score_select() (kin_select.h) and
// copies the page list to HBM.  With few, long lists and a workspace, `chunks`
// workgroups score a slice of one list's candidates each into global memory and
// the last one to finish selects.
#include "kin_select.h"

namespace kin {

struct ScoreTopkParams {
  const uint16_t* q;
  const uint16_t* kbar;
  const int32_t* page_indices;
  const int32_t* page_indptr;
  const int32_t* last_page_len;
  int32_t* sel_pages;
  int32_t* sel_count;
  int32_t* sel_logical;  // may be null
  float* scores_out;     // may be null
  int batch, num_q_heads, num_kv_heads, group;
  int kbar_pages, sel_stride, topk, sink_pages, local_tokens, page_size;
  int sort_cap;
  int table_cap;       // LDS entries for the copy of a sequence's page table (0: none)
  int chunks;          // workgroups per list
  int32_t* ws_count;   // [lists] arrival counters, zero at launch and left zero
  uint32_t* ws_keys;   // [lists, score_key_stride(kbar_pages)]
  const int32_t* slot_ids;  // kbar row block of each sequence (null: the sequence's own index)
  int num_slots;
};

// Dynamic LDS layout: uint32 keys[kbar_pages_padded] | uint64 sortbuf[sort_cap] | int32 table[table_cap] |
// int32 sel[sink + topk + local]
template <int UNROLL, bool F16, int HD = kHeadDim>
__global__ __launch_bounds__(kThreads) void score_topk_kernel(ScoreTopkParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ int sh_last;
  __shared__ SelectScratch ss;
  const int tid = threadIdx.x;
  clear_select_scratch<kThreads>(&ss);
  const int list_id = blockIdx.x / p.chunks, chunk = blockIdx.x - list_id * p.chunks;
  int b, h;
  if (!xcd_list_of(list_id, p.batch, p.num_kv_heads, b, h)) return;
  const int item = b * p.num_kv_heads + h;

  const int ps = p.page_indptr[b], pe = p.page_indptr[b + 1];
  const int n_pages = pe - ps;
  int32_t* sel = p.sel_pages + (int64_t)item * p.sel_stride;
  if (n_pages <= 0) {
    if (chunk) return;
    for (int i = tid; i < p.sel_stride; i += kThreads) sel[i] = -1;
    if (tid == 0) p.sel_count[item] = 0;
    return;
  }
  const size_t sel_off = select_lds_bytes(p.kbar_pages, p.sort_cap, p.table_cap);
  int32_t* sel_lds = reinterpret_cast<int32_t*>(smem + sel_off);
  int32_t* table_lds = reinterpret_cast<int32_t*>(smem + select_table_offset(p.kbar_pages, p.sort_cap));

  SelectArgs a;
  a.q_bh = p.q + ((int64_t)b * p.num_q_heads + (int64_t)h * p.group) * HD;
  a.G = p.group;
  a.n_pages = n_pages;
  const int kb = kbar_block_of(p.slot_ids, p.num_slots, b);  // (a sequence without mean keys has no candidates)
  split_pages(n_pages, p.last_page_len[b], p.sink_pages, p.local_tokens, kb >= 0 ? p.kbar_pages : 0, p.page_size, a.n_sink, a.n_cand,
              a.n_local);
  a.kb = reinterpret_cast<const char*>(p.kbar) + kbar_row_index(max(kb, 0), h, a.n_sink, p.num_kv_heads, p.kbar_pages) * (HD * 2);
  a.topk = p.topk;
  a.table = p.page_indices + ps;
  a.sel_logical = p.sel_logical ? p.sel_logical + (int64_t)item * p.topk : nullptr;
  a.scores_out = p.scores_out ? p.scores_out + (int64_t)item * p.kbar_pages + a.n_sink : nullptr;
  a.keys = reinterpret_cast<uint32_t*>(smem);
  a.sortbuf = reinterpret_cast<unsigned long long*>(smem + (size_t)((p.kbar_pages + 3) & ~3) * 4);
  a.sort_cap = p.sort_cap;
  a.ss = &ss;
  a.table_lds = nullptr;
  a.digit0_counted = false;
  a.sorted = true;
  int n_list;
  if (p.chunks > 1) {
    // This workgroup's slice of the candidates -> keys in global memory, written and
    // (by the workgroup that counts in last) read at device scope: no cache
    // maintenance, every wave waits for its own stores before the workgroup counts in.
    uint32_t* gkeys = p.ws_keys + (int64_t)item * score_key_stride(p.kbar_pages);
    const int n_score = (min(a.topk, a.n_cand) > 0 || a.scores_out) ? a.n_cand : 0;
    const int per = ((n_score + p.chunks - 1) / p.chunks + 63) & ~63;
    const int r0 = min(chunk * per, n_score), r1 = min(r0 + per, n_score);
    score_rows<UNROLL, kThreads, true, F16, false, HD>(a, r0, r1, gkeys);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0)
      sh_last = (__hip_atomic_fetch_add(&p.ws_count[item], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.chunks - 1)
                    ? 1 : 0;
    __syncthreads();
    if (!sh_last) return;
    if (tid == 0) __hip_atomic_store(&p.ws_count[item], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    a.table_lds = prefetch_table<kThreads>(a.table, n_pages, table_lds, p.table_cap);
    load_shared_keys<kThreads>(gkeys, n_score, a.keys);
    __builtin_amdgcn_s_waitcnt(0);  // the table copy has landed too
    __syncthreads();
    n_list = select_from_keys<kThreads>(a, sel_lds);
  } else {
    a.table_lds = prefetch_table<kThreads>(a.table, n_pages, table_lds, p.table_cap);
    __syncthreads();  // histograms zeroed
    n_list = score_select<UNROLL, kThreads, F16, HD>(a, sel_lds);
  }

  for (int i = tid; i < p.sel_stride; i += kThreads) sel[i] = (i < n_list) ? sel_lds[i] : -1;
  if (tid == 0) p.sel_count[item] = n_list;
}

}  // namespace kin

namespace kin {
static int score_topk_impl(const char* fn, bool f16, const uint16_t* q, const uint16_t* kbar, const int32_t* page_indices,
                           const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                           int sink_pages, int local_tokens,
                           int32_t* sel_pages, int32_t* sel_count,
                           int32_t* sel_logical, float* scores_out, int batch, int num_q_heads,
                           int num_kv_heads, int head_dim, int page_size, int kbar_pages, int sel_stride,
                           void* workspace, size_t workspace_bytes, const int32_t* slot_ids, int num_slots,
                           kin_stream_t stream) {
  if (!q || !kbar || !page_indices || !page_indptr || !last_page_len || !sel_pages || !sel_count)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_common_dims(fn, batch, num_q_heads, num_kv_heads, head_dim, page_size, true);
  if (st) return st;
  if (topk < 0) return fail(KIN_ERR_BAD_SHAPE, "%s: topk=%d is negative", fn, topk);
  st = check_fixed_pages(fn, sink_pages, local_tokens);
  if (st) return st;
  const int list_cap = topk + sink_pages + max_local_pages(local_tokens);
  if (sel_stride < list_cap)
    return fail(KIN_ERR_BAD_SHAPE, "%s: sel_stride=%d must be at least kin_sel_list_capacity(topk, sink_pages, local_tokens) = %d",
                fn, sel_stride, list_cap);
  if (kbar_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: kbar_pages=%d must be >= 1", fn, kbar_pages);
  if (slot_ids && num_slots < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_slots=%d must be >= 1 when slot_ids is given", fn, num_slots);
  if (topk > kMaxTopk) return fail(KIN_ERR_UNSUPPORTED, "%s: topk=%d exceeds the limit %d", fn, topk, kMaxTopk);
  if (kbar_pages > kMaxCandidates)
    return fail(KIN_ERR_UNSUPPORTED, "%s: kbar_pages=%d exceeds the limit %d", fn, kbar_pages, kMaxCandidates);
  if (!aligned16(q) || !aligned16(kbar)) return fail(KIN_ERR_MISALIGNED, "%s: q and kbar must be 16-byte aligned", fn);
  if (batch == 0) return KIN_OK;

  ScoreTopkParams p;
  p.q = q;
  p.kbar = kbar;
  p.page_indices = page_indices;
  p.page_indptr = page_indptr;
  p.last_page_len = last_page_len;
  p.sel_pages = sel_pages;
  p.sel_count = sel_count;
  p.sel_logical = sel_logical;
  p.scores_out = scores_out;
  p.batch = batch;
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.group = num_q_heads / num_kv_heads;
  p.kbar_pages = kbar_pages;
  p.sel_stride = sel_stride;
  p.topk = topk;
  p.sink_pages = sink_pages;
  p.local_tokens = local_tokens;
  p.page_size = page_size;
  p.slot_ids = slot_ids;
  p.num_slots = slot_ids ? num_slots : batch;
  p.sort_cap = select_sort_cap(topk, kbar_pages);
  p.table_cap = select_table_cap(kbar_pages + max_local_pages(local_tokens) + 1);
  const size_t lds = select_lds_bytes(kbar_pages, p.sort_cap, p.table_cap) + (size_t)list_cap * 4;
  const int64_t items = (int64_t)batch * num_kv_heads;
  if (xcd_grid_size(batch, num_kv_heads) > 0x7fffffffLL)
    return fail(KIN_ERR_UNSUPPORTED, "%s: batch*num_kv_heads too large", fn);
  // Few long lists: spread the scoring of each over several workgroups, given a workspace.
  p.chunks = score_chunks(batch, num_kv_heads, kbar_pages);
  const size_t ws_need = score_workspace_bytes(items, kbar_pages);
  if (p.chunks > 1 && workspace && aligned16(workspace) && workspace_bytes >= ws_need) {
    p.ws_count = static_cast<int32_t*>(workspace);
    p.ws_keys = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + score_count_bytes(items));
  } else {
    p.chunks = 1;
    p.ws_count = nullptr;
    p.ws_keys = nullptr;
  }
  const int64_t grid = xcd_grid_size(batch, num_kv_heads) * p.chunks;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (p.chunks > 1) {
    fill_zero_i32_kernel<<<(unsigned)((items + 255) / 256), 256, 0, hs>>>(p.ws_count, (int)items);
    st = check_hip(hipGetLastError(), "fill_zero_i32_kernel launch");
    if (st) return st;
  }
  // Few workgroups cannot saturate HBM with 4 loads per lane in flight: give a
  // small grid 16 (more registers, which it can afford).
  const bool small_grid = items < 512;
  const void* fn_ptr;
#define KIN_SCORE_KERNEL(HD_)                                                                      \
  (f16 ? (small_grid ? reinterpret_cast<const void*>(&score_topk_kernel<16, true, HD_>)            \
                     : reinterpret_cast<const void*>(&score_topk_kernel<4, true, HD_>))            \
       : (small_grid ? reinterpret_cast<const void*>(&score_topk_kernel<16, false, HD_>)           \
                     : reinterpret_cast<const void*>(&score_topk_kernel<4, false, HD_>)))
  fn_ptr = head_dim == kHeadDimSmall ? KIN_SCORE_KERNEL(kHeadDimSmall) : KIN_SCORE_KERNEL(kHeadDim);
#undef KIN_SCORE_KERNEL
  if (lds > 48 * 1024) {
    // Above the default dynamic-LDS allowance the runtime wants an explicit opt-in.
    st = check_hip(hipFuncSetAttribute(fn_ptr, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                   "hipFuncSetAttribute(score_topk_kernel)");
    if (st) return st;
  }
  void* args[] = {&p};
  return check_hip(hipLaunchKernel(fn_ptr, dim3((unsigned)grid), dim3(kThreads), args, lds, hs), "score_topk_kernel launch");
}
}  // namespace kin

extern "C" int kin_block_score_topk(const kin_bf16_t* q, const kin_bf16_t* kbar, const int32_t* page_indices,
                                    const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                                    int sink_pages, int local_tokens, int32_t* sel_pages, int32_t* sel_count,
                                    int32_t* sel_logical, float* scores_out, int batch, int num_q_heads,
                                    int num_kv_heads, int head_dim, int page_size, int kbar_pages, int sel_stride,
                                    void* workspace, size_t workspace_bytes, const int32_t* slot_ids, int num_slots,
                                    kin_stream_t stream) {
  return kin::score_topk_impl("kin_block_score_topk", false, q, kbar, page_indices, page_indptr, last_page_len, topk,
                              sink_pages, local_tokens, sel_pages, sel_count, sel_logical, scores_out, batch, num_q_heads,
                              num_kv_heads, head_dim, page_size, kbar_pages, sel_stride, workspace, workspace_bytes, slot_ids, num_slots, stream);
}

extern "C" int kin_block_score_topk_f16(const kin_f16_t* q, const kin_f16_t* kbar, const int32_t* page_indices,
                                        const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                                        int sink_pages, int local_tokens, int32_t* sel_pages, int32_t* sel_count,
                                        int32_t* sel_logical, float* scores_out, int batch, int num_q_heads,
                                        int num_kv_heads, int head_dim, int page_size, int kbar_pages, int sel_stride,
                                        void* workspace, size_t workspace_bytes, const int32_t* slot_ids, int num_slots,
                                        kin_stream_t stream) {
  return kin::score_topk_impl("kin_block_score_topk_f16", true, q, kbar, page_indices, page_indptr, last_page_len, topk,
                              sink_pages, local_tokens, sel_pages, sel_count, sel_logical, scores_out, batch, num_q_heads,
                              num_kv_heads, head_dim, page_size, kbar_pages, sel_stride, workspace, workspace_bytes, slot_ids, num_slots, stream);
}
