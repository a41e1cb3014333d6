// Token-level top-k sparse decode attention in one launch: for every (sequence,
// KV head) every token of the context is scored, the sink tokens, the local
// window and the top-k tokens in between are listed, and attended to
// (token_score_keys() / token_select_list() / attend_tokens(), kin_token.h).
// `chunks` workgroups share the scoring of one list, each a run of pages; the first
// `parts` of them then select for themselves and attend a share of the token list,
// and the last of those to finish merges the partial results (the team scheme of the
// fused block top-k step).  Splitting keeps a few long lists from leaving most of
// the GPU idle.
#include "kin_token_kernel.h"

namespace kin {

// Bytes of the arrival counters (two per list) in front of the score arrays.
static size_t token_count_bytes(int64_t lists) { return ((size_t)lists * 2 * sizeof(int32_t) + 255) & ~(size_t)255; }

// Most members of a team that go on to select and attend: a share of at least 128 listed tokens each.
constexpr int kMaxTokenParts = 16;
static int token_team_parts(int chunks, int list_cap) {
  int parts = list_cap / 128;
  if (parts > chunks) parts = chunks;
  if (parts > kMaxTokenParts) parts = kMaxTokenParts;
  return parts < 2 ? 1 : parts;
}
// What teams need behind the score arrays: the members' first-digit histograms and the partial results
// (sized for the largest group, so that the sizing entry points need not know the group).
static size_t token_team_bytes(int64_t lists, int chunks) {
  if (chunks <= 1) return 0;
  const int parts = chunks < kMaxTokenParts ? chunks : kMaxTokenParts;
  return (size_t)lists * chunks * 256 * sizeof(uint32_t) + (size_t)lists * parts * kMaxGroup * (kHeadDim + 1) * sizeof(float);
}

// Workgroups that share the scoring of one list (each at least 64 pages = 256 KiB
// of keys; with 256 the 8 lists of a small batch occupied 64 CUs: 109 against 97 us
// at 32 K tokens): as many as it takes to give every CU one when the lists are fewer
// than the CUs, otherwise one -- with the GPU already full, splitting only adds
// workgroups, the extra pass that recounts the first radix digit and a second
// round of launches (measured: 6.35 -> 7.1 ms at 4096 lists of 32 K tokens).
static int token_score_chunks(int64_t lists, int max_pages_per_seq) {
  const int by_len = max_pages_per_seq / 64;
  const int64_t want = kNumCus / lists;
  if (by_len < 2 || want < 2) return 1;
  return (int)(want < by_len ? want : by_len);
}

// Lists that a batch has beyond a multiple of the CUs, when they are few enough to be worth a launch of
// their own (see launch_token_policy) and the multiple is whole sequences; else 0.
constexpr int kMaxTokenTailLists = 96;
static int64_t token_tail_lists(int64_t lists, int num_kv_heads) {
  if (lists <= kNumCus || kNumCus % num_kv_heads != 0) return 0;
  const int64_t tail = lists % kNumCus;
  return tail <= kMaxTokenTailLists ? tail : 0;
}
// Workspace of one launch over `lists` lists: counters, keys (and scores: arrays = 2), what teams need.
static size_t token_workspace_need(int64_t lists, int max_pages_per_seq, int arrays) {
  return token_count_bytes(lists) + (size_t)arrays * lists * max_pages_per_seq * kPageSize * sizeof(uint32_t) +
         token_team_bytes(lists, token_score_chunks(lists, max_pages_per_seq));
}
// The same for a call, which may be two launches that use the workspace one after the other.
static size_t token_workspace_bytes(int batch, int num_kv_heads, int max_pages_per_seq, int arrays) {
  if (batch <= 0 || num_kv_heads <= 0 || max_pages_per_seq <= 0) return 0;
  const int64_t lists = (int64_t)batch * num_kv_heads;
  size_t need = token_workspace_need(lists, max_pages_per_seq, arrays);
  const int64_t tail = token_tail_lists(lists, num_kv_heads);
  if (tail > 0) {
    const size_t t = token_workspace_need(tail, max_pages_per_seq, arrays);
    if (t > need) need = t;
  }
  return need;
}

// Shared by the two entry points.  topk counts tokens (block == 0) or blocks.
static int launch_token_policy(const char* fn, bool f16, const kin_bf16_t* q, const kin_bf16_t* kv_cache,
                               const int32_t* page_indices, const int32_t* page_indptr, const int32_t* last_page_len,
                               int topk, int block, int stride, int sink_tokens, int local_tokens,
                               int first_page_offset, int32_t* sel_tokens, int32_t* sel_count, kin_bf16_t* out,
                               float* lse, void* workspace, size_t workspace_bytes, int batch, int num_q_heads,
                               int num_kv_heads, int head_dim, int page_size, int64_t num_pages,
                               int max_pages_per_seq, int sel_stride, float sm_scale, kin_stream_t stream,
                               bool may_split = true) {
  const bool strided = block > 0;
  if (!q || !kv_cache || !page_indices || !page_indptr || !last_page_len || !out)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_common_dims(fn, batch, num_q_heads, num_kv_heads, head_dim, page_size, true);
  if (st) return st;
  st = check_page_size_16(fn, page_size);
  if (st) return st;
  st = check_first_page_offset(fn, first_page_offset);
  if (st) return st;
  if (num_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_pages=%lld must be >= 1", fn, (long long)num_pages);
  if (num_pages > 0x7fffffffLL / kPageSize)
    return fail(KIN_ERR_UNSUPPORTED, "%s: num_pages=%lld: token ids do not fit 31 bits", fn, (long long)num_pages);
  if (topk < 0 || sink_tokens < 0 || local_tokens < 0)
    return fail(KIN_ERR_BAD_SHAPE, "%s: the budget (%d), sink_tokens=%d and local_tokens=%d must not be negative", fn,
                topk, sink_tokens, local_tokens);
  if (max_pages_per_seq < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: max_pages_per_seq=%d must be >= 1", fn, max_pages_per_seq);
  int budget_tokens = topk;
  if (strided) {
    if (block > 64 || stride < 1)
      return fail(KIN_ERR_BAD_SHAPE, "%s: block_size=%d must be in [1, 64] and stride=%d at least 1", fn, block, stride);
    if ((int64_t)topk * block > kMaxTopkTokens)
      return fail(KIN_ERR_UNSUPPORTED, "%s: topk_blocks * block_size = %lld exceeds the limit %d", fn,
                  (long long)topk * block, kMaxTopkTokens);
    budget_tokens = topk * block;
    if (budget_tokens < block) budget_tokens = block;  // sequences shorter than a block are listed whole
  }
  if (budget_tokens > kMaxTopkTokens || sink_tokens > kMaxSinkTokens || local_tokens > kMaxWindowTokens)
    return fail(KIN_ERR_UNSUPPORTED, "%s: limits are %d selected tokens, sink_tokens <= %d, local_tokens <= %d", fn,
                kMaxTopkTokens, kMaxSinkTokens, kMaxWindowTokens);
  const int list_cap = budget_tokens + sink_tokens + local_tokens;
  if (sel_tokens && sel_stride < list_cap)
    return fail(KIN_ERR_BAD_SHAPE, "%s: sel_stride=%d must be at least %d (selected + sink + local tokens)", fn,
                sel_stride, list_cap);
  if (sel_tokens && !sel_count) return fail(KIN_ERR_NULL_POINTER, "%s: sel_tokens given without sel_count", fn);
  if (!aligned16(q) || !aligned16(kv_cache) || !aligned16(out))
    return fail(KIN_ERR_MISALIGNED, "%s: q, kv_cache and out must be 16-byte aligned", fn);
  const int64_t items = (int64_t)batch * num_kv_heads;
  const size_t count_bytes = token_count_bytes(items);
  const size_t key_bytes = (size_t)items * max_pages_per_seq * kPageSize * sizeof(uint32_t);
  const size_t need = count_bytes + (strided ? 2 * key_bytes : key_bytes);
  if (batch == 0) return KIN_OK;
  if (!workspace || workspace_bytes < need)
    return fail(KIN_ERR_WORKSPACE, "%s: needs %zu workspace bytes, got %zu", fn, need,
                workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(KIN_ERR_MISALIGNED, "%s: workspace must be 16-byte aligned", fn);

  // A few lists more than a multiple of the CUs: the GPU hands out workgroups in order, so the last few
  // lists would run on a few CUs after everybody else has finished (a 12-wave workgroup has a CU to
  // itself: 300 lists are two rounds, the second of 44).  Two launches instead, one after the other on
  // the stream: the whole rounds, then the rest with the GPU to themselves (shared scoring and teams,
  // as for any small batch; the workspace is used by one launch at a time).  Measured, 2048 tokens of
  // 32 K, one launch | two: 264 lists 545 | 423 us; 300: 575 | 497; 352: 616 | 590; 528: 942 | 835;
  // 800: 1311 | 1223; 1056: 1670 | 1585.
  if (may_split && token_tail_lists(items, num_kv_heads) > 0) {
    const int b0 = (int)((items - token_tail_lists(items, num_kv_heads)) / num_kv_heads);
    const int hq = num_q_heads, d = head_dim;
    st = launch_token_policy(fn, f16, q, kv_cache, page_indices, page_indptr, last_page_len, topk, block, stride, sink_tokens,
                             local_tokens, first_page_offset, sel_tokens, sel_count, out, lse, workspace, workspace_bytes, b0,
                             num_q_heads, num_kv_heads, head_dim, page_size, num_pages, max_pages_per_seq, sel_stride, sm_scale,
                             stream, false);
    if (st) return st;
    return launch_token_policy(fn, f16, q + (size_t)b0 * hq * d, kv_cache, page_indices, page_indptr + b0, last_page_len + b0, topk,
                               block, stride, sink_tokens, local_tokens, first_page_offset,
                               sel_tokens ? sel_tokens + (size_t)b0 * num_kv_heads * sel_stride : nullptr,
                               sel_count ? sel_count + (size_t)b0 * num_kv_heads : nullptr, out + (size_t)b0 * hq * d,
                               lse ? lse + (size_t)b0 * hq : nullptr, workspace, workspace_bytes, batch - b0, num_q_heads,
                               num_kv_heads, head_dim, page_size, num_pages, max_pages_per_seq, sel_stride, sm_scale, stream,
                               false);
  }

  TokenTopkParams p;
  p.q = q;
  p.kv = kv_cache;
  p.page_indices = page_indices;
  p.page_indptr = page_indptr;
  p.last_page_len = last_page_len;
  p.sel_tokens = sel_tokens;
  p.sel_count = sel_count;
  p.out = out;
  p.lse = lse;
  p.count = static_cast<int32_t*>(workspace);
  p.count2 = p.count + items;
  p.keys = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + count_bytes);
  p.scores = strided ? reinterpret_cast<float*>(static_cast<char*>(workspace) + count_bytes + key_bytes) : nullptr;
  p.parts = 1;
  p.stage_scores = 0;
  p.spin_limit = team_spin_limit();
  p.ws_hist = nullptr;
  p.ws_po = nullptr;
  p.ws_plse = nullptr;
  p.block = block;
  p.stride = stride;
  p.list_cap = list_cap > 0 ? list_cap : 1;
  p.batch = batch;
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.group = num_q_heads / num_kv_heads;
  p.topk = topk;
  p.sink_tokens = sink_tokens;
  p.local_tokens = local_tokens;
  p.first_page_offset = first_page_offset;
  p.max_pages_per_seq = max_pages_per_seq;
  p.sel_stride = sel_stride;
  p.num_pages = num_pages;
  const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim);
  p.scale_log2 = scale * 1.4426950408889634f;

  // How a list's token keys travel from scoring to selection.  Kept in LDS when they fit
  // and the lists alone occupy at least half the CUs: key stores to HBM between the loads
  // of a saturated stream cost far more than their bytes.  One 12-wave workgroup per CU
  // while the lists are no more than the CUs or the keys need the room, else three 4-wave
  // workgroups per CU (the same 12 waves).  Otherwise the keys go through the workspace:
  // few lists split their scoring into chunks, and workgroups have 8 waves until 4-wave
  // ones fill the GPU (the per-token addressing needs ~140 registers, so 16 do not fit).
  const size_t bitmap_bytes = strided ? ((size_t)max_pages_per_seq * kPageSize / 32 + 1) * 4 : 0;
  const size_t tail_bytes = (size_t)p.list_cap * 4 + bitmap_bytes;
  const size_t key_lds = ((size_t)max_pages_per_seq * kPageSize + 4) * sizeof(uint32_t);
  const size_t small = (key_lds > (size_t)attend_lds_bytes(4) ? key_lds : (size_t)attend_lds_bytes(4)) + tail_bytes;
  const size_t big = (key_lds > (size_t)attend_lds_bytes(12) ? key_lds : (size_t)attend_lds_bytes(12)) + tail_bytes;
  const bool ldsk = items >= kNumCus / 2 && big <= 156 * 1024;
  int nw;
  if (ldsk) {
    p.chunks = 1;
    nw = items > kNumCus && small <= 50 * 1024 ? 4 : 12;
  } else {
    p.chunks = token_score_chunks(items, max_pages_per_seq);
    // Teams: the members that scored go on to select and attend a share of the list each, given
    // the room for their histograms and partial results behind the score arrays.
    const size_t team_bytes = token_team_bytes(items, p.chunks);
    const int parts = token_team_parts(p.chunks, list_cap);
    if (parts > 1 && workspace_bytes >= need + team_bytes) {
      p.parts = parts;
      char* w = static_cast<char*>(workspace) + need;
      p.ws_hist = reinterpret_cast<uint32_t*>(w);
      p.ws_po = p.ws_hist + (size_t)items * p.chunks * 256;
      p.ws_plse = p.ws_po + (size_t)items * parts * p.group * head_dim;
    }
    // Up to one list per CU: 12 waves once a sequence may have more keys than 8 waves hold in
    // registers through the select's passes (32 K; 8 lists of 32 K tokens: 97 -> 83 us), else 8.
    nw = items <= kNumCus && (int64_t)max_pages_per_seq * kPageSize > 8 * 4096 ? 12 : (items <= 2 * kNumCus ? 8 : 4);
    if (nw == 12 && (size_t)attend_lds_bytes(12) + tail_bytes > 150 * 1024) nw = 8;  // room for the strided policy's bitmap
  }
  const int64_t grid = xcd_grid_size(batch, num_kv_heads) * p.chunks;
  if (grid > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: batch*num_kv_heads too large", fn);
  size_t region0 = (size_t)attend_lds_bytes(nw);
  if (ldsk && key_lds > region0) region0 = (key_lds + 15) & ~(size_t)15;
  if (!ldsk && strided && p.parts > 1) {
    const size_t staged = key_lds > region0 ? ((key_lds + 15) & ~(size_t)15) : region0;
    if (staged + tail_bytes <= 150 * 1024) {
      region0 = staged;
      p.stage_scores = 1;
    }
  }
  p.region0_bytes = (int)region0;
  const size_t lds = region0 + tail_bytes;
  if (lds > 150 * 1024 && !ldsk)
    return fail(KIN_ERR_UNSUPPORTED, "%s: max_pages_per_seq=%d is too long for the strided policy's token bitmap", fn,
                max_pages_per_seq);
  const void* kernel = head_dim == kHeadDimSmall ? token_kernel_small_head(f16, strided, p.group, nw, ldsk)
                                                 : token_kernel_for<kHeadDim>(f16, strided, p.group, nw, ldsk);
  if (lds > 48 * 1024) {
    st = check_hip(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                   "hipFuncSetAttribute(token_topk_kernel)");
    if (st) return st;
  }
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (p.chunks > 1) {
    // a kernel, not a memset node: this launch sequence may be captured into a HIP graph
    fill_zero_i32_kernel<<<(unsigned)((2 * items + 255) / 256), 256, 0, hs>>>(p.count, (int)(2 * items));
    st = check_hip(hipGetLastError(), "fill_zero_i32_kernel launch");
    if (st) return st;
  }
  void* args[] = {&p};
  return check_hip(hipLaunchKernel(kernel, dim3((unsigned)grid), dim3(nw * 64), args, lds, hs), "token_topk_kernel launch");
}

}  // namespace kin

#ifdef KIN_TUNE
KIN_STAMP_ACCESSOR(kin_debug_stamps_token)
#endif

extern "C" {

size_t kin_token_topk_workspace_bytes(int batch, int num_kv_heads, int max_pages_per_seq) {
  return kin::token_workspace_bytes(batch, num_kv_heads, max_pages_per_seq, 1);
}

size_t kin_strided_topk_workspace_bytes(int batch, int num_kv_heads, int max_pages_per_seq) {
  return kin::token_workspace_bytes(batch, num_kv_heads, max_pages_per_seq, 2);
}

int kin_token_topk_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache, const int32_t* page_indices,
                          const int32_t* page_indptr, const int32_t* last_page_len, int topk_tokens,
                          int sink_tokens, int local_tokens, int first_page_offset, int32_t* sel_tokens,
                          int32_t* sel_count, kin_bf16_t* out, float* lse, void* workspace, size_t workspace_bytes,
                          int batch, int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                          int64_t num_pages, int max_pages_per_seq, int sel_stride, float sm_scale,
                          kin_stream_t stream) {
  return kin::launch_token_policy("kin_token_topk_decode", false, q, kv_cache, page_indices, page_indptr, last_page_len,
                                  topk_tokens, 0, 0, sink_tokens, local_tokens, first_page_offset, sel_tokens,
                                  sel_count, out, lse, workspace, workspace_bytes, batch, num_q_heads, num_kv_heads,
                                  head_dim, page_size, num_pages, max_pages_per_seq, sel_stride, sm_scale, stream);
}

int kin_token_topk_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache, const int32_t* page_indices,
                              const int32_t* page_indptr, const int32_t* last_page_len, int topk_tokens,
                              int sink_tokens, int local_tokens, int first_page_offset, int32_t* sel_tokens,
                              int32_t* sel_count, kin_f16_t* out, float* lse, void* workspace, size_t workspace_bytes,
                              int batch, int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                              int64_t num_pages, int max_pages_per_seq, int sel_stride, float sm_scale,
                              kin_stream_t stream) {
  return kin::launch_token_policy("kin_token_topk_decode_f16", true, q, kv_cache, page_indices, page_indptr, last_page_len,
                                  topk_tokens, 0, 0, sink_tokens, local_tokens, first_page_offset, sel_tokens,
                                  sel_count, out, lse, workspace, workspace_bytes, batch, num_q_heads, num_kv_heads,
                                  head_dim, page_size, num_pages, max_pages_per_seq, sel_stride, sm_scale, stream);
}

int kin_strided_topk_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache, const int32_t* page_indices,
                            const int32_t* page_indptr, const int32_t* last_page_len, int topk_blocks,
                            int block_size, int stride, int sink_tokens, int local_tokens, int first_page_offset,
                            int32_t* sel_tokens, int32_t* sel_count, kin_bf16_t* out, float* lse, void* workspace,
                            size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                            int page_size, int64_t num_pages, int max_pages_per_seq, int sel_stride, float sm_scale,
                            kin_stream_t stream) {
  if (block_size < 1)
    return kin::fail(KIN_ERR_BAD_SHAPE, "kin_strided_topk_decode: block_size=%d must be in [1, 64]", block_size);
  return kin::launch_token_policy("kin_strided_topk_decode", false, q, kv_cache, page_indices, page_indptr, last_page_len,
                                  topk_blocks, block_size, stride, sink_tokens, local_tokens, first_page_offset,
                                  sel_tokens, sel_count, out, lse, workspace, workspace_bytes, batch, num_q_heads,
                                  num_kv_heads, head_dim, page_size, num_pages, max_pages_per_seq, sel_stride,
                                  sm_scale, stream);
}

int kin_strided_topk_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache, const int32_t* page_indices,
                                const int32_t* page_indptr, const int32_t* last_page_len, int topk_blocks,
                                int block_size, int stride, int sink_tokens, int local_tokens, int first_page_offset,
                                int32_t* sel_tokens, int32_t* sel_count, kin_f16_t* out, float* lse, void* workspace,
                                size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                int page_size, int64_t num_pages, int max_pages_per_seq, int sel_stride,
                                float sm_scale, kin_stream_t stream) {
  if (block_size < 1)
    return kin::fail(KIN_ERR_BAD_SHAPE, "kin_strided_topk_decode_f16: block_size=%d must be in [1, 64]", block_size);
  return kin::launch_token_policy("kin_strided_topk_decode_f16", true, q, kv_cache, page_indices, page_indptr,
                                  last_page_len, topk_blocks, block_size, stride, sink_tokens, local_tokens,
                                  first_page_offset, sel_tokens, sel_count, out, lse, workspace, workspace_bytes, batch,
                                  num_q_heads, num_kv_heads, head_dim, page_size, num_pages, max_pages_per_seq,
                                  sel_stride, sm_scale, stream);
}

}  // extern "C"
