// Token-level top-k sparse decode attention in one launch: for every (sequence,
// KV head) every token of the context is scored, the sink tokens, the local
// window and the top-k tokens in between are listed, and attended to
// (token_score_keys() / token_select_list() / attend_tokens(), kin_token.h).
// `chunks` workgroups share the scoring of one list, each a run of pages; the first
// `parts` of them then select for themselves and attend a share of the token list,
// and the last of those to finish merges the partial results (the team scheme of the
// fused block top-k step).  Splitting keeps a few long lists from leaving most of
// the GPU idle.
#include "kin_step.h"
#include "kin_token.h"

namespace kin {

struct TokenTopkParams {
  const uint16_t* q;
  const uint16_t* kv;
  const int32_t* page_indices;
  const int32_t* page_indptr;
  const int32_t* last_page_len;
  int32_t* sel_tokens;  // optional [lists, sel_stride]
  int32_t* sel_count;   // optional [lists]
  uint16_t* out;
  float* lse;           // optional
  int chunks;           // workgroups per list
  int parts;            // of them, how many go on to select and attend a share of the list (1: the last arriver alone)
  int spin_limit;       // polls a member waits for its team before it scores the whole list itself
  int stage_scores;     // strided policy in a team: region 0 has room for the sequence's scores, which the members copy
                        // from the workspace to LDS before they select (block means from LDS, not from memory)
  int32_t* count;       // workspace: [lists] arrival counters of the scoring, zero at launch
  int32_t* count2;      // workspace, parts > 1: [lists] arrival counters of the partial results, zero at launch
  uint32_t* ws_hist;    // workspace, parts > 1: [lists, chunks, 256] first-digit histograms of the members' keys
  uint32_t* ws_po;      // workspace, parts > 1: [lists, parts, G, 128] normalised partial outputs (fp32 bits)
  uint32_t* ws_plse;    // workspace, parts > 1: [lists, parts, G] their base-2 log-sum-exps
  uint32_t* keys;       // workspace: [lists, max_pages_per_seq * 16] (token keys, or block keys)
  float* scores;        // workspace, strided blocks only: [lists, max_pages_per_seq * 16]
  int block, stride;    // strided blocks only
  int list_cap;         // entries of the LDS token list
  int region0_bytes;    // K staging (and, LDSK, the key array under it) in front of the token list
  int batch, num_q_heads, num_kv_heads, group;
  int topk, sink_tokens, local_tokens, first_page_offset;
  int max_pages_per_seq, sel_stride;
  int64_t num_pages;
  float scale_log2;
};

// STRIDED = false: token-level top-k (p.topk tokens); true: strided overlapping
// blocks (p.topk blocks).  LDSK: the per-token keys / scores live in LDS instead of
// the HBM workspace (one workgroup per list, the sequence short enough).  F16: float16 tensors.
// Dynamic LDS: region 0 (p.region0_bytes: K staging attend_lds_bytes(NW), which the keys
// of an LDSK kernel share: they are dead when the attention starts) | int32 list[list_cap]
// | uint32 bitmap[] (strided only)
template <int NG, int NW, bool STRIDED, bool LDSK, bool F16>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void token_topk_kernel(TokenTopkParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float sm_m[NW][4 * NG];
  __shared__ float sm_l[NW][4 * NG];
  __shared__ KeySelectShared sh;
  __shared__ int sh_last;
  constexpr int NT = NW * 64;

  const int tid = threadIdx.x;
  KIN_STAMP_RESET();
  KIN_STAMP(0);
  const int list_id = blockIdx.x / p.chunks, chunk = blockIdx.x - list_id * p.chunks;
  int b, h;
  if (!xcd_list_of(list_id, p.batch, p.num_kv_heads, b, h)) return;
  const int item = b * p.num_kv_heads + h;
  const int G = p.group;
  const int64_t hq0 = (int64_t)b * p.num_q_heads + (int64_t)h * G;

  const int ps = p.page_indptr[b], pe = p.page_indptr[b + 1];
  const int n_pages = pe - ps;
  const int last_len = p.last_page_len[b];
  const int kv_len = (n_pages - 1) * kPageSize + min(max(last_len, 1), kPageSize);
  const int seq_len = kv_len - p.first_page_offset;  // tokens of the sequence
  int32_t* sel_out = p.sel_tokens ? p.sel_tokens + (int64_t)item * p.sel_stride : nullptr;
  if (n_pages <= 0 || seq_len <= 0 || n_pages > p.max_pages_per_seq) {
    // Nothing to attend (or a sequence longer than the scratch array was sized for:
    // reported as count -1 rather than written past its end).
    if (chunk) return;
    if (sel_out)
      for (int i = tid; i < p.sel_stride; i += NT) sel_out[i] = -1;
    if (p.sel_count && tid == 0) p.sel_count[item] = (n_pages > p.max_pages_per_seq) ? -1 : 0;
    for (int i = tid; i < G * kHeadDim; i += NT) p.out[hq0 * kHeadDim + i] = 0;
    if (p.lse && tid < G) p.lse[hq0 + tid] = kNegInf;
    return;
  }

  int32_t* list = reinterpret_cast<int32_t*>(smem + p.region0_bytes);
  TokenArgs t;
  t.q_bh = p.q + hq0 * kHeadDim;
  t.kvb = reinterpret_cast<const char*>(p.kv) + (int64_t)h * kRowBytes;
  t.row_bytes = p.num_kv_heads * kRowBytes;
  t.page_bytes = 2 * kPageSize * t.row_bytes;
  t.span = t.page_bytes - h * kRowBytes;
  t.num_pages = p.num_pages;
  t.G = G;
  t.table = p.page_indices + ps;
  t.n_pages = n_pages;
  t.pad = p.first_page_offset;
  t.n_sink = min(p.sink_tokens, seq_len);
  t.n_local = min(p.local_tokens, seq_len - t.n_sink);
  t.n_dyn = seq_len - t.n_sink - t.n_local;
  t.topk = p.topk;
  t.keys = p.keys + (int64_t)item * p.max_pages_per_seq * kPageSize;
  t.lds_keys = reinterpret_cast<uint32_t*>(smem);
  t.list = list;
  t.sel_tokens = sel_out;
  t.rotate = (unsigned)item * 2654435761u >> 12;  // a different starting point for every list
  StridedArgs sa;
  if (STRIDED) {
    sa.block = p.block;
    sa.stride = p.stride;
    sa.topk_blocks = p.topk;
    sa.scores = p.scores + (int64_t)item * p.max_pages_per_seq * kPageSize;
    sa.block_keys = t.keys;
    sa.bitmap = reinterpret_cast<uint32_t*>(list + p.list_cap);
    // the K staging area is idle until the attention starts (and the LDS scores are dead once the
    // block keys exist): 2 * topk_blocks <= 2 * kMaxTopkTokens block numbers fit its
    // attend_lds_bytes(4) = 32 KiB
    sa.winners = reinterpret_cast<int32_t*>(smem);
  }
  const bool scored = STRIDED ? strided_needs_scores(t, sa) : token_needs_scores(t);
  const bool team = p.parts > 1;  // several members select and attend
  if (!scored && chunk && !team) return;  // nothing to share: chunk 0 does the list alone
  if (team && chunk >= p.parts && !scored) return;
  bool first_digit_counted = !STRIDED && (p.chunks == 1 || team);
  if (scored) {
    const int per = ((n_pages + p.chunks - 1) / p.chunks + 3) & ~3;  // whole quads of pages
    const int pg0 = min(chunk * per, n_pages), pg1 = min(pg0 + per, n_pages);
    if (first_digit_counted) {
      if (tid < 256) sh.hist[0][tid] = 0;
      __syncthreads();
    }
    if (STRIDED) strided_score_tokens<NW, LDSK, F16>(t, sa, pg0, pg1);
    else token_score_keys<NW, LDSK, F16>(t, pg0, pg1, first_digit_counted ? sh.hist[0] : nullptr);
    // Every wave waits for its own stores to be acknowledged; after the barrier the
    // workgroup's scores are in memory.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    KIN_STAMP(50);  // this workgroup's share of the tokens is scored
    if (p.chunks > 1) {
      // The slices meet through memory without cache maintenance: scores, histograms and the
      // arrival counters are written and read at device scope.
      uint32_t* my_hist = p.ws_hist + ((int64_t)item * p.chunks + chunk) * 256;
      if (team && !STRIDED) {
        if (tid < 256) __hip_atomic_store(my_hist + tid, sh.hist[0][tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
      }
      if (!team) {
        // Whoever counts in last sees everybody's scores and carries on alone; the others are done.
        if (tid == 0)
          sh_last = (__hip_atomic_fetch_add(&p.count[item], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.chunks - 1)
                        ? 1 : 0;
        __syncthreads();
        if (!sh_last) return;
      } else {
        if (tid == 0) __hip_atomic_fetch_add(&p.count[item], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (chunk >= p.parts) return;  // a member that only scores is done
        // The members that go on need everybody's scores.  The wait is bounded, and a member whose
        // patience runs out scores the whole list for itself (the same values land in the same
        // places): an optimisation, never a dependency between workgroups.
        if (tid == 0) {
          int seen = __hip_atomic_load(&p.count[item], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          for (int spins = 0; seen < p.chunks && spins < p.spin_limit; ++spins) {
            __builtin_amdgcn_s_sleep(4);
            seen = __hip_atomic_load(&p.count[item], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          sh_last = seen >= p.chunks ? 1 : 0;
        }
        __syncthreads();
        if (__builtin_amdgcn_readfirstlane(sh_last)) {
          if (!STRIDED) {
            // The list's first-digit histogram is the sum of the members': every thread takes one bin of
            // every (NT / 256)-th member, 16 loads in flight at a time (reads past the last member return 0).
            if (tid < 256) sh.hist[0][tid] = 0;
            __syncthreads();
            const __amdgpu_buffer_rsrc_t rh = make_rsrc(p.ws_hist + (int64_t)item * p.chunks * 256, p.chunks * 256 * 4);
            constexpr int kStep = NT / 256;
            const int bin = tid & 255;
            uint32_t sum = 0;
            for (int c0 = tid >> 8; c0 < p.chunks; c0 += 16 * kStep) {
              uint32_t x[16];
#pragma unroll
              for (int i = 0; i < 16; ++i)
                x[i] = __builtin_amdgcn_raw_buffer_load_b32(rh, ((c0 + i * kStep) * 256 + bin) * 4, 0, kDeviceScope);
#pragma unroll
              for (int i = 0; i < 16; ++i) sum += x[i];
            }
            if (sum) atomicAdd(&sh.hist[0][bin], sum);
          }
        } else {
          if (!STRIDED) {
            if (tid < 256) sh.hist[0][tid] = 0;
            __syncthreads();
            token_score_keys<NW, LDSK, F16>(t, 0, n_pages, sh.hist[0]);
          } else {
            strided_score_tokens<NW, LDSK, F16>(t, sa, 0, n_pages);
          }
          __builtin_amdgcn_s_waitcnt(0);
        }
        __syncthreads();
      }
    }
  }
  if (team && chunk != 0) t.sel_tokens = nullptr;  // the token positions are reported once, by member 0
  KIN_STAMP(51);  // every share is scored: the select starts
  int n;
  if constexpr (STRIDED && !LDSK) {
    if (team && p.stage_scores && scored) {
      // One wide trip brings the sequence's scores on chip: the block means then cost LDS reads
      // instead of a chain of memory round trips per thread (30 of 85 us at 8 lists of 32 K tokens).
      load_shared_keys<NT>(reinterpret_cast<const uint32_t*>(sa.scores), n_pages * kPageSize, t.lds_keys);
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      n = strided_select_list<NG, NW, true>(t, sa, &sh);
    } else {
      n = strided_select_list<NG, NW, false>(t, sa, &sh);
    }
  } else {
    n = STRIDED ? strided_select_list<NG, NW, LDSK>(t, sa, &sh) : token_select_list<NG, NW, LDSK>(t, &sh, first_digit_counted);
  }
  KIN_STAMP(52);  // token list ready
  if (sel_out && (!team || chunk == 0))
    for (int i = n + tid; i < p.sel_stride; i += NT) sel_out[i] = -1;
  if (p.sel_count && tid == 0 && (!team || chunk == 0)) p.sel_count[item] = n;
  // This member's share of the list: whole tiles of 16 entries.
  int e0 = 0, e1 = n;
  if (team) {
    const int per = (((n + p.parts - 1) / p.parts) + kPageSize - 1) & ~(kPageSize - 1);
    e0 = min(chunk * per, n);
    e1 = min(e0 + per, n);
  }

  AttendArgs a;
  a.q_bh = t.q_bh;
  a.kvb = t.kvb;
  a.row_bytes = t.row_bytes;
  a.page_bytes = t.page_bytes;
  a.span = t.span;
  a.num_pages = p.num_pages;
  a.G = G;
  a.scale_log2 = p.scale_log2;
  a.n = e1 - e0;
  a.p0 = 0;
  a.p1 = a.n;
  a.last_len = kPageSize;
  a.first_skip = 0;
  a.rotate = 0;
  a.page_size = kPageSize;
  attend_tokens<NG, NW, F16>(a, list + e0, smem, sm_m, sm_l, [&](int g, int d, float o, float lse2) {
    if (team) {
      // partial result, read by a workgroup that may sit on another XCD: device-scope stores
      const int64_t row = ((int64_t)item * p.parts + chunk) * G + g;
      __hip_atomic_store(p.ws_po + row * kHeadDim + d, __float_as_uint(o), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (d == 0) __hip_atomic_store(p.ws_plse + row, __float_as_uint(lse2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      p.out[(hq0 + g) * kHeadDim + d] = (uint16_t)f32_to_elem<F16>(o);
      if (p.lse && d == 0) p.lse[hq0 + g] = lse2 * kLn2;
    }
  });
  KIN_STAMP(53);  // listed tokens attended
  if (!team) return;
  // Every wave waits for its partial stores to be acknowledged, then the workgroup counts in;
  // whoever counts in last sees all parts and merges them.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0)
    sh_last = (__hip_atomic_fetch_add(&p.count2[item], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.parts - 1) ? 1 : 0;
  __syncthreads();
  if (!__builtin_amdgcn_readfirstlane(sh_last)) return;
  merge_list_parts<NT, F16>(smem, p.ws_po, p.ws_plse, item, p.parts, G, p.out + hq0 * kHeadDim, p.lse ? p.lse + hq0 : nullptr);
  KIN_STAMP(45);  // parts merged
}

}  // namespace kin

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

// Shared by the two entry points.  topk counts tokens (block == 0) or blocks.
static int launch_token_policy(const char* fn, bool f16, const kin_bf16_t* q, const kin_bf16_t* kv_cache,
                               const int32_t* page_indices, const int32_t* page_indptr, const int32_t* last_page_len,
                               int topk, int block, int stride, int sink_tokens, int local_tokens,
                               int first_page_offset, int32_t* sel_tokens, int32_t* sel_count, kin_bf16_t* out,
                               float* lse, void* workspace, size_t workspace_bytes, int batch, int num_q_heads,
                               int num_kv_heads, int head_dim, int page_size, int64_t num_pages,
                               int max_pages_per_seq, int sel_stride, float sm_scale, kin_stream_t stream) {
  const bool strided = block > 0;
  if (!q || !kv_cache || !page_indices || !page_indptr || !last_page_len || !out)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_common_dims(fn, batch, num_q_heads, num_kv_heads, head_dim, page_size);
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
      p.ws_plse = p.ws_po + (size_t)items * parts * p.group * kHeadDim;
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
#define KIN_TOKEN_KERNEL(NG_, NW_, S_, L_)                                                   \
  (f16 ? reinterpret_cast<const void*>(&token_topk_kernel<NG_, NW_, S_, L_, true>)           \
       : reinterpret_cast<const void*>(&token_topk_kernel<NG_, NW_, S_, L_, false>))
#define KIN_TOKEN_PICK(NG_, S_)                                                             \
  (ldsk ? (nw == 12 ? KIN_TOKEN_KERNEL(NG_, 12, S_, true) : KIN_TOKEN_KERNEL(NG_, 4, S_, true)) \
        : (nw == 12 ? KIN_TOKEN_KERNEL(NG_, 12, S_, false) : nw == 8 ? KIN_TOKEN_KERNEL(NG_, 8, S_, false) : KIN_TOKEN_KERNEL(NG_, 4, S_, false)))
  const void* kernel;
  if (strided)
    kernel = p.group <= 4 ? KIN_TOKEN_PICK(1, true) : KIN_TOKEN_PICK(4, true);
  else
    kernel = p.group <= 4 ? KIN_TOKEN_PICK(1, false) : KIN_TOKEN_PICK(4, false);
#undef KIN_TOKEN_PICK
#undef KIN_TOKEN_KERNEL
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
  if (batch <= 0 || num_kv_heads <= 0 || max_pages_per_seq <= 0) return 0;
  const int64_t lists = (int64_t)batch * num_kv_heads;
  return kin::token_count_bytes(lists) + (size_t)lists * max_pages_per_seq * kin::kPageSize * sizeof(uint32_t) +
         kin::token_team_bytes(lists, kin::token_score_chunks(lists, max_pages_per_seq));
}

size_t kin_strided_topk_workspace_bytes(int batch, int num_kv_heads, int max_pages_per_seq) {
  if (batch <= 0 || num_kv_heads <= 0 || max_pages_per_seq <= 0) return 0;
  const int64_t lists = (int64_t)batch * num_kv_heads;
  return kin::token_count_bytes(lists) + 2 * (size_t)lists * max_pages_per_seq * kin::kPageSize * sizeof(uint32_t) +
         kin::token_team_bytes(lists, kin::token_score_chunks(lists, max_pages_per_seq));
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
