// Fused decode step: append -> score -> select -> attend in ONE launch, one
// workgroup of NW waves per (sequence, KV head): 4 waves when there are enough
// lists to fill the GPU, 8 when there are few (one workgroup per CU).  With lists
// for at most half the CUs, several workgroups share a list (see StepParams).
//
// Compared with the three stand-alone kernels this removes two dependent
// dispatches, the selector's drain (its last workgroups finish their LDS-only
// select phase with the memory system idle) and the attention kernel's ramp-up;
// workgroups drift out of phase, so one workgroup's select overlaps its
// neighbours' streaming.  The selected page ids stay in LDS (HBM copies are
// optional outputs).  Same building blocks and arithmetic as the stand-alone
// kernels: score_select() (kin_select.h) and attend_list() (kin_attend.h).
#include <atomic>

#include "kin_append.h"
#include "kin_attend.h"
#include "kin_select.h"

namespace kin {

struct StepParams {
  const uint16_t* q;
  const uint32_t* k;  // new token's K/V rows as dwords; null = no append
  const uint32_t* v;
  uint16_t* kv;
  uint16_t* kbar;
  const int32_t* page_indices;
  const int32_t* page_indptr;
  const int32_t* last_page_len;
  int32_t* sel_pages;  // optional HBM copy of the page lists
  int32_t* sel_count;  // optional
  uint16_t* out;
  float* lse;  // optional
  int batch, num_q_heads, num_kv_heads, group;
  int kbar_pages, sel_stride, topk, sink_pages, local_tokens, first_page_offset, sort_cap, page_size;
  int region0_bytes;  // LDS: max(attend staging, select scratch); the page list follows it
  // Split scoring (few, long sequences): `chunks` workgroups per list score a slice of the
  // candidates each into ws_keys; the last one to finish selects and attends.
  int chunks;
  int32_t* ws_count;   // [lists], zero at launch and left zero
  uint32_t* ws_keys;   // [lists, score_key_stride(kbar_pages)]
  // Split attention (lists for at most half the CUs): `parts` workgroups per list.  Each scores
  // and selects the whole list for itself (identical results), attends its share of the listed
  // pages and leaves a partial result; the last one to finish merges them.
  int parts;
  uint32_t* ws_po;    // [lists, parts, group, 128] fp32 bits: normalised partial outputs
  uint32_t* ws_plse;  // [lists, parts, group] fp32 bits: base-2 log-sum-exp of the parts
  int64_t num_pages;
  float scale_log2;
  int deep_score;      // few lists: more mean-key loads in flight per lane (see the kernel)
  int rotate;          // attend_rotates(lists)
};

template <int NG, int NW, bool F16>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void blocktopk_step_kernel(StepParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float sm_m[NW][4 * NG];
  __shared__ float sm_l[NW][4 * NG];
  constexpr int NT = NW * 64;

  __shared__ int sh_last;
  const int tid = threadIdx.x;
  int b, h, chunk = 0, part = 0;
  if (p.chunks > 1 || p.parts > 1) {
    const int per_list = p.chunks > 1 ? p.chunks : p.parts;
    const int list = blockIdx.x / per_list;
    const int sub = blockIdx.x - list * per_list;
    if (p.chunks > 1) chunk = sub; else part = sub;
    b = list / p.num_kv_heads;
    h = list - b * p.num_kv_heads;
  } else if (!xcd_list_of(blockIdx.x, p.batch, p.num_kv_heads, b, h)) {
    return;
  }
  const int item = b * p.num_kv_heads + h;
  const int G = p.group;
  const int64_t hq0 = (int64_t)b * p.num_q_heads + (int64_t)h * G;

  const int ps = p.page_indptr[b], pe = p.page_indptr[b + 1];
  const int n_pages = pe - ps;
  if (n_pages <= 0) {  // empty sequence: nothing to append, select or attend
    if (chunk != 0 || part != 0) return;
    if (p.sel_pages)
      for (int i = tid; i < p.sel_stride; i += NT) p.sel_pages[(int64_t)item * p.sel_stride + i] = -1;
    if (p.sel_count && tid == 0) p.sel_count[item] = 0;
    for (int i = tid; i < G * kHeadDim; i += NT) p.out[hq0 * kHeadDim + i] = 0;
    if (p.lse && tid < G) p.lse[hq0 + tid] = kNegInf;
    return;
  }
  const int last_len = p.last_page_len[b];

  // ---- append (wave 0): same byte moves and mean-key update as append_kernel ----
  // With split scoring the workgroup that ends up attending does it (see below).
  auto append_token = [&]() {
    if (p.k != nullptr && tid < 64) {
      uint32_t* kbar_row =
          reinterpret_cast<uint32_t*>(p.kbar) + kbar_row_index(b, h, n_pages - 1, p.num_kv_heads, p.kbar_pages) * (kHeadDim / 2);
      append_token_row<F16>(p.k + (int64_t)item * (kHeadDim / 2), p.v + (int64_t)item * (kHeadDim / 2),
                       reinterpret_cast<uint32_t*>(p.kv), kbar_row, p.page_indices[pe - 1], last_len, n_pages, p.kbar_pages, h,
                       p.num_kv_heads, p.num_pages, tid, p.page_size);
      // The attention phase of this workgroup reads the row back: make the stores
      // visible before the barriers that separate the phases.
      __threadfence_block();
    }
  };
  if (p.chunks <= 1 && p.parts <= 1) append_token();

  // ---- score + select: page list into LDS -------------------------------------
  int32_t* sel_lds = reinterpret_cast<int32_t*>(smem + p.region0_bytes);
  SelectArgs s;
  s.q_bh = p.q + hq0 * kHeadDim;
  s.G = G;
  s.n_pages = n_pages;
  split_pages(n_pages, last_len, p.sink_pages, p.local_tokens, p.kbar_pages, p.page_size, s.n_sink, s.n_cand, s.n_local);
  s.kb = reinterpret_cast<const char*>(p.kbar) + kbar_row_index(b, h, s.n_sink, p.num_kv_heads, p.kbar_pages) * kRowBytes;
  s.topk = p.topk;
  s.table = p.page_indices + ps;
  s.sel_logical = nullptr;
  s.scores_out = nullptr;
  s.keys = reinterpret_cast<uint32_t*>(smem);
  s.sortbuf = reinterpret_cast<unsigned long long*>(smem + (size_t)((p.kbar_pages + 3) & ~3) * 4);
  s.sort_cap = p.sort_cap;
  int n;
  if (p.chunks > 1) {
    // This workgroup's slice of the candidates -> keys in HBM.
    uint32_t* gkeys = p.ws_keys + (int64_t)item * score_key_stride(p.kbar_pages);
    const int n_score = min(s.topk, s.n_cand) > 0 ? s.n_cand : 0;
    const int per = ((n_score + p.chunks - 1) / p.chunks + 63) & ~63;
    const int r0 = min(chunk * per, n_score), r1 = min(r0 + per, n_score);
    score_rows<4, NT, true, F16>(s, r0, r1, gkeys);
    // The slices meet through memory without cache maintenance: keys and the
    // arrival counter are written and read at device scope (they bypass the
    // XCD-private L2), and every wave waits for its own stores to be acknowledged
    // before the workgroup counts in.  Whoever counts in last sees everybody's
    // keys and carries on alone; the others are done.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0)
      sh_last = (__hip_atomic_fetch_add(&p.ws_count[item], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.chunks - 1)
                    ? 1 : 0;
    __syncthreads();
    if (!sh_last) return;
    if (tid == 0) __hip_atomic_store(&p.ws_count[item], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    append_token();
    load_shared_keys<NT>(gkeys, n_score, s.keys);
    __syncthreads();
    n = select_from_keys<NT>(s, sel_lds);
  } else {
    // Mean-key loads in flight per lane.  4 saturate HBM while several rounds of workgroups overlap
    // (4096 lists; more only lengthens the last pass of short lists).  With fewer lists the workgroups
    // score in step and each has to keep 64 KiB in flight: 16 / 8 loads at 4 / 8 waves
    // (1024 lists of 2048 pages: 5 % faster than with 4).
    if (p.deep_score) {
      constexpr int kDeep = NW <= 4 ? 16 : 8;
      n = score_select<kDeep, NT, F16>(s, sel_lds);
    } else {
      n = score_select<4, NT, F16>(s, sel_lds);
    }
  }
  if (p.sel_pages && part == 0) {
    int32_t* sel = p.sel_pages + (int64_t)item * p.sel_stride;
    for (int i = tid; i < p.sel_stride; i += NT) sel[i] = (i < n) ? sel_lds[i] : -1;
  }
  if (p.sel_count && tid == 0 && part == 0) p.sel_count[item] = n;
  int p0 = 0, p1 = n;
  if (p.parts > 1) {
    const int per = (n + p.parts - 1) / p.parts;
    p0 = min(part * per, n);
    p1 = min(p0 + per, n);
    // The new token goes into the sequence's last page, which closes every list and is
    // nobody's candidate (local_tokens >= 1): the part that attends it appends it first.
    if (p1 == n && p1 > p0) {
      append_token();
      __syncthreads();
    }
  }

  // ---- attend over the listed pages (select scratch is dead: reuse as staging) ---
  AttendArgs a;
  a.q_bh = s.q_bh;
  a.kvb = reinterpret_cast<const char*>(p.kv) + (int64_t)h * kRowBytes;
  a.row_bytes = p.num_kv_heads * kRowBytes;
  a.page_bytes = 2 * p.page_size * a.row_bytes;
  a.span = a.page_bytes - h * kRowBytes;
  a.page_size = p.page_size;
  a.num_pages = p.num_pages;
  a.G = G;
  a.scale_log2 = p.scale_log2;
  a.n = n;
  a.p0 = p0;
  a.p1 = p1;
  a.last_len = last_len;
  a.first_skip = p.first_page_offset;
  a.rotate = p.rotate ? attend_rotation(item, part) : 0u;
  attend_list<NG, NW, F16>(
      a, [&](int i) -> int { return __builtin_amdgcn_readfirstlane(sel_lds[i]); }, smem, sm_m, sm_l,
      [&](int g, int d, float o, float lse2) {
        if (p.parts > 1) {
          // partial result, read by a workgroup that may sit on another XCD: device-scope stores
          const int64_t row = ((int64_t)item * p.parts + part) * G + g;
          __hip_atomic_store(p.ws_po + row * kHeadDim + d, __float_as_uint(o), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (d == 0) __hip_atomic_store(p.ws_plse + row, __float_as_uint(lse2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          p.out[(hq0 + g) * kHeadDim + d] = (uint16_t)f32_to_elem<F16>(o);
          if (p.lse && d == 0) p.lse[hq0 + g] = lse2 * kLn2;
        }
      });
  if (p.parts <= 1) return;
  // Every wave waits for its partial stores to be acknowledged, then the workgroup counts in;
  // whoever counts in last sees all parts and merges them (as merge_splits_kernel does).
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0)
    sh_last = (__hip_atomic_fetch_add(&p.ws_count[item], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.parts - 1) ? 1 : 0;
  __syncthreads();
  if (!sh_last) return;
  if (tid == 0) __hip_atomic_store(&p.ws_count[item], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
  // The parts' log-sum-exps become weights in LDS (the attention's staging area is dead), then every
  // thread sums its output element over the parts with independent device-scope loads.
  float* wl = reinterpret_cast<float*>(smem);  // [parts][G] weights, then [G] denominators
  float* den_g = wl + p.parts * G;
  const int64_t first_row = (int64_t)item * p.parts * G;
  const __amdgpu_buffer_rsrc_t rl = make_rsrc(p.ws_plse + first_row, p.parts * G * (int)sizeof(float));
  for (int i = tid; i < p.parts * G; i += NT)
    wl[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rl, i * 4, 0, kDeviceScope));
  __syncthreads();
  if (tid < G) {
    float mm = kNegInf;
    for (int sp = 0; sp < p.parts; ++sp) mm = fmaxf(mm, wl[sp * G + tid]);
    const float m_safe = (mm == kNegInf) ? 0.f : mm;
    float den = 0.f;
    for (int sp = 0; sp < p.parts; ++sp) {
      const float wgt = fast_exp2(wl[sp * G + tid] - m_safe);
      wl[sp * G + tid] = wgt;
      den += wgt;
    }
    den_g[tid] = den;
    if (p.lse) p.lse[hq0 + tid] = (den > 0.f) ? (mm + fast_log2(den)) * kLn2 : kNegInf;
  }
  __syncthreads();
  const __amdgpu_buffer_rsrc_t ro = make_rsrc(p.ws_po + first_row * kHeadDim, p.parts * G * kHeadDim * (int)sizeof(float));
  for (int idx = tid; idx < G * kHeadDim; idx += NT) {
    const int g = idx >> 7, d = idx & (kHeadDim - 1);
    float num = 0.f;
#pragma unroll 8
    for (int sp = 0; sp < p.parts; ++sp)
      num += __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ro, ((sp * G + g) * kHeadDim + d) * 4, 0, kDeviceScope)) *
             wl[sp * G + g];
    const float den = den_g[g];
    p.out[(hq0 + g) * kHeadDim + d] = (uint16_t)f32_to_elem<F16>(den > 0.f ? num / den : 0.f);
  }
}

}  // namespace kin

namespace kin {

// How the workgroups of a launch share the lists.  chunks > 1: split scoring (few lists
// with many candidates); parts > 1: split attention (lists for at most half the CUs);
// never both.  need: workspace bytes of the mode chosen (arrival counters first).
struct StepPlan {
  int chunks, parts;
  size_t need;
};

constexpr int kMaxParts = 64;

static size_t parts_workspace_bytes(int64_t items, int parts, int group) {
  return score_count_bytes(items) + (size_t)items * parts * group * (kHeadDim + 1) * sizeof(float);
}

// list_tiles: upper bound of the 16-token tiles a page list holds.  avail: bytes the caller's
// workspace has (a smaller one gets fewer parts, or none, never an error).
//
// Split attention: as many parts as keep the launch at one workgroup per CU, each with at
// least four tiles for each of its 8 waves (below that the merge costs more than it saves;
// 64 lists x 4 parts of k = 128 pages: 48 us against 46 in 2 parts and 47 whole; a launch
// that fills every CU wants longer lists still: 128 lists x 2 parts lose 6 % at k = 128
// and gain 5 % at k = 512).  Every part
// scores the whole list for itself, ~7 ns per mean key on one CU (more once over 128
// workgroups pull whole lists through HBM at the same time), where split scoring takes a
// few us for any length; a tile costs the lone attending workgroup ~0.15 us.  So where the
// shape could split its scoring instead, parts are taken only if they save more attention
// than the repeated scoring costs (8 lists of 4097 pages, k = 512: 59 us in parts, 103 us
// with split scoring; k = 128: 49 against 43; one list of 2049 pages, k = 128: 30 against 37).
static StepPlan plan_step(int batch, int num_kv_heads, int group, int kbar_pages, int64_t list_tiles, size_t avail) {
  const int64_t items = (int64_t)batch * num_kv_heads;
  StepPlan plan{1, 1, 0};
  if (items <= 0) return plan;
  const int chunks = score_chunks(batch, num_kv_heads, kbar_pages);
  int64_t parts = 1;
  if (items * 2 <= kNumCus && list_tiles >= (items * 2 <= kNumCus - 32 ? 96 : 384)) {
    parts = kNumCus / items;
    const int64_t by_work = list_tiles / 32;
    if (parts > by_work) parts = by_work;
    if (parts > kMaxParts) parts = kMaxParts;
    while (parts > 1 && parts_workspace_bytes(items, (int)parts, group) > avail) parts /= 2;
    if (parts < 1) parts = 1;
  }
  const bool chunks_fit = chunks > 1 && score_workspace_bytes(items, kbar_pages) <= avail;
  if (parts > 1 && chunks_fit) {
    const int64_t groups = items * parts;  // workgroups that would each score a whole list
    if (24 * (list_tiles - list_tiles / parts) * 128 <= (int64_t)kbar_pages * (groups > 128 ? groups : 128)) parts = 1;
  }
  if (parts > 1) {
    plan.parts = (int)parts;
    plan.need = parts_workspace_bytes(items, plan.parts, group);
  } else if (chunks_fit) {
    plan.chunks = chunks;
    plan.need = score_workspace_bytes(items, kbar_pages);
  }
  return plan;
}

}  // namespace kin

extern "C" size_t kin_step_workspace_bytes(int batch, int num_kv_heads, int kbar_pages) {
  // Enough for whichever mode the launch picks, whatever the group size and page budget.
  const int64_t items = (int64_t)batch * num_kv_heads;
  if (items <= 0) return 0;
  size_t need = 0;
  if (kin::score_chunks(batch, num_kv_heads, kbar_pages) > 1) need = kin::score_workspace_bytes(items, kbar_pages);
  if (items * 2 <= kin::kNumCus) {
    int64_t parts = kin::kNumCus / items;
    if (parts > kin::kMaxParts) parts = kin::kMaxParts;
    const size_t split = kin::parts_workspace_bytes(items, (int)parts, kin::kMaxGroup);
    if (split > need) need = split;
  }
  return need;
}

namespace kin {

// Validation and launch shared by kin_blocktopk_decode_step (workspace from the
// caller) and kin_blocktopk_decode_step_static (workspace = this library's own
// device array).  fn: the entry point's name, for error messages.
static int launch_step(const char* fn, bool f16, const uint16_t* q, const uint16_t* k, const uint16_t* v,
                       uint16_t* kv_cache, uint16_t* kbar, const int32_t* page_indices,
                       const int32_t* page_indptr, const int32_t* last_page_len, int topk, int sink_pages,
                       int local_tokens, int32_t* sel_pages, int32_t* sel_count, kin_bf16_t* out, float* lse,
                       int batch, int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                       int64_t num_pages, int kbar_pages, int sel_stride, int first_page_offset, float sm_scale,
                       void* workspace, size_t workspace_bytes, kin_stream_t stream) {
  if (!q || !kv_cache || !kbar || !page_indices || !page_indptr || !last_page_len || !out)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if ((k == nullptr) != (v == nullptr))
    return fail(KIN_ERR_NULL_POINTER, "%s: k and v must both be given or both be null", fn);
  int st = check_common_dims(fn, batch, num_q_heads, num_kv_heads, head_dim, page_size);
  if (st) return st;
  if (num_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_pages=%lld must be >= 1", fn, (long long)num_pages);
  if (topk < 0) return fail(KIN_ERR_BAD_SHAPE, "%s: topk=%d is negative", fn, topk);
  if (kbar_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: kbar_pages=%d must be >= 1", fn, kbar_pages);
  st = check_fixed_pages(fn, sink_pages, local_tokens);
  if (st) return st;
  st = check_first_page_offset(fn, first_page_offset, page_size);
  if (st) return st;
  if (first_page_offset > 0 && sink_pages < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: first_page_offset=%d needs sink_pages >= 1 (a padded page has no mean key)", fn,
                first_page_offset);
  const int list_cap = topk + sink_pages + max_local_pages(local_tokens);
  if (sel_pages && sel_stride < list_cap)
    return fail(KIN_ERR_BAD_SHAPE, "%s: sel_stride=%d must be at least kin_sel_list_capacity(topk, sink_pages, local_tokens) = %d",
                fn, sel_stride, list_cap);
  if (sel_pages && !sel_count) return fail(KIN_ERR_NULL_POINTER, "%s: sel_pages given without sel_count", fn);
  if (topk > kMaxTopk) return fail(KIN_ERR_UNSUPPORTED, "%s: topk=%d exceeds the limit %d", fn, topk, kMaxTopk);
  if (kbar_pages > kMaxCandidates)
    return fail(KIN_ERR_UNSUPPORTED, "%s: kbar_pages=%d exceeds the limit %d", fn, kbar_pages, kMaxCandidates);
  if (!aligned16(q) || !aligned16(kv_cache) || !aligned16(kbar) || !aligned16(out) || (k && !aligned16(k)) ||
      (v && !aligned16(v)))
    return fail(KIN_ERR_MISALIGNED, "%s: q, k, v, kv_cache, kbar and out must be 16-byte aligned", fn);
  if (batch == 0) return KIN_OK;

  StepParams p;
  p.q = q;
  p.k = reinterpret_cast<const uint32_t*>(k);
  p.v = reinterpret_cast<const uint32_t*>(v);
  p.kv = kv_cache;
  p.kbar = kbar;
  p.page_indices = page_indices;
  p.page_indptr = page_indptr;
  p.last_page_len = last_page_len;
  p.sel_pages = sel_pages;
  p.sel_count = sel_count;
  p.out = out;
  p.lse = lse;
  p.batch = batch;
  p.num_q_heads = num_q_heads;
  p.num_kv_heads = num_kv_heads;
  p.group = num_q_heads / num_kv_heads;
  p.kbar_pages = kbar_pages;
  p.sel_stride = sel_stride;
  p.topk = topk;
  p.sink_pages = sink_pages;
  p.local_tokens = local_tokens;
  p.first_page_offset = first_page_offset;
  p.page_size = page_size;
  p.sort_cap = select_sort_cap(topk, kbar_pages);
  // Waves per workgroup.  The kernels hold 140-145 registers, so a CU runs 12 waves: three
  // 4-wave workgroups, or one of 8 while the lists are no more than the CUs (measured: 8 waves
  // beat 4, 6, 12 and a 16-wave build that spills, by 2-20 %; from 257 lists on, 8-wave
  // workgroups would take two rounds and 4 waves win by 3-25 %).
  const int64_t items = (int64_t)batch * num_kv_heads;
  if (xcd_grid_size(batch, num_kv_heads) > 0x7fffffffLL)
    return fail(KIN_ERR_UNSUPPORTED, "%s: batch*num_kv_heads too large", fn);
  const int nw = items <= kNumCus ? 8 : 4;
  // Few lists: several workgroups share one (split attention, or split scoring for very long sequences).
  const StepPlan plan = plan_step(batch, num_kv_heads, p.group, kbar_pages, (int64_t)list_cap << page_tile_shift(page_size),
                                  workspace && aligned16(workspace) ? workspace_bytes : 0);
  p.chunks = plan.chunks;
  p.parts = plan.parts;
  p.ws_count = nullptr;
  p.ws_keys = nullptr;
  p.ws_po = nullptr;
  p.ws_plse = nullptr;
  if (plan.chunks > 1 || plan.parts > 1) {
    char* after_counters = static_cast<char*>(workspace) + score_count_bytes(items);
    p.ws_count = static_cast<int32_t*>(workspace);
    if (plan.chunks > 1) {
      p.ws_keys = reinterpret_cast<uint32_t*>(after_counters);
    } else {
      p.ws_po = reinterpret_cast<uint32_t*>(after_counters);
      p.ws_plse = p.ws_po + (size_t)items * plan.parts * p.group * kHeadDim;
    }
  }
  p.deep_score = items < 4096 ? 1 : 0;
  p.rotate = attend_rotates(items) ? 1 : 0;
  const size_t sel_scratch = select_lds_bytes(kbar_pages, p.sort_cap);
  const size_t attend_bytes = (size_t)attend_lds_bytes(nw);
  size_t region0 = sel_scratch > attend_bytes ? sel_scratch : attend_bytes;
  region0 = (region0 + 15) & ~(size_t)15;
  p.region0_bytes = (int)region0;
  p.num_pages = num_pages;
  const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim);
  p.scale_log2 = scale * 1.4426950408889634f;
  const size_t lds = region0 + (size_t)list_cap * 4;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const void* kernel;
#define KIN_STEP_KERNEL(NG_, NW_)                                                        \
  (f16 ? reinterpret_cast<const void*>(&blocktopk_step_kernel<NG_, NW_, true>)           \
       : reinterpret_cast<const void*>(&blocktopk_step_kernel<NG_, NW_, false>))
  if (p.group <= 4)
    kernel = nw == 8 ? KIN_STEP_KERNEL(1, 8) : KIN_STEP_KERNEL(1, 4);
  else
    kernel = nw == 8 ? KIN_STEP_KERNEL(4, 8) : KIN_STEP_KERNEL(4, 4);
#undef KIN_STEP_KERNEL
  if (lds > 48 * 1024) {
    // Above the default dynamic-LDS allowance the runtime wants an explicit opt-in.
    st = check_hip(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds),
                   "hipFuncSetAttribute(blocktopk_step_kernel)");
    if (st) return st;
  }
  unsigned grid = (unsigned)xcd_grid_size(batch, num_kv_heads);
  if (p.chunks > 1 || p.parts > 1) {
    // the arrival counters start at zero (a fill kernel, so that the launch pair can be captured in a graph)
    fill_zero_i32_kernel<<<(unsigned)((items + 255) / 256), 256, 0, s>>>(p.ws_count, (int)items);
    st = check_hip(hipGetLastError(), "fill_zero_i32_kernel launch");
    if (st) return st;
    grid = (unsigned)(items * (p.chunks > 1 ? p.chunks : p.parts));
  }
  void* args[] = {&p};
  st = check_hip(hipLaunchKernel(kernel, dim3(grid), dim3(nw * 64), args, lds, s), "blocktopk_step_kernel launch");
  return st;
}

// ---- device memory of the entry point that allocates nothing -------------------
// Workspace of the launches that share lists between workgroups (arrival counters,
// then keys or partial results) for callers that cannot bring one.  Every GPU the library's code object is loaded on holds its own copy
// until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels get the address that call returns.
constexpr size_t kStaticScratchBytes = KIN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up once per device).
static int static_scratch_address(const char* fn, void** ptr) {
  int dev = -1;
  int st = check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (st) return st;
  if (dev < 0 || dev >= kMaxDevices) return fail(KIN_ERR_UNSUPPORTED, "%s: device ordinal %d is beyond %d", fn, dev, kMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    st = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (st) return st;
    if (!p) return fail(KIN_ERR_LAUNCH, "%s: hipGetSymbolAddress returned a null address", fn);
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing threads store the same value
  }
  *ptr = p;
  return KIN_OK;
}

}  // namespace kin

extern "C" int kin_blocktopk_decode_step(const kin_bf16_t* q, const kin_bf16_t* k, const kin_bf16_t* v,
                                         kin_bf16_t* kv_cache, kin_bf16_t* kbar, const int32_t* page_indices,
                                         const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                                         int sink_pages, int local_tokens, int32_t* sel_pages, int32_t* sel_count,
                                         kin_bf16_t* out, float* lse, int batch, int num_q_heads, int num_kv_heads,
                                         int head_dim, int page_size, int64_t num_pages, int kbar_pages,
                                         int sel_stride, int first_page_offset, float sm_scale, void* workspace,
                                         size_t workspace_bytes, kin_stream_t stream) {
  return kin::launch_step("kin_blocktopk_decode_step", false, q, k, v, kv_cache, kbar, page_indices, page_indptr,
                          last_page_len, topk, sink_pages, local_tokens, sel_pages, sel_count, out, lse, batch, num_q_heads,
                          num_kv_heads, head_dim, page_size, num_pages, kbar_pages, sel_stride, first_page_offset, sm_scale,
                          workspace, workspace_bytes, stream);
}

extern "C" int kin_blocktopk_decode_step_f16(const kin_f16_t* q, const kin_f16_t* k, const kin_f16_t* v,
                                             kin_f16_t* kv_cache, kin_f16_t* kbar, const int32_t* page_indices,
                                             const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                                             int sink_pages, int local_tokens, int32_t* sel_pages, int32_t* sel_count,
                                             kin_f16_t* out, float* lse, int batch, int num_q_heads, int num_kv_heads,
                                             int head_dim, int page_size, int64_t num_pages, int kbar_pages,
                                             int sel_stride, int first_page_offset, float sm_scale, void* workspace,
                                             size_t workspace_bytes, kin_stream_t stream) {
  return kin::launch_step("kin_blocktopk_decode_step_f16", true, q, k, v, kv_cache, kbar, page_indices, page_indptr,
                          last_page_len, topk, sink_pages, local_tokens, sel_pages, sel_count, out, lse, batch, num_q_heads,
                          num_kv_heads, head_dim, page_size, num_pages, kbar_pages, sel_stride, first_page_offset, sm_scale,
                          workspace, workspace_bytes, stream);
}

extern "C" size_t kin_static_scratch_bytes(void) { return kin::kStaticScratchBytes; }

extern "C" int kin_blocktopk_decode_step_static(const kin_bf16_t* q, const kin_bf16_t* k, const kin_bf16_t* v,
                                                kin_bf16_t* kv_cache, kin_bf16_t* kbar, const int32_t* page_indices,
                                                const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                                                int sink_pages, int local_tokens, int32_t* sel_pages,
                                                int32_t* sel_count, kin_bf16_t* out, float* lse, int batch,
                                                int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                                int64_t num_pages, int kbar_pages, int sel_stride,
                                                int first_page_offset, float sm_scale, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_blocktopk_decode_step_static";
  // What this shape's way of sharing lists between workgroups needs, from the dimensions
  // alone.  Split scoring beyond the array is an error, not a silent fall-back to the
  // slower single-workgroup scoring; split attention always fits (kMaxGroup heads included).
  size_t need = 0;
  if (batch > 0 && num_kv_heads > 0 && num_q_heads >= num_kv_heads && kbar_pages > 0 && topk >= 0 && sink_pages >= 0 &&
      local_tokens >= 1 && page_size >= kPageSize) {
    const int64_t list_cap = (int64_t)topk + sink_pages + max_local_pages(local_tokens);
    need = plan_step(batch, num_kv_heads, num_q_heads / num_kv_heads, kbar_pages, list_cap << page_tile_shift(page_size),
                     ~(size_t)0).need;
  }
  if (need > kStaticScratchBytes)
    return fail(KIN_ERR_WORKSPACE,
                "%s: batch=%d x num_kv_heads=%d lists of kbar_pages=%d need %zu bytes of scratch, the built-in array has %zu "
                "(use kin_blocktopk_decode_step with a workspace of kin_step_workspace_bytes() bytes)",
                fn, batch, num_kv_heads, kbar_pages, need, kStaticScratchBytes);
  void* ws = nullptr;
  if (need > 0) {
    const int st = static_scratch_address(fn, &ws);
    if (st) return st;
  }
  return launch_step(fn, false, q, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, topk, sink_pages, local_tokens,
                     sel_pages, sel_count, out, lse, batch, num_q_heads, num_kv_heads, head_dim, page_size, num_pages,
                     kbar_pages, sel_stride, first_page_offset, sm_scale, ws, ws ? kStaticScratchBytes : 0, stream);
}
