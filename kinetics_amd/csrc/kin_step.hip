// Fused decode step: append -> score -> select -> attend in ONE launch, one
// workgroup of NW waves per (sequence, KV head): 4 waves when there are enough
// lists to fill the GPU, 8 when there are few (one workgroup per CU).  Lists that
// would leave CUs idle -- few lists, a batch just above one list per CU, the last
// lists of a batch a little larger than the GPU holds at once -- are handled by a
// *team* of workgroups each (see StepParams).
//
// Compared with the three stand-alone kernels this removes two dependent
// dispatches, the selector's drain (its last workgroups finish their LDS-only
// select phase with the memory system idle) and the attention kernel's ramp-up;
// workgroups drift out of phase, so one workgroup's select overlaps its
// neighbours' streaming.  The selected page ids stay in LDS (HBM copies are
// optional outputs).  Same building blocks and arithmetic as the stand-alone
// kernels: score_select() (kin_select.h) and attend_list() (kin_attend.h).
#include <atomic>
#include <cstdio>
#include <cstdlib>

#include "kin_append.h"
#include "kin_attend.h"
#include "kin_select.h"
#include "kin_step.h"

namespace kin {

// A list with fewer candidates and fewer tiles to attend than this is handled by one member of its team
// alone (see the kernel): about 2.5 + 8 us of streaming for one workgroup, what a team's overhead costs.
constexpr int kTeamMinCandidates = 256;
constexpr int kTeamMinTiles = 24;

// HD: elements of a head row, 128 or 64.
template <int NG, int NW, bool F16, int HD = kHeadDim>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void blocktopk_step_kernel(StepParams p) {
  constexpr int kRowB = HD * 2;  // bytes of a head row
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float sm_m[NW][4 * NG];
  __shared__ float sm_l[NW][4 * NG];
  constexpr int NT = NW * 64;

  __shared__ int sh_last;
  __shared__ SelectScratch ss;
  const int tid = threadIdx.x;
  clear_select_scratch<NT>(&ss);
  KIN_STAMP_RESET();
  KIN_STAMP(0);
  // The first head_blocks workgroups own a list each; behind them come the teams, `team`
  // consecutive workgroups per list from list head_lists on.
  int b, h, member = 0, team = 1, parts = 1;
  if ((int)blockIdx.x >= p.head_blocks) {
    const int i = blockIdx.x - p.head_blocks;
    const int list = p.head_lists + i / p.team;
    member = i - (i / p.team) * p.team;
    team = p.team;
    parts = p.parts;
    b = list / p.num_kv_heads;
    h = list - b * p.num_kv_heads;
  } else if (p.head_lists == p.batch * p.num_kv_heads) {
    if (!xcd_list_of(blockIdx.x, p.batch, p.num_kv_heads, b, h)) return;
  } else if (p.head_lists % (kNumXcds * p.num_kv_heads) == 0) {
    // whole groups of 8 sequences in front of the teams: the same placement as without teams
    xcd_list_of(blockIdx.x, p.head_lists / p.num_kv_heads, p.num_kv_heads, b, h);
  } else {
    b = blockIdx.x / p.num_kv_heads;
    h = blockIdx.x - b * p.num_kv_heads;
  }
  const int part = member;  // members 0 .. parts-1 also select and attend a share of the page list
  const int item = b * p.num_kv_heads + h;
  const int G = p.group;
  const int64_t hq0 = (int64_t)b * p.num_q_heads + (int64_t)h * G;

  // The caller's per-slot token counter (a KV manager's kv_offset) follows the append: one thread per sequence.
  if (p.slot_lens && p.k && h == 0 && member == 0 && tid == 0) {
    const int sl = p.slot_ids ? p.slot_ids[b] : b;
    if ((unsigned)sl < (unsigned)p.num_slots) p.slot_lens[sl] += 1;
  }
  const int ps = p.page_indptr[b], pe = p.page_indptr[b + 1];
  const int n_pages = pe - ps;
  if (n_pages <= 0) {  // empty sequence: nothing to append, select or attend (every member sees that)
    if (member != 0) return;
    if (p.sel_pages)
      for (int i = tid; i < p.sel_stride; i += NT) p.sel_pages[(int64_t)item * p.sel_stride + i] = -1;
    if (p.sel_count && tid == 0) p.sel_count[item] = 0;
    for (int i = tid; i < G * HD; i += NT) p.out[hq0 * HD + i] = 0;
    if (p.lse && tid < G) p.lse[hq0 + tid] = kNegInf;
    return;
  }
  const int last_len = p.last_page_len[b];
  const int kb = kbar_block_of(p.slot_ids, p.num_slots, b);  // (a sequence without mean keys has no candidates)
  KIN_STAMP(1);  // the sequence's table entries are known

  // ---- append (wave 0): same byte moves and mean-key update as append_kernel ----
  // In a team the member that attends the sequence's last page does it (see below).
  auto append_token = [&]() {
    if (p.k != nullptr && tid < 64) {
      uint32_t* kbar_row = kb < 0 ? nullptr
                                  : reinterpret_cast<uint32_t*>(p.kbar) +
                                        kbar_row_index(kb, h, n_pages - 1, p.num_kv_heads, p.kbar_pages) * (HD / 2);
      append_token_row<F16, HD>(p.k + (int64_t)item * (HD / 2), p.v + (int64_t)item * (HD / 2),
                       reinterpret_cast<uint32_t*>(p.kv), kbar_row, p.page_indices[pe - 1], last_len, n_pages, p.kbar_pages, h,
                       p.num_kv_heads, p.num_pages, tid, p.page_size);
      // The attention phase of this workgroup reads the row back: make the stores
      // visible before the barriers that separate the phases.
      __threadfence_block();
    }
  };
  if (team == 1) append_token();
  KIN_STAMP(2);  // appended (one workgroup per list)

  // ---- score + select: page list into LDS -------------------------------------
  int32_t* sel_lds = reinterpret_cast<int32_t*>(smem + p.region0_bytes);
  SelectArgs s;
  s.q_bh = p.q + hq0 * HD;
  s.G = G;
  s.n_pages = n_pages;
  split_pages(n_pages, last_len, p.sink_pages, p.local_tokens, kb >= 0 ? p.kbar_pages : 0, p.page_size, s.n_sink, s.n_cand, s.n_local);
  s.kb = reinterpret_cast<const char*>(p.kbar) + kbar_row_index(max(kb, 0), h, s.n_sink, p.num_kv_heads, p.kbar_pages) * kRowB;
  s.topk = p.topk;
  s.table = p.page_indices + ps;
  s.sel_logical = nullptr;
  s.scores_out = nullptr;
  s.keys = reinterpret_cast<uint32_t*>(smem);
  s.sortbuf = reinterpret_cast<unsigned long long*>(smem + (size_t)((p.kbar_pages + 3) & ~3) * 4);
  s.sort_cap = p.sort_cap;
  s.ss = &ss;
  s.table_lds = nullptr;
  s.digit0_counted = false;
  s.sorted = p.sel_pages != nullptr;
  int32_t* table_lds = reinterpret_cast<int32_t*>(smem + select_table_offset(p.kbar_pages, p.sort_cap));
  int n;
  if (team > 1) {
    // Teams are planned from the batch's capacity (kbar_pages, the page budget), not from the lengths,
    // which only the GPU knows.  A list too short to be worth sharing -- the exchange, the second
    // select and the merge cost about 10 us -- is member 0's alone: the others leave at once and
    // nothing goes through the workspace.
    const int tiles = (min(s.topk, s.n_cand) + s.n_sink + s.n_local) << page_tile_shift(p.page_size);
    if (s.n_cand < kTeamMinCandidates && tiles < kTeamMinTiles) {
      if (member != 0) return;
      team = parts = 1;
      append_token();
    }
  }
  if (team > 1) {
    // This member's slice of the candidates -> keys in HBM.
    const int titem = item - p.head_lists;
    uint32_t* gkeys = p.ws_keys + (int64_t)titem * score_key_stride(p.kbar_pages);
    const int n_score = min(s.topk, s.n_cand) > 0 ? s.n_cand : 0;
    const int per = ((n_score + team - 1) / team + 63) & ~63;
    const int r0 = min(member * per, n_score), r1 = min(r0 + per, n_score);
    constexpr int kDeep = NW <= 4 ? 16 : 8;
    score_rows<kDeep, NT, true, F16, false, HD>(s, r0, r1, gkeys);
    // The slices meet through memory without cache maintenance: keys and the
    // arrival counter are written and read at device scope (they bypass the
    // XCD-private L2), and every wave waits for its own stores to be acknowledged
    // before the workgroup counts in.
    KIN_STAMP(40);  // slice issued
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    KIN_STAMP(41);  // slice scored, keys stored
    if (tid == 0) __hip_atomic_fetch_add(&p.ws_count[titem], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (member >= parts) return;  // a member that only scores is done
    // The members that go on need everybody's keys.  The others are running or about to be
    // dispatched (a team's workgroups are neighbours in the grid), so the wait is short; it is
    // bounded all the same, and a member whose patience runs out -- whatever keeps its team-mates:
    // a GPU shared with another job, a dispatch order that is no one's promise -- scores the whole
    // list for itself and gets the same keys.  The wait is an optimisation, never a dependency.
    s.table_lds = prefetch_table<NT>(s.table, n_pages, table_lds, p.table_cap);
    if (tid == 0) {
      int seen = __hip_atomic_load(&p.ws_count[titem], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      for (int spins = 0; seen < team && spins < p.spin_limit; ++spins) {
        __builtin_amdgcn_s_sleep(4);
        seen = __hip_atomic_load(&p.ws_count[titem], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      sh_last = seen >= team ? 1 : 0;
    }
    __syncthreads();
    KIN_STAMP(42);  // team complete (or patience over)
    if (__builtin_amdgcn_readfirstlane(sh_last)) {
      load_shared_keys<NT>(gkeys, n_score, s.keys);
    } else {
      score_rows<kDeep, NT, false, F16, false, HD>(s, 0, n_score, s.keys);
    }
    __builtin_amdgcn_s_waitcnt(0);  // the table copy has landed too
    __syncthreads();
    KIN_STAMP(43);  // keys in LDS
    n = select_from_keys<NT>(s, sel_lds);
  } else {
    s.table_lds = prefetch_table<NT>(s.table, n_pages, table_lds, p.table_cap);
    __syncthreads();  // histograms zeroed
    // Mean-key loads in flight per lane.  4 saturate HBM while several rounds of workgroups overlap
    // (4096 lists; more only lengthens the last pass of short lists).  With fewer lists the workgroups
    // score in step and each has to keep 64 KiB in flight: 16 / 8 loads at 4 / 8 waves
    // (1024 lists of 2048 pages: 5 % faster than with 4).
    if (p.deep_score) {
      constexpr int kDeep = NW <= 4 ? 16 : 8;
      n = score_select<kDeep, NT, F16, HD>(s, sel_lds);
    } else {
      n = score_select<4, NT, F16, HD>(s, sel_lds);
    }
  }
  KIN_STAMP(30);  // list ready
  if (p.sel_pages && part == 0) {
    int32_t* sel = p.sel_pages + (int64_t)item * p.sel_stride;
    for (int i = tid; i < p.sel_stride; i += NT) sel[i] = (i < n) ? sel_lds[i] : -1;
  }
  if (p.sel_count && tid == 0 && part == 0) p.sel_count[item] = n;
  int p0 = 0, p1 = n;
  if (team > 1) {
    const int per = (n + parts - 1) / parts;
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
  a.kvb = reinterpret_cast<const char*>(p.kv) + (int64_t)h * kRowB;
  a.row_bytes = p.num_kv_heads * kRowB;
  a.page_bytes = 2 * p.page_size * a.row_bytes;
  a.span = a.page_bytes - h * kRowB;
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
  attend_list<NG, NW, F16, HD>(
      a, [&](int i) -> int { return __builtin_amdgcn_readfirstlane(sel_lds[i]); }, smem, sm_m, sm_l,
      [&](int g, int d, float o, float lse2) {
        if (parts > 1) {
          // partial result, read by a workgroup that may sit on another XCD: device-scope stores
          const int64_t row = ((int64_t)(item - p.head_lists) * parts + part) * G + g;
          __hip_atomic_store(p.ws_po + row * HD + d, __float_as_uint(o), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (d == 0) __hip_atomic_store(p.ws_plse + row, __float_as_uint(lse2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          p.out[(hq0 + g) * HD + d] = (uint16_t)f32_to_elem<F16>(o);
          if (p.lse && d == 0) p.lse[hq0 + g] = lse2 * kLn2;
        }
      });
  KIN_STAMP(31);  // attended
  if (parts <= 1) return;
  // Every wave waits for its partial stores to be acknowledged, then the workgroup counts in;
  // whoever counts in last sees all parts and merges them (as merge_splits_kernel does).
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0)
    sh_last = (__hip_atomic_fetch_add(&p.ws_count2[item - p.head_lists], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == parts - 1) ? 1 : 0;
  __syncthreads();
  KIN_STAMP(44);  // partial stored, counted in
  if (!__builtin_amdgcn_readfirstlane(sh_last)) return;
  merge_list_parts<NT, F16, HD>(smem, p.ws_po, p.ws_plse, item - p.head_lists, parts, G, p.out + hq0 * HD, p.lse ? p.lse + hq0 : nullptr);
  KIN_STAMP(45);  // merged
}

}  // namespace kin

namespace kin {

// How the workgroups of a launch share the lists: the first head_lists lists have a workgroup
// each, every later list a team of `team` workgroups of which `parts` also attend (see
// StepParams).  nw: waves per workgroup.  need: workspace bytes.
struct StepPlan {
  int head_lists, team, parts, nw;
  size_t need;
};

constexpr int kMaxTeam = 64;
// Most lists beyond a multiple of the CUs that still get teams (see plan_step).
constexpr int kMaxTailLists = 96;

static size_t round256(size_t n) { return (n + 255) & ~(size_t)255; }

// Workspace of `team_lists` lists handled by teams: two arrival counters per list, the shared
// keys, the partial results.
static size_t team_workspace_bytes(int64_t team_lists, int parts, int group, int kbar_pages) {
  if (team_lists <= 0) return 0;
  size_t need = round256((size_t)team_lists * 2 * sizeof(int32_t));
  need += round256((size_t)team_lists * score_key_stride(kbar_pages) * sizeof(uint32_t));
  if (parts > 1) need += (size_t)team_lists * parts * group * (kHeadDim + 1) * sizeof(float);
  return need;
}

// list_tiles: upper bound of the 16-token tiles a page list holds.  avail: bytes the caller's
// workspace has (a smaller one gets smaller teams, or none, never an error).
//
// Teams are formed when the lists are at most a third of the CUs (or half of them, for page lists
// of 384 tiles or more): as many members as put one 8-wave workgroup on every CU, no more than
// give every scoring slice 64 KiB of mean keys or every attending member 16 tiles (below that the
// exchange and the merge cost more than they save), and of them as many attend as have 16 tiles
// each.  Measured on MI355X (ctx 32 K, k = 128, G = 4, us per step; one workgroup per list |
// teams | the earlier scheme, in which every part scored the whole list for itself): 8 lists
// 38 | 30 | 35; 32 lists 45 | 35 | 45; 64 lists 48 | 42 | 50; 128 lists 54 | 56 | 56.
// A batch of up to kMaxTailLists lists more than a multiple of the CUs keeps one workgroup per list for
// that multiple and forms teams of 2-4 for the rest (one workgroup per list | with tail teams, us per step:
// ctx 32 K, k = 128, G = 4: 264 lists 95 | 81; 304 lists 101 | 93; 352 lists 108 | 104; 384 lists 109 |
// 112 (not formed); G = 8, k = 256: 264 lists 171 | 137; 304 lists 175 | 149; 352 lists 180 | 165;
// ctx 16 K, k = 64: 264 lists 55.9 | 50.0; 352 lists 61.4 | 59.9; 8 KV heads of G = 2, k = 64: 264
// lists 71.5 | 60.6; 352 lists 78.3 | 75.4; the best team size falls from 4-8 at 8 extra lists to 2 at 96;
// ctx 32 K, k = 128, G = 4 again: 528 lists 154 | 141; 600: 166 | 164; 784: 228 | 210; 864: 241 | 237; 1040: 269 |
// 259; 1552: 400 | 378; 2080: 521 | 499; 4128: 1078 | 1050; G = 8, k = 256: 528 lists 279 | 242; 816: 401 | 354;
// 1040: 475 | 446; 1600: 703 | 664).  A batch that is a multiple of the CUs gains nothing from teams for its last
// lists (4096 lists: 961 | 962-988; 1024 lists of 8 heads: 430 | 435-471).
// Tried and not kept, because one workgroup per list is faster there: teams of two or three for
// every list of 129 .. 400 (160 lists 53 | 73; 256 lists 74 | 92; 300 lists 102 | 109: the streaming
// phases are bound by HBM either way, and the exchange, the second select and the merge add
// 9 us to every list's critical path, a fill launch in front 4 more), and teams for the lists
// of the second round of a batch a little larger than the GPU holds at once (1024 lists of
// 8 heads, k = 256: 428 | 452).
static StepPlan plan_step(int64_t items, int group, int kbar_pages, int64_t list_tiles, size_t avail) {
  StepPlan plan{(int)items, 1, 1, items <= kNumCus ? 8 : 4, 0};
  if (items <= 0) return plan;
  int64_t head = items, team = 1, parts = 1;
  const int64_t by_attend = list_tiles / 16;
  const int64_t by_score = kbar_pages / 256;
  // (short lists -- under 96 tiles to attend and under 1024 mean keys to score -- are quicker in one workgroup:
  // 8 .. 64 lists of 8 K tokens, k = 64: 25 .. 28 us against 26 .. 29)
  if ((items * 3 <= kNumCus && (list_tiles >= 96 || kbar_pages >= 1024)) || (items * 2 <= kNumCus && list_tiles >= 384)) {
    team = kNumCus / items;
    const int64_t useful = by_attend > by_score ? by_attend : by_score;
    if (team > useful) team = useful;
    if (team > kMaxTeam) team = kMaxTeam;
    parts = team < by_attend ? team : by_attend;
    head = 0;
  } else if (items > kNumCus && items % kNumCus != 0 && items % kNumCus <= kMaxTailLists &&
             (list_tiles >= 96 || kbar_pages >= 1024)) {
    // A few lists more than a multiple of the CUs: the GPU hands out workgroups in order, so the
    // last few would run on a few CUs (beside another list each, or alone at the end) while the
    // others wait for them.  Those lists get teams instead, small enough that every CU ends up
    // with about the same bytes.
    const int64_t tail = items % kNumCus;
    team = tail <= 32 ? 4 : (tail <= 72 ? 3 : 2);
    const int64_t useful = by_attend > by_score ? by_attend : by_score;
    if (team > useful) team = useful;
    parts = team < by_attend ? team : by_attend;
    head = items - tail;
  }
  if (parts < 1) parts = 1;
  if (team < 2) {
    team = parts = 1;
    head = items;
  }
#ifdef KIN_TUNE
  // experiments only: KIN_TEAM=head_lists,team,parts,nw
  int env_nw = 0;
  if (const char* e = getenv("KIN_TEAM")) {
    long long eh = 0;
    int et = 1, ep = 1;
    if (sscanf(e, "%lld,%d,%d,%d", &eh, &et, &ep, &env_nw) >= 3 && et >= 1 && ep >= 1 && ep <= et && eh >= 0 && eh <= items) {
      head = et > 1 && eh < items ? eh : items;
      team = head < items ? et : 1;
      parts = head < items ? ep : 1;
    }
  }
#endif
  // a workspace too small: fewer parts, then no teams
  while (team > 1 && team_workspace_bytes(items - head, (int)parts, group, kbar_pages) > avail) {
    if (parts > 1) {
      parts /= 2;
    } else {
      team = 1;
      head = items;
    }
  }
  plan.head_lists = (int)head;
  plan.team = (int)team;
  plan.parts = (int)parts;
  const int64_t wgs = head + (items - head) * team;
  plan.nw = wgs <= kNumCus ? 8 : 4;
#ifdef KIN_TUNE
  if (env_nw == 4 || env_nw == 8) plan.nw = env_nw;
#endif
  plan.need = team > 1 ? team_workspace_bytes(items - head, plan.parts, group, kbar_pages) : 0;
  return plan;
}

}  // namespace kin

extern "C" size_t kin_step_workspace_bytes(int batch, int num_kv_heads, int kbar_pages) {
  // Enough for whichever teams the launch forms, whatever the group size and page budget.
  const int64_t items = (int64_t)batch * num_kv_heads;
  if (items <= 0) return 0;
  size_t need = kin::plan_step(items, kin::kMaxGroup, kbar_pages, kin::kMaxTopk + 2 * kin::kMaxFixedPages, ~(size_t)0).need;
#ifdef KIN_TUNE
  if (need < ((size_t)192 << 20)) need = (size_t)192 << 20;
#endif
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
                       void* workspace, size_t workspace_bytes, const int32_t* slot_ids, int num_slots, int32_t* slot_lens,
                       kin_stream_t stream) {
  if (!q || !kv_cache || !kbar || !page_indices || !page_indptr || !last_page_len || !out)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if ((k == nullptr) != (v == nullptr))
    return fail(KIN_ERR_NULL_POINTER, "%s: k and v must both be given or both be null", fn);
  int st = check_common_dims(fn, batch, num_q_heads, num_kv_heads, head_dim, page_size, true);
  if (st) return st;
  if (num_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_pages=%lld must be >= 1", fn, (long long)num_pages);
  if (topk < 0) return fail(KIN_ERR_BAD_SHAPE, "%s: topk=%d is negative", fn, topk);
  if (kbar_pages < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: kbar_pages=%d must be >= 1", fn, kbar_pages);
  if (slot_ids && num_slots < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_slots=%d must be >= 1 when slot_ids is given", fn, num_slots);
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
  p.slot_ids = slot_ids;
  p.num_slots = slot_ids ? num_slots : batch;
  p.slot_lens = slot_lens;
  p.sort_cap = select_sort_cap(topk, kbar_pages);
  p.table_cap = select_table_cap(kbar_pages + max_local_pages(local_tokens) + 1);
  const int64_t items = (int64_t)batch * num_kv_heads;
  if (xcd_grid_size(batch, num_kv_heads) > 0x7fffffffLL || items * kMaxTeam > 0x7fffffffLL)
    return fail(KIN_ERR_UNSUPPORTED, "%s: batch*num_kv_heads too large", fn);
  p.num_pages = num_pages;
  const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim);
  p.scale_log2 = scale * 1.4426950408889634f;
  p.deep_score = items < 4096 ? 1 : 0;
  p.rotate = attend_rotates(items) ? 1 : 0;
  // Lists that would leave CUs idle get teams of workgroups (given a workspace).
  const StepPlan plan = plan_step(items, p.group, kbar_pages, (int64_t)list_cap << page_tile_shift(page_size),
                                  workspace && aligned16(workspace) ? workspace_bytes : 0);
  // Waves per workgroup.  The kernels hold 140-145 registers, so a CU runs 12 waves: three
  // 4-wave workgroups, or one of 8 while the workgroups are no more than the CUs (measured: 8 waves
  // beat 4, 6, 12 and a 16-wave build that spills, by 2-20 %; from 257 workgroups on, 8-wave
  // workgroups would take two rounds and 4 waves win by 3-25 %).
  const int nw = plan.nw;
  p.head_lists = plan.head_lists;
  p.team = plan.team;
  p.parts = plan.parts;
  p.head_blocks = plan.head_lists == items ? (int)xcd_grid_size(batch, num_kv_heads) : plan.head_lists;
  p.spin_limit = team_spin_limit();
  p.ws_count = p.ws_count2 = nullptr;
  p.ws_keys = nullptr;
  p.ws_po = nullptr;
  p.ws_plse = nullptr;
  const int64_t team_lists = items - plan.head_lists;
  if (plan.team > 1) {
    char* w = static_cast<char*>(workspace);
    p.ws_count = reinterpret_cast<int32_t*>(w);
    p.ws_count2 = p.ws_count + team_lists;
    w += round256((size_t)team_lists * 2 * sizeof(int32_t));
    p.ws_keys = reinterpret_cast<uint32_t*>(w);
    w += round256((size_t)team_lists * score_key_stride(kbar_pages) * sizeof(uint32_t));
    p.ws_po = reinterpret_cast<uint32_t*>(w);
    p.ws_plse = p.ws_po + (size_t)team_lists * plan.parts * p.group * head_dim;
  }
  const size_t sel_scratch = select_lds_bytes(kbar_pages, p.sort_cap, p.table_cap);
  const size_t attend_bytes = (size_t)attend_lds_bytes(nw);
  size_t region0 = sel_scratch > attend_bytes ? sel_scratch : attend_bytes;
  region0 = (region0 + 15) & ~(size_t)15;
  p.region0_bytes = (int)region0;
  const size_t lds = region0 + (size_t)list_cap * 4;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const void* kernel;
#define KIN_STEP_KERNEL(NG_, NW_)                                                                              \
  (head_dim == kHeadDimSmall                                                                                   \
       ? (f16 ? reinterpret_cast<const void*>(&blocktopk_step_kernel<NG_, NW_, true, kHeadDimSmall>)           \
              : reinterpret_cast<const void*>(&blocktopk_step_kernel<NG_, NW_, false, kHeadDimSmall>))         \
       : (f16 ? reinterpret_cast<const void*>(&blocktopk_step_kernel<NG_, NW_, true, kHeadDim>)                \
              : reinterpret_cast<const void*>(&blocktopk_step_kernel<NG_, NW_, false, kHeadDim>)))
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
  const unsigned grid = (unsigned)(p.head_blocks + team_lists * plan.team);
  if (plan.team > 1) {
    // the arrival counters start at zero (a fill kernel, so that the launch pair can be captured in a graph)
    fill_zero_i32_kernel<<<(unsigned)((2 * team_lists + 255) / 256), 256, 0, s>>>(p.ws_count, (int)(2 * team_lists));
    st = check_hip(hipGetLastError(), "fill_zero_i32_kernel launch");
    if (st) return st;
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
                                         size_t workspace_bytes, const int32_t* slot_ids, int num_slots,
                                         int32_t* slot_lens, kin_stream_t stream) {
  return kin::launch_step("kin_blocktopk_decode_step", false, q, k, v, kv_cache, kbar, page_indices, page_indptr,
                          last_page_len, topk, sink_pages, local_tokens, sel_pages, sel_count, out, lse, batch, num_q_heads,
                          num_kv_heads, head_dim, page_size, num_pages, kbar_pages, sel_stride, first_page_offset, sm_scale,
                          workspace, workspace_bytes, slot_ids, num_slots, slot_lens, stream);
}

extern "C" int kin_blocktopk_decode_step_f16(const kin_f16_t* q, const kin_f16_t* k, const kin_f16_t* v,
                                             kin_f16_t* kv_cache, kin_f16_t* kbar, const int32_t* page_indices,
                                             const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                                             int sink_pages, int local_tokens, int32_t* sel_pages, int32_t* sel_count,
                                             kin_f16_t* out, float* lse, int batch, int num_q_heads, int num_kv_heads,
                                             int head_dim, int page_size, int64_t num_pages, int kbar_pages,
                                             int sel_stride, int first_page_offset, float sm_scale, void* workspace,
                                             size_t workspace_bytes, const int32_t* slot_ids, int num_slots,
                                             int32_t* slot_lens, kin_stream_t stream) {
  return kin::launch_step("kin_blocktopk_decode_step_f16", true, q, k, v, kv_cache, kbar, page_indices, page_indptr,
                          last_page_len, topk, sink_pages, local_tokens, sel_pages, sel_count, out, lse, batch, num_q_heads,
                          num_kv_heads, head_dim, page_size, num_pages, kbar_pages, sel_stride, first_page_offset, sm_scale,
                          workspace, workspace_bytes, slot_ids, num_slots, slot_lens, stream);
}

#ifdef KIN_TUNE
KIN_STAMP_ACCESSOR(kin_debug_stamps_step)
#endif

extern "C" size_t kin_static_scratch_bytes(void) { return kin::kStaticScratchBytes; }

extern "C" int kin_blocktopk_decode_step_static(const kin_bf16_t* q, const kin_bf16_t* k, const kin_bf16_t* v,
                                                kin_bf16_t* kv_cache, kin_bf16_t* kbar, const int32_t* page_indices,
                                                const int32_t* page_indptr, const int32_t* last_page_len, int topk,
                                                int sink_pages, int local_tokens, int32_t* sel_pages,
                                                int32_t* sel_count, kin_bf16_t* out, float* lse, int batch,
                                                int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                                int64_t num_pages, int kbar_pages, int sel_stride,
                                                int first_page_offset, float sm_scale, const int32_t* slot_ids,
                                                int num_slots, int32_t* slot_lens, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_blocktopk_decode_step_static";
  // What the teams of this shape need, from the dimensions alone.  With few lists (up to one for
  // every other CU) the teams are what keeps the GPU busy at all: if theirs do not fit the array
  // (long sequences: 4 bytes per candidate page and list), that is an error, not a silent
  // fall-back to one workgroup per list.  Larger batches take the teams that fit, or none.
  size_t need = 0;
  if (batch > 0 && num_kv_heads > 0 && num_q_heads >= num_kv_heads && kbar_pages > 0 && topk >= 0 && sink_pages >= 0 &&
      local_tokens >= 1 && page_size >= kPageSize) {
    const int64_t list_cap = (int64_t)topk + sink_pages + max_local_pages(local_tokens);
    const int64_t lists = (int64_t)batch * num_kv_heads;
    need = plan_step(lists, num_q_heads / num_kv_heads, kbar_pages, list_cap << page_tile_shift(page_size), ~(size_t)0).need;
    if (lists * 2 > kNumCus && need > kStaticScratchBytes)
      need = plan_step(lists, num_q_heads / num_kv_heads, kbar_pages, list_cap << page_tile_shift(page_size), kStaticScratchBytes).need;
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
                     kbar_pages, sel_stride, first_page_offset, sm_scale, ws, ws ? kStaticScratchBytes : 0, slot_ids, num_slots,
                     slot_lens, stream);
}
