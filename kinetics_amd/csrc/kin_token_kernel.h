// The token-granular decode kernel (token-level top-k and strided overlapping blocks) and the table
// of its instantiations for one head dimension.  Included by one translation unit per head dimension,
// so that the two sets of kernels compile side by side.
#pragma once

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
  uint32_t* ws_po;      // workspace, parts > 1: [lists, parts, G, HD] normalised partial outputs (fp32 bits)
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
template <int NG, int NW, bool STRIDED, bool LDSK, bool F16, int HD>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void token_topk_kernel(TokenTopkParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float sm_m[NW][4 * NG];
  __shared__ float sm_l[NW][4 * NG];
  __shared__ KeySelectShared sh;
  __shared__ int sh_last;
  constexpr int NT = NW * 64;
  constexpr int kRowB = HD * 2;  // bytes of one head's row

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
    for (int i = tid; i < G * HD; i += NT) p.out[hq0 * HD + i] = 0;
    if (p.lse && tid < G) p.lse[hq0 + tid] = kNegInf;
    return;
  }

  int32_t* list = reinterpret_cast<int32_t*>(smem + p.region0_bytes);
  TokenArgs t;
  t.q_bh = p.q + hq0 * HD;
  t.kvb = reinterpret_cast<const char*>(p.kv) + (int64_t)h * kRowB;
  t.row_bytes = p.num_kv_heads * kRowB;
  t.page_bytes = 2 * kPageSize * t.row_bytes;
  t.span = t.page_bytes - h * kRowB;
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
    if (STRIDED) strided_score_tokens<NW, LDSK, F16, HD>(t, sa, pg0, pg1);
    else token_score_keys<NW, LDSK, F16, HD>(t, pg0, pg1, first_digit_counted ? sh.hist[0] : nullptr);
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
            token_score_keys<NW, LDSK, F16, HD>(t, 0, n_pages, sh.hist[0]);
          } else {
            strided_score_tokens<NW, LDSK, F16, HD>(t, sa, 0, n_pages);
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
  attend_tokens<NG, NW, F16, HD>(a, list + e0, smem, sm_m, sm_l, [&](int g, int d, float o, float lse2) {
    if (team) {
      // partial result, read by a workgroup that may sit on another XCD: device-scope stores
      const int64_t row = ((int64_t)item * p.parts + chunk) * G + g;
      __hip_atomic_store(p.ws_po + row * HD + d, __float_as_uint(o), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (d == 0) __hip_atomic_store(p.ws_plse + row, __float_as_uint(lse2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      p.out[(hq0 + g) * HD + d] = (uint16_t)f32_to_elem<F16>(o);
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
  merge_list_parts<NT, F16, HD>(smem, p.ws_po, p.ws_plse, item, p.parts, G, p.out + hq0 * HD, p.lse ? p.lse + hq0 : nullptr);
  KIN_STAMP(45);  // parts merged
}

}  // namespace kin

namespace kin {

// The kernel for one launch configuration: group <= 4 takes the narrow form, nw is 4, 8 or 12 waves
// (an LDSK kernel has 4 or 12).
template <int HD>
const void* token_kernel_for(bool f16, bool strided, int group, int nw, bool ldsk) {
#define KIN_TOKEN_KERNEL(NG_, NW_, S_, L_)                                                      \
  (f16 ? reinterpret_cast<const void*>(&token_topk_kernel<NG_, NW_, S_, L_, true, HD>)          \
       : reinterpret_cast<const void*>(&token_topk_kernel<NG_, NW_, S_, L_, false, HD>))
#define KIN_TOKEN_PICK(NG_, S_)                                                                 \
  (ldsk ? (nw == 12 ? KIN_TOKEN_KERNEL(NG_, 12, S_, true) : KIN_TOKEN_KERNEL(NG_, 4, S_, true)) \
        : (nw == 12 ? KIN_TOKEN_KERNEL(NG_, 12, S_, false) : nw == 8 ? KIN_TOKEN_KERNEL(NG_, 8, S_, false) : KIN_TOKEN_KERNEL(NG_, 4, S_, false)))
  if (strided) return group <= 4 ? KIN_TOKEN_PICK(1, true) : KIN_TOKEN_PICK(4, true);
  return group <= 4 ? KIN_TOKEN_PICK(1, false) : KIN_TOKEN_PICK(4, false);
#undef KIN_TOKEN_PICK
#undef KIN_TOKEN_KERNEL
}

// token_kernel_for<kHeadDimSmall>, compiled in its own translation unit.
const void* token_kernel_small_head(bool f16, bool strided, int group, int nw, bool ldsk);

}  // namespace kin
