// Device-side building blocks of token-level top-k sparse decode attention for
// one (sequence, KV head), run by workgroups of NW waves:
//
//   token_score_keys()    streams the K half of a run of the sequence's pages once
//       (16-byte loads straight to registers; the mean over the group's heads of
//       q_g . k_t is (mean_g q_g) . k_t, one fp32 dot product per token) and
//       turns the score of every token of the "dynamic" part (after the sink
//       tokens, before the local window) into an order-preserving 32-bit key in
//       a key array: in LDS when the sequence's keys fit there beside the token
//       list (LDSK = true; up to ~34 K tokens), else in an HBM scratch array;
//   token_select_list()   radix-selects the k-th largest key and compacts the
//       winners, in ascending token order, into a token list in LDS: sink
//       tokens, winners, local-window tokens;
//   strided_score_tokens() / strided_select_list()   the same two steps for the
//       strided overlapping-block policy (fp32 scores, block means, a bitmap);
//   attend_tokens()       attention over such a list: the page loop of
//       attend_list() with one address per token row instead of one per page.
//
// HBM-bound on the key stream: 256 B per context token, plus 512 B per listed
// token.  Keys in HBM (4 B per token, written and read back at device scope so
// that several workgroups can share the scoring of one sequence) add 5 % of traffic
// and, interleaved with a saturated read stream, up to 14 % of time; keys in LDS
// cost neither.
#pragma once

#include "kin_attend.h"
#include "kin_select.h"

namespace kin {

constexpr int kMaxTopkTokens = 4096;
constexpr int kMaxSinkTokens = 64;
constexpr int kMaxWindowTokens = 1024;

// Wave-uniform description of one token selection problem.
struct TokenArgs {
  const uint16_t* q_bh;  // the group's G query rows
  const char* kvb;       // kv_cache base + h * 256 bytes
  int row_bytes;         // bytes between token rows of a page
  int page_bytes;
  int span;              // bytes addressable from kvb within one page
  int64_t num_pages;
  int G;
  const int32_t* table;  // the sequence's page table (logical -> physical)
  int n_pages;
  int pad;               // unused slots in front of token 0 (first_page_offset)
  int n_sink, n_dyn, n_local;  // tokens: always attended / candidates / always attended
  int topk;
  uint32_t* keys;        // HBM scratch, n_pages * 16 entries, 16-byte aligned
  uint32_t* lds_keys;    // LDSK kernels: the same array in LDS, n_pages * 16 + 4 entries (the last 4: a dump slot)
  int32_t* list;         // LDS, >= n_sink + min(topk, n_dyn) + n_local entries
  int32_t* sel_tokens;   // HBM, the listed tokens' positions in the sequence, or null
  unsigned rotate;       // where in its page range this list starts streaming (any value)
};

// Physical token id (page * 16 + slot) of cache slot c of the sequence.
__device__ __forceinline__ int phys_token(const int32_t* table, int c) {
  return table[c >> 4] * kPageSize + (c & (kPageSize - 1));
}

// list[first .. first + count) holds cache slots (LDS); replaces each by its
// physical token id and reports the tokens' positions.  One independent table
// lookup per thread and entry, all in flight together -- inside the ordered
// compaction the same lookups would be a chain of dependent memory round trips.
// Barriers before and after are the caller's.
template <int NT>
__device__ __forceinline__ void translate_slots(int32_t* list, int first, int count, const int32_t* table, int pad,
                                                int32_t* sel_tokens) {
  for (int i = threadIdx.x; i < count; i += NT) {
    const int c = list[first + i];
    list[first + i] = phys_token(table, c);
    if (sel_tokens) sel_tokens[first + i] = c - pad;
  }
}

// LDS scratch of the two functions below.
struct KeySelectShared {
  uint32_t hist[4][256];  // one histogram per radix digit (see radix_select_emit)
  uint32_t wave_gt[16], wave_eq[16];
};

// Keys one trip to memory brings into registers: kSelLoads 16-byte loads per lane.
// Under a saturated key stream every dependent round trip costs microseconds, so
// the select passes below make few, wide trips instead of many narrow ones.
constexpr int kSelLoads = 16;

// Chunk c0 of the key array -> registers: wave w holds the 1024 * kSelLoads / 4
// consecutive keys from c0 + w * 256 * kSelLoads, load u the keys 256 * u + 4 * lane
// + 0..3 of them (so wave, u, lane, j ascending is index ascending).  keys (GlobalKeys
// or LdsKeys below) covers exactly the n_keys (a multiple of 4) keys: entries past
// them read as 0, "not a candidate".
template <int NW, typename Keys>
__device__ __forceinline__ void load_key_chunk(const Keys& keys, int c0, u32x4 (&kk)[kSelLoads]) {
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), l = threadIdx.x & 63;
  const int base = c0 + w * (256 * kSelLoads) + 4 * l;
#pragma unroll
  for (int u = 0; u < kSelLoads; ++u) kk[u] = keys(base + u * 256);
}

// Where the select reads its keys: four consecutive keys from index i (a multiple
// of 4), zeros past the end.
struct GlobalKeys {  // device-scope loads through a descriptor over exactly the keys
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ __forceinline__ u32x4 operator()(int i) const {
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, i * 4, 0, kDeviceScope);
  }
};
struct LdsKeys {  // 16-byte aligned LDS array of n (a multiple of 4) keys
  const uint32_t* keys;
  int n;
  __device__ __forceinline__ u32x4 operator()(int i) const {
    return i < n ? *reinterpret_cast<const u32x4*>(keys + i) : u32x4{0u, 0u, 0u, 0u};
  }
};

// Most-significant-digit-first radix select over n_keys (a multiple of 16) 32-bit
// keys in global memory (GlobalKeys: a descriptor over exactly those keys, written at
// device scope) or in LDS (LdsKeys), run by a workgroup of NW waves, followed by the ordered
// compaction of the winners: finds the k-th largest non-zero key (zero keys are
// "not a candidate"; at least k >= 1 keys are non-zero), then calls emit(pos, index)
// for every key above it and for the lowest-indexed keys equal to it that complete
// the k, pos = 0, 1, ... in ascending index order.
// first_digit_counted: sh->hist[0] already holds the histogram of the top byte of
// the non-zero keys (counted while they were produced).  The writes of the keys
// have completed (s_waitcnt + barrier, or the arrival counter of split scoring).
// Up to NW * 4096 keys are loaded once and stay in registers through all passes;
// longer arrays are walked in chunks of that size, one trip per chunk and pass.
template <int NW, typename Keys, typename Emit>
__device__ __forceinline__ void radix_select_emit(const Keys& keys, int n_keys, uint32_t k,
                                                  bool first_digit_counted, KeySelectShared* sh, Emit emit) {
  constexpr int kChunk = NW * 256 * kSelLoads;
  constexpr int NT = NW * 64;
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63;
  const bool single = n_keys <= kChunk;
  u32x4 kk[kSelLoads];
  if (single) load_key_chunk<NW>(keys, 0, kk);
  KIN_STAMP(54);  // keys requested
  // Loads of this wave that hold keys at all (the others read zeros past the end and are skipped:
  // the passes below are bound by vector instructions, 64 keys per lane).
  auto loads_with_keys = [&](int c0) -> int {
    const int left = n_keys - (c0 + w * (256 * kSelLoads));
    return left <= 0 ? 0 : (left >= 256 * kSelLoads ? kSelLoads : (left + 255) >> 8);
  };
  // The histograms of the digits still to be counted start at zero (one per digit: no wave
  // clears what another still reads, so a digit costs one barrier).
  for (int i = tid + (first_digit_counted ? 256 : 0); i < 4 * 256; i += NT) (&sh->hist[0][0])[i] = 0;
  __syncthreads();

  uint32_t prefix = 0, mask = 0, remaining = k;
  bool whole_bin = false;  // every key that matches the digits fixed so far is wanted: no further digit needed
  for (int pass = 0; pass < 4 && !whole_bin; ++pass) {
    const int shift = 24 - 8 * pass;
    if (pass != 0 || !first_digit_counted) {
      uint32_t* hist = sh->hist[pass];
      for (int c0 = 0; c0 < n_keys; c0 += kChunk) {
        if (!single) load_key_chunk<NW>(keys, c0, kk);
        const int nu = loads_with_keys(c0);
#pragma unroll
        for (int u = 0; u < kSelLoads; ++u) {
          if (u < nu) {
            const uint32_t k4[4] = {kk[u].x, kk[u].y, kk[u].z, kk[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (k4[j] && (k4[j] & mask) == prefix) atomicAdd(&hist[(k4[j] >> shift) & 255u], 1u);
          }
          __builtin_amdgcn_sched_barrier(0);  // keeps the lane masks of one load at a time in scalar registers
        }
      }
      __syncthreads();
    }
    uint32_t bin;
    radix_pick_bin_uniform(sh->hist[pass], remaining, l, bin, remaining, whole_bin);  // every wave for itself: no hand-over
    prefix |= bin << shift;
    mask |= 255u << shift;
    KIN_STAMP(55 + pass);  // digit fixed
  }
  uint32_t thr = prefix;  // the k-th largest key (>= 1) ...
  if (whole_bin && mask != 0xffffffffu) {
    // ... or, after an early exit, the largest value below every winner: all keys that start with
    // `prefix` are taken, none is ranked among its equals.
    thr = prefix ? prefix - 1u : 0u;
    remaining = 0;
  }

  // Ordered compaction, chunk by chunk: count per wave, prefix over the waves, emit.
  uint32_t run_all = 0, eq_all = 0;  // winners / threshold-equal keys in the chunks before this one
  for (int c0 = 0; c0 < n_keys; c0 += kChunk) {
    if (!single) load_key_chunk<NW>(keys, c0, kk);
    const int nu = loads_with_keys(c0);
    uint32_t gt = 0, eq = 0;
#pragma unroll
    for (int u = 0; u < kSelLoads; ++u) {
      if (u < nu) {
        const uint32_t k4[4] = {kk[u].x, kk[u].y, kk[u].z, kk[u].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          gt += (k4[j] > thr) ? 1u : 0u;
          eq += (k4[j] == thr) ? 1u : 0u;
        }
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      gt += __shfl_xor(gt, off);
      eq += __shfl_xor(eq, off);
    }
    if (l == 0) {
      sh->wave_gt[w] = gt;
      sh->wave_eq[w] = eq;
    }
    __syncthreads();
    uint32_t run = run_all, eq_run = eq_all;  // ... at lower indices than this wave's keys
    {
      uint32_t r = run_all, e_acc = eq_all;
      for (int wv = 0; wv < NW; ++wv) {
        if (wv == w) {
          run = r;
          eq_run = e_acc;
        }
        const uint32_t e = sh->wave_eq[wv];
        const uint32_t left = remaining > e_acc ? remaining - e_acc : 0u;
        r += sh->wave_gt[wv] + min(e, left);
        e_acc += e;
      }
      run_all = r;
      eq_all = e_acc;
    }
    const int wave_base = c0 + w * (256 * kSelLoads) + 4 * l;
    const bool rank_equals = remaining > 0 && eq > 0;  // wave-uniform: some key of this wave's equals the threshold
#pragma unroll
    for (int u = 0; u < kSelLoads; ++u) {
      if (u < nu) {  // wave-uniform: the loads behind hold no keys
        const int i0 = wave_base + u * 256;  // this lane's 4 consecutive indices
        const uint32_t k4[4] = {kk[u].x, kk[u].y, kk[u].z, kk[u].w};
        // Lanes hold ascending indices, so positions come from prefix sums over the wave (DPP
        // scans).  Keys equal to the threshold are rare: they are ranked only where there are any.
        uint32_t eq_before = eq_run, eq_total = 0;
        if (rank_equals) {
          const uint32_t eq_mine = (k4[0] == thr ? 1u : 0u) + (k4[1] == thr ? 1u : 0u) + (k4[2] == thr ? 1u : 0u) +
                                   (k4[3] == thr ? 1u : 0u);
          const uint32_t incl = wave_inclusive_sum(eq_mine);
          eq_before += incl - eq_mine;
          eq_total = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        }
        bool take[4];
        uint32_t seen = 0, cnt = 0;
  #pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool is_eq = k4[j] == thr;
          take[j] = k4[j] > thr || (is_eq && eq_before + seen < remaining);
          seen += is_eq ? 1u : 0u;
          cnt += take[j] ? 1u : 0u;
        }
        const uint32_t incl = wave_inclusive_sum(cnt);
        uint32_t pos = run + incl - cnt;  // winners at lower indices
  #pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (take[j]) {
            emit((int)pos, i0 + j);
            ++pos;
          }
        }
        run += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        eq_run += eq_total;
      }
      __builtin_amdgcn_sched_barrier(0);  // one load's scan at a time: interleaving them only costs registers
    }
    __syncthreads();  // wave_gt / wave_eq are rewritten by the next chunk
  }
  KIN_STAMP(59);  // winners listed
}

// Streams the K plane of the pages pg0 <= p < pg1 (pg0 a multiple of 4) of the
// sequence once and calls emit(c, score, valid) from every lane; the calls with
// valid == true, one per key row, carry score = (mean_g q_g) . k_c in fp32 for every cache slot c of
// those pages (slots past the last token included).  emit must not branch around
// vector memory operations (store through a descriptor, out of range when !valid).  16-byte loads straight to registers, 16 of them in flight per
// lane; no LDS, no barrier.
template <int NW, bool F16 = false, int HD = kHeadDim, typename Emit>
__device__ __forceinline__ void stream_token_scores(const TokenArgs& a, int pg0, int pg1, Emit emit) {
  constexpr int LPR = HD / 8;          // lanes that share a key row (16-byte chunks of it): 16 or 8
  constexpr int RPI = 64 / LPR;        // key rows one load instruction of a wave covers: 4 or 8
  constexpr int LPP = kPageSize / RPI; // loads per page (a K plane of 16 rows): 4 or 2
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, rg = l / LPR, cc = l & (LPR - 1);
  const int G = a.G;
  const int32_t* table = a.table;
  // The mean over the group's heads of q_g . k_t is (mean_g q_g) . k_t: one dot
  // product per token.  Lane owns columns d = 8*cc .. +7 of the mean query;
  // LPR lanes share a key row, one load instruction of a wave covers RPI rows.
  float qm[8];
  {
#pragma unroll
    for (int u = 0; u < 8; ++u) qm[u] = 0.f;
    const uint16_t* qp = a.q_bh + 8 * cc;
    for (int g = 0; g < G; ++g) {
      const uint4 x = *reinterpret_cast<const uint4*>(qp + (int64_t)g * HD);
      qm[0] += elem_lo<F16>(x.x); qm[1] += elem_hi<F16>(x.x);
      qm[2] += elem_lo<F16>(x.y); qm[3] += elem_hi<F16>(x.y);
      qm[4] += elem_lo<F16>(x.z); qm[5] += elem_hi<F16>(x.z);
      qm[6] += elem_lo<F16>(x.w); qm[7] += elem_hi<F16>(x.w);
    }
    const float inv = 1.0f / (float)G;
#pragma unroll
    for (int u = 0; u < 8; ++u) qm[u] *= inv;
  }
  // A wave streams whole K planes (16 rows, contiguous for one KV head; LPP 16-byte loads per lane:
  // load i covers key rows RPI*i .. RPI*i + RPI-1), four consecutive pages at a time: the
  // quads pg0/4 + w, + NW, ... of the page range, the next quad in flight.  After
  // a quad every lane holds one score -- lane l that of the row l / LPR of the quad's load l % LPR
  // (load j = LPP * page + i) -- so one emit per quad covers 64 consecutive cache
  // slots (256 B of keys: full lines, a quarter of the stores).
  constexpr int kPF = 4;
  const __attribute__((address_space(4))) int32_t* tab_c =
      reinterpret_cast<const __attribute__((address_space(4))) int32_t*>(reinterpret_cast<uintptr_t>(table));
  const int voff = rg * a.row_bytes + cc * 16;
  const int row_step = RPI * a.row_bytes;
  const int k_span = kPageSize * a.row_bytes - (a.span < a.page_bytes ? a.page_bytes - a.span : 0);  // K plane only
  auto load_page = [&](int p, u32x4 (&dst)[LPP]) {
    // Pages past the end (or with an id outside the cache) are read through an
    // empty descriptor: zeros, no memory traffic.
    const bool in = p < pg1;
    const int id = tab_c[in ? p : 0];
    const bool ok = in && id >= 0 && (int64_t)id < a.num_pages;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(a.kvb + (int64_t)(ok ? id : 0) * a.page_bytes, ok ? k_span : 0);
#pragma unroll
    for (int i = 0; i < LPP; ++i) dst[i] = __builtin_amdgcn_raw_buffer_load_b128(r, voff + i * row_step, 0, kStreamLoad);
  };
  const int my_load = cc;                                   // the quad's load whose row this lane reports
  const int my_page = my_load / LPP, my_row = RPI * (my_load % LPP) + rg;
  // The wave's quads are qi = w, w + NW, ... of the range's nq quads, visited from a
  // list-specific starting quad (a.rotate) and wrapping around: scores are stored by
  // position, so the order is free, and equal lists that run in step then read from
  // all over the cache instead of from one narrow window of it (reading only the K
  // half of consecutive pages loads the memory channels unevenly).
  const int nq = (pg1 - pg0 + kPF - 1) / kPF;  // pg0 is a multiple of 4
  const int rot = nq > 0 ? (int)(a.rotate % (unsigned)nq) : 0;
  auto quad_page = [&](int qi) -> int {  // first page of quad qi, or pg1 (nothing to read) past the end
    if (qi >= nq) return pg1;
    const int qq = qi + rot;
    return pg0 + kPF * (qq >= nq ? qq - nq : qq);
  };
  u32x4 x[kPF][LPP];
  {
    const int p0 = quad_page(w);
#pragma unroll
    for (int u = 0; u < kPF; ++u) {
      load_page(p0 + u, x[u]);
      // Issue order = consumption order: the wait at the top of the loop is sized for the worse
      // of the two ways into it, and a reordered prologue would leave only a few loads in flight.
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  for (int qi = w; qi < nq; qi += NW) {
    const int base = quad_page(qi), next = quad_page(qi + NW);
    float mine = 0.f;
#pragma unroll
    for (int u = 0; u < kPF; ++u) {
      u32x4 kx[LPP];
#pragma unroll
      for (int i = 0; i < LPP; ++i) kx[i] = x[u][i];
      load_page(next + u, x[u]);
      float acc[LPP];
#pragma unroll
      for (int i = 0; i < LPP; ++i) {
        float s = 0.f;
        s = fmaf(qm[0], elem_lo<F16>(kx[i].x), s); s = fmaf(qm[1], elem_hi<F16>(kx[i].x), s);
        s = fmaf(qm[2], elem_lo<F16>(kx[i].y), s); s = fmaf(qm[3], elem_hi<F16>(kx[i].y), s);
        s = fmaf(qm[4], elem_lo<F16>(kx[i].z), s); s = fmaf(qm[5], elem_hi<F16>(kx[i].z), s);
        s = fmaf(qm[6], elem_lo<F16>(kx[i].w), s); s = fmaf(qm[7], elem_hi<F16>(kx[i].w), s);
        acc[i] = row_sum<LPR>(s);
      }
      const int i_mine = my_load % LPP;
      float pick = acc[0];
#pragma unroll
      for (int i = 1; i < LPP; ++i) pick = i_mine == i ? acc[i] : pick;
      if (my_page == u) mine = pick;
    }
    // Called by every lane, without a branch: conditionally executed memory operations in
    // this loop would keep the compiler from counting how many loads may stay in flight.
    const int p = base + my_page;
    emit(p * kPageSize + my_row, mine, p < pg1);
  }
}

// Token-level top-k in three steps, so that the scoring of one sequence can be
// shared by several workgroups: token_needs_scores() (false: the budget covers
// every candidate, or is zero), token_score_keys() over a page range, and
// token_select_list().

__device__ __forceinline__ bool token_needs_scores(const TokenArgs& a) {
  const int k_eff = min(a.topk, a.n_dyn);
  return k_eff > 0 && k_eff < a.n_dyn;
}

// Scores the tokens of the pages pg0 <= p < pg1 into a.keys (device-scope stores) or,
// LDSK, into a.lds_keys; 0 marks "not a candidate", order_key is never 0 for a finite
// score.  hist: 256 zeroed LDS counters that receive the histogram of the keys' top
// byte, or null.  No barrier inside; the stores are complete after s_waitcnt(0).
template <int NW, bool LDSK = false, bool F16 = false, int HD = kHeadDim>
__device__ __forceinline__ void token_score_keys(const TokenArgs& a, int pg0, int pg1, uint32_t* hist) {
  const int dyn_lo = a.pad + a.n_sink, dyn_hi = dyn_lo + a.n_dyn;  // cache slots of the candidates
  const __amdgpu_buffer_rsrc_t keys_rsrc = make_rsrc(a.keys, LDSK ? 0 : a.n_pages * kPageSize * 4);
  uint32_t* lds_keys = a.lds_keys;
  const int dump = a.n_pages * kPageSize;  // lanes without a row write here
  stream_token_scores<NW, F16, HD>(a, pg0, pg1, [&](int c, float score, bool valid) {
    const uint32_t key = (c >= dyn_lo && c < dyn_hi) ? order_key(score) : 0u;
    if constexpr (LDSK)
      lds_keys[valid ? c : dump] = key;
    else  // lanes without a row store at an offset outside the descriptor: dropped by the hardware
      __builtin_amdgcn_raw_buffer_store_b32(key, keys_rsrc, valid ? c * 4 : -1, 0, kDeviceScope);
    if (hist && valid && key) atomicAdd(&hist[key >> 24], 1u);
  });
}

// Writes the token list (physical token ids) to a.list: sink tokens, the k
// candidates with the largest keys in ascending position, local tokens; returns
// its length.  When token_needs_scores(), a.keys is complete and, if
// first_digit_counted, sh->hist[0] holds the histogram of the keys' top byte.  Every
// thread of the workgroup calls this; it ends with a workgroup barrier.
template <int NG, int NW, bool LDSK = false>
__device__ __forceinline__ int token_select_list(const TokenArgs& a, KeySelectShared* sh, bool first_digit_counted) {
  constexpr int NT = NW * 64;
  const int tid = threadIdx.x;
  const int k_eff = min(a.topk, a.n_dyn);
  const int dyn_lo = a.pad + a.n_sink;
  const int n_keys = a.n_pages * kPageSize;
  int32_t* list = a.list;
  const int32_t* table = a.table;

  if (token_needs_scores(a)) {
    auto put = [&](int pos, int c) { list[a.n_sink + pos] = c; };
    if constexpr (LDSK)
      radix_select_emit<NW>(LdsKeys{a.lds_keys, n_keys}, n_keys, (uint32_t)k_eff, first_digit_counted, sh, put);
    else
      radix_select_emit<NW>(GlobalKeys{make_rsrc(a.keys, n_keys * 4)}, n_keys, (uint32_t)k_eff, first_digit_counted, sh, put);
    __syncthreads();
    translate_slots<NT>(list, a.n_sink, k_eff, table, a.pad, a.sel_tokens);
  } else if (k_eff > 0) {
    // Budget covers every candidate: all of them, no key needed.
    for (int i = tid; i < k_eff; i += NT) {
      list[a.n_sink + i] = phys_token(table, dyn_lo + i);
      if (a.sel_tokens) a.sel_tokens[a.n_sink + i] = a.n_sink + i;
    }
  }
  for (int i = tid; i < a.n_sink + a.n_local; i += NT) {
    const bool sink = i < a.n_sink;
    const int t = sink ? i : a.n_sink + a.n_dyn + (i - a.n_sink);  // position in the sequence
    const int pos = sink ? i : k_eff + i;
    list[pos] = phys_token(table, a.pad + t);
    if (a.sel_tokens) a.sel_tokens[pos] = t;
  }
  __syncthreads();
  return a.n_sink + k_eff + a.n_local;
}

// What the strided overlapping-block policy needs on top of TokenArgs
// (a.topk and a.keys are not used by it).
struct StridedArgs {
  int block;             // tokens per block
  int stride;            // tokens between block starts
  int topk_blocks;       // budget: 2 * topk_blocks blocks are chosen, at most topk_blocks * block tokens kept
  float* scores;         // HBM scratch, n_pages * 16 entries (LDSK kernels: TokenArgs::lds_keys holds them instead)
  uint32_t* block_keys;  // HBM scratch, >= n_pages * 16 entries, 16-byte aligned
  uint32_t* bitmap;      // LDS, one bit per candidate token: (n_dyn + 31) / 32 words
  int32_t* winners;      // LDS, room for 2 * topk_blocks block numbers
};

// Strided overlapping-block top-k: block i covers the candidate tokens
// [i*stride, i*stride + block); the min(2*topk_blocks, num_blocks) blocks with the
// largest mean score are chosen, their tokens united, and the topk_blocks*block
// lowest-positioned of those kept.  With fewer candidates than one block every
// token is listed.  strided_needs_scores() / strided_score_tokens() over a page
// range / strided_select_list(), as for the token policy.

__device__ __forceinline__ bool strided_needs_scores(const TokenArgs& a, const StridedArgs& sa) {
  if (a.n_dyn < sa.block || sa.topk_blocks <= 0) return false;
  const int num_blocks = (a.n_dyn - sa.block) / sa.stride + 1;
  return 2 * sa.topk_blocks < num_blocks;  // otherwise every block is chosen
}

// fp32 scores of the tokens of the pages pg0 <= p < pg1 -> sa.scores (device-scope
// stores) or, LDSK, -> a.lds_keys (as bit patterns).
template <int NW, bool LDSK = false, bool F16 = false, int HD = kHeadDim>
__device__ __forceinline__ void strided_score_tokens(const TokenArgs& a, const StridedArgs& sa, int pg0, int pg1) {
  const __amdgpu_buffer_rsrc_t scores_rsrc = make_rsrc(sa.scores, LDSK ? 0 : a.n_pages * kPageSize * 4);
  uint32_t* lds_scores = a.lds_keys;
  const int dump = a.n_pages * kPageSize;
  stream_token_scores<NW, F16, HD>(a, pg0, pg1, [&](int c, float score, bool valid) {
    if constexpr (LDSK)
      lds_scores[valid ? c : dump] = __float_as_uint(score);
    else
      __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(score), scores_rsrc, valid ? c * 4 : -1, 0, kDeviceScope);
  });
}

// Writes the token list to a.list (sink tokens, kept tokens in ascending order,
// local tokens) and returns its length; sa.scores (LDSK: a.lds_keys) is complete when
// strided_needs_scores().  sa.winners may overlap the LDS scores: they are dead by the
// time the winners are written.  Ends with a barrier.
template <int NG, int NW, bool LDSK = false>
__device__ __forceinline__ int strided_select_list(const TokenArgs& a, const StridedArgs& sa, KeySelectShared* sh) {
  constexpr int NT = NW * 64;
  __shared__ uint32_t wave_cnt[NW];
  uint32_t* hist = sh->hist[0];

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63;
  const int dyn_lo = a.pad + a.n_sink;
  const int L = a.n_dyn;
  int32_t* list = a.list;
  const int32_t* table = a.table;
  int kept = 0;  // candidate tokens listed

  if (L < sa.block) {
    // Too short for block sparsity: everything is attended.
    for (int i = tid; i < L; i += NT) {
      list[a.n_sink + i] = phys_token(table, dyn_lo + i);
      if (a.sel_tokens) a.sel_tokens[a.n_sink + i] = a.n_sink + i;
    }
    kept = L;
  } else {
    const int num_blocks = (L - sa.block) / sa.stride + 1;
    const int k_blocks = min(2 * sa.topk_blocks, num_blocks);
    const int budget = sa.topk_blocks * sa.block;
    const int n_words = (L + 31) >> 5;
    for (int i = tid; i < n_words; i += NT) sa.bitmap[i] = 0u;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    // ---- chosen blocks -> token bitmap ---------------------------------------
    auto mark_block = [&](int i) {
      const int t0 = i * sa.stride, t1 = t0 + sa.block;  // candidate-relative token range
      for (int wd = t0 >> 5; wd <= (t1 - 1) >> 5; ++wd) {
        const int lo = max(t0, wd << 5) & 31, hi = min(t1, (wd + 1) << 5) - (wd << 5);  // bits [lo, hi) of the word
        const uint32_t m = (hi >= 32 ? 0xffffffffu : ((1u << hi) - 1u)) & ~((1u << lo) - 1u);
        atomicOr(&sa.bitmap[wd], m);
      }
    };
    if (k_blocks == 0) {
      // no budget: nothing of the dynamic part is attended
    } else if (k_blocks < num_blocks) {
      // block means -> keys (padded with "no candidate" to a multiple of 16)
      const int nb_pad = (num_blocks + 15) & ~15;
      const float inv = 1.0f / (float)sa.block;
      const __amdgpu_buffer_rsrc_t scores_rsrc = make_rsrc(sa.scores, a.n_pages * kPageSize * 4);
      const __amdgpu_buffer_rsrc_t bkeys_rsrc = make_rsrc(sa.block_keys, nb_pad * 4);
      for (int i = tid; i < nb_pad; i += NT) {
        uint32_t key = 0u;
        if (i < num_blocks) {
          const int off = (dyn_lo + i * sa.stride) * 4;
          float sum = 0.f;
          if constexpr (LDSK) {
            for (int t = 0; t < sa.block; ++t) sum += __uint_as_float(a.lds_keys[(off >> 2) + t]);
          } else {
            // 16 scores requested together (one memory round trip per 16 instead of one per score), added in token order
            for (int t0 = 0; t0 < sa.block; t0 += 16) {
              uint32_t x[16];
#pragma unroll
              for (int i = 0; i < 16; ++i)
                x[i] = __builtin_amdgcn_raw_buffer_load_b32(scores_rsrc, off + (t0 + i) * 4, 0, kDeviceScope);
#pragma unroll
              for (int i = 0; i < 16; ++i)
                if (t0 + i < sa.block) sum += __uint_as_float(x[i]);
            }
          }
          key = order_key(sum * inv);
          atomicAdd(&hist[key >> 24], 1u);
        }
        __builtin_amdgcn_raw_buffer_store_b32(key, bkeys_rsrc, i * 4, 0, kDeviceScope);
      }
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      radix_select_emit<NW>(GlobalKeys{bkeys_rsrc}, nb_pad, (uint32_t)k_blocks, true, sh, [&](int pos, int i) { sa.winners[pos] = i; });
      __syncthreads();
      for (int i = tid; i < k_blocks; i += NT) mark_block(sa.winners[i]);
    } else {
      for (int i = tid; i < num_blocks; i += NT) mark_block(i);
    }
    __syncthreads();
    // ---- bitmap -> token list, ascending, the first `budget` tokens ----------------
    const int per = (n_words + NT - 1) / NT;  // consecutive words per thread
    const int w_lo = min(tid * per, n_words), w_hi = min(w_lo + per, n_words);
    uint32_t cnt = 0;
    for (int i = w_lo; i < w_hi; ++i) cnt += __popc(sa.bitmap[i]);
    uint32_t incl = cnt;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off);
      if (l >= off) incl += up;
    }
    if (l == 63) wave_cnt[w] = incl;
    __syncthreads();
    uint32_t pos = incl - cnt, total = 0;
    for (int wv = 0; wv < NW; ++wv) {
      if (wv < w) pos += wave_cnt[wv];
      total += wave_cnt[wv];
    }
    for (int i = w_lo; i < w_hi && pos < (uint32_t)budget; ++i) {
      uint32_t bits = sa.bitmap[i];
      while (bits && pos < (uint32_t)budget) {
        const int t = (i << 5) + __builtin_ctz(bits);
        bits &= bits - 1u;
        list[a.n_sink + pos] = dyn_lo + t;  // cache slot; translated below
        ++pos;
      }
    }
    kept = (int)min(total, (uint32_t)budget);
    __syncthreads();
    translate_slots<NT>(list, a.n_sink, kept, table, a.pad, a.sel_tokens);
  }
  for (int i = tid; i < a.n_sink + a.n_local; i += NT) {
    const bool sink = i < a.n_sink;
    const int t = sink ? i : a.n_sink + a.n_dyn + (i - a.n_sink);  // position in the sequence
    const int pos = sink ? i : kept + i;
    list[pos] = phys_token(table, a.pad + t);
    if (a.sel_tokens) a.sel_tokens[pos] = t;
  }
  __syncthreads();
  return a.n_sink + kept + a.n_local;
}

// Attention over a list of n = a.n physical token ids in LDS (a.p0 / a.p1 /
// a.last_len / a.first_skip of AttendArgs are not used).  Same tiles, staging
// and online softmax as attend_list(); a "page" is any 16 consecutive list
// entries, each K and V row fetched from its own address.
// lds: attend_lds_bytes(NW); sm_m / sm_l: NW x (4*NG) floats each.
template <int NG, int NW, bool F16 = false, int HD = kHeadDim, typename Emit>
__device__ __forceinline__ void attend_tokens(const AttendArgs& a, const int32_t* list, unsigned char* lds,
                                              float (*sm_m)[4 * NG], float (*sm_l)[4 * NG], Emit emit) {
  constexpr int CPR = HD / 8;                   // 16-byte chunks of a head row
  constexpr int KC = HD / 32;                   // matrix steps over the head dimension = LDS-direct loads per tile
  constexpr int RPI = 64 / CPR;                 // K rows one LDS-direct load brings
  constexpr int NV = attend_v_loads<NG, HD>();  // V rows per lane and tile
  constexpr int kStage = kPageSize * HD * 2;    // bytes of one K stage
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, kg = l >> 4, c16 = l & 15, gq = l & 3, cc = c16 & (CPR - 1);
  const int half = NV == 2 ? (c16 >> 3) : 0;
  const int vrow0 = 4 * kg + 2 * half;          // tile row of this lane's first V row
  const int G = a.G;
  const int n = a.n;

  uint4 qB[KC];
  {
    const int g = min(NG == 4 ? c16 : gq, G - 1);
    const uint16_t* qp = a.q_bh + (int64_t)g * HD + 8 * kg;
#pragma unroll
    for (int c = 0; c < KC; ++c) qB[c] = *reinterpret_cast<const uint4*>(qp + 32 * c);
  }

  const int row_bytes = a.row_bytes;
  const int page_bytes = a.page_bytes;
  const char* kvb = a.kvb;
  const int64_t max_tok = a.num_pages * kPageSize;
  unsigned char* kl = lds + w * (kAttendStages * kStage);
  int krow[KC], kchunk[KC], lds_r[KC];
#pragma unroll
  for (int c = 0; c < KC; ++c) {
    krow[c] = RPI * c + l / CPR;                                           // K row this lane helps to fetch with load c
    kchunk[c] = ((cc ^ attend_swizzle<HD>(krow[c])) & (CPR - 1)) * 16;      // the chunk that belongs at its LDS position
    lds_r[c] = c16 * (HD * 2) + (((4 * c + kg) ^ attend_swizzle<HD>(c16)) & (CPR - 1)) * 16;
  }
  const int vchunk = kPageSize * row_bytes + cc * 16;  // V plane of the page, this lane's columns

  float m_run = kNegInf, l_run = 0.f;
  floatx4 O[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) O[u] = floatx4{0.f, 0.f, 0.f, 0.f};
  auto scores = [&](const uint4 (&ka)[KC], float (&pr)[4], int valid) {
    if constexpr (NG == 4)
      page_scores_wide<F16, KC>(ka, qB, m_run, l_run, O, pr, a.scale_log2, 0, valid, kg);
    else
      page_scores<F16, KC>(ka, qB, m_run, l_run, O, pr, a.scale_log2, 0, valid, kg);
  };
  auto pv = [&](const u32x4 (&vr)[NV], const float (&pr)[4]) {
    if constexpr (NG == 4)
      page_pv_wide<F16, HD>(vr, pr, O, 16 * (c16 >> 3));
    else
      page_pv<F16, NV>(vr, pr, O, half);
  };

  // This wave takes the 16-entry groups w, w+NW, ...  Entries past the end (and
  // ids outside the cache) read token 0 of the cache and are masked.
  const int groups = (n + kPageSize - 1) / kPageSize;
  const int iters = (groups > w) ? (groups - w + NW - 1) / NW : 0;
  auto row_ptr = [&](int tok) -> const char* {
    const bool ok = tok >= 0 && (int64_t)tok < max_tok;
    const int t = ok ? tok : 0;
    return kvb + (int64_t)(t >> 4) * page_bytes + (t & (kPageSize - 1)) * row_bytes;
  };
  struct Ids { int k[KC], v[NV], valid; };
  auto fetch_ids = [&](int it) {
    Ids ids;
    const int base = (w + NW * it) * kPageSize;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int e = base + krow[c];
      ids.k[c] = (e < n) ? list[e] : -1;
    }
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int e = base + vrow0 + r;
      ids.v[r] = (e < n) ? list[e] : -1;
    }
    ids.valid = max(0, min(kPageSize, n - base));
    return ids;
  };
  auto issue_v = [&](const Ids& ids, u32x4 (&vv)[NV]) {
#pragma unroll
    for (int r = 0; r < NV; ++r)
      vv[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row_ptr(ids.v[r]) + vchunk));
  };
  auto issue_k = [&](const Ids& ids, int stage) {
    __attribute__((address_space(3))) unsigned char* dst =
        (__attribute__((address_space(3))) unsigned char*)(kl + stage * kStage);
#pragma unroll
    for (int c = 0; c < KC; ++c)
      __builtin_amdgcn_global_load_lds(
          reinterpret_cast<const __attribute__((address_space(1))) void*>(
              reinterpret_cast<uintptr_t>(row_ptr(ids.k[c]) + kchunk[c])),
          dst + c * 1024, 16, 0, kStreamLoad);
  };
  auto read_k = [&](int stage, uint4 (&ka)[KC]) {
#pragma unroll
    for (int c = 0; c < KC; ++c) ka[c] = *reinterpret_cast<const uint4*>(kl + stage * kStage + lds_r[c]);
  };

  // Same explicit wait as in attend_list(): when it executes, exactly the NV V
  // loads issued just before it may be outstanding.
  if (iters > 0) {
    u32x4 vA[NV], vB[NV];
    uint4 ka[KC];
    float pr[4];
    Ids idA = fetch_ids(0), idB;
    issue_k(idA, 0);
    issue_v(idA, vA);
    for (int it = 0; it < iters; it += 2) {
      {
        idB = fetch_ids(it + 1);
        __builtin_amdgcn_sched_barrier(0);
        issue_v(idB, vB);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(wait_vm_imm(NV));
        __builtin_amdgcn_sched_barrier(0);
        read_k(0, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(idB, 1);
        __builtin_amdgcn_sched_barrier(0);
        scores(ka, pr, idA.valid);
        if (idA.valid != kPageSize) clear_unused_v_rows<NV>(vA, 0, idA.valid, vrow0);
        pv(vA, pr);
      }
      {
        idA = fetch_ids(it + 2);
        __builtin_amdgcn_sched_barrier(0);
        issue_v(idA, vA);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(wait_vm_imm(NV));
        __builtin_amdgcn_sched_barrier(0);
        read_k(1, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(idA, 0);
        __builtin_amdgcn_sched_barrier(0);
        scores(ka, pr, idB.valid);
        if (idB.valid != kPageSize) clear_unused_v_rows<NV>(vB, 0, idB.valid, vrow0);
        pv(vB, pr);
      }
    }
  }
  attend_finish<NG, NW, HD>(m_run, l_run, O, G, lds, sm_m, sm_l, emit);
}

}  // namespace kin
