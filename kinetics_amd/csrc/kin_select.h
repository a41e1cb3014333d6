// Device-side building block: page scoring + top-k page selection for one
// (sequence, KV head), run by one workgroup of NT = 256 .. 1024 threads.  Shared by the
// stand-alone selector kernel and the fused decode-step kernel.
//
//   phase 1  stream the sequence's representative keys (256 B each) once,
//            16 lanes per key with 16-byte loads, fp32 dot with the group-mean
//            query, DPP reduction inside each 16-lane row; scores stay in LDS
//            as order-preserving 32-bit keys (never written to HBM);
//   phase 2  8-bit radix select in LDS for the k-th largest key (the first digit
//            is counted while the scores are produced);
//   phase 3  gather the winners (ties at the threshold by lowest index), order
//            them (score descending, index ascending) in LDS -- by counting for
//            k <= 512, by bitonic sort above -- translate logical -> physical
//            page ids and append the last page.  The sequence's page table is
//            copied to LDS while the mean keys stream, so the translation costs
//            no memory round trip (under a saturated read stream a dependent
//            global load takes microseconds).
// HBM-bound on phase 1: n_cand * 256 B per workgroup.
#pragma once

#include "kin_common.h"

namespace kin {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Monotone map float -> uint32: a < b  <=>  key(a) < key(b)  (-0 < +0).
__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}

constexpr int kThreads = 256;  // workgroup size of the stand-alone selector
constexpr int kRankSortMax = 512;   // up to here winners are ordered by counting, above by bitonic sort

// Statically allocated LDS of one selection problem (one per workgroup).
struct SelectScratch {
  uint32_t hist[4][256];  // one histogram per radix digit; all zero when a selection starts (see clear_select_scratch)
  uint32_t wave_tot[16];
  uint32_t count;
  uint32_t run_cnt[kMaxCandidates / 64];  // winners in each run of 64 candidates (index-ordered listing)
};

// Zeroes the histograms.  Every thread of the workgroup calls it; the caller puts a
// barrier between this and the first score_rows<..., COUNT0 = true> / select_from_keys().
template <int NT>
__device__ __forceinline__ void clear_select_scratch(SelectScratch* ss) {
  for (int i = threadIdx.x; i < 4 * 256; i += NT) (&ss->hist[0][0])[i] = 0;
}

// Wave-uniform description of one selection problem.
struct SelectArgs {
  const uint16_t* q_bh;       // the group's G query rows
  int G;
  const char* kb;             // representative key of the first candidate of (b, h); the others follow, 256 B each
  int n_pages;                // pages of the sequence (>= 1)
  int n_sink;                 // leading pages that are always attended (not candidates)
  int n_cand;                 // candidates: logical pages n_sink .. n_sink + n_cand - 1
  int n_local;                // trailing pages that are always attended (>= 1: the open page last)
  int topk;
  const int32_t* table;       // the sequence's page table (logical -> physical)
  int32_t* sel_logical;       // HBM, topk entries, or null
  float* scores_out;          // HBM, entry n = score of candidate n, or null
  uint32_t* keys;             // LDS, >= n_cand entries
  unsigned long long* sortbuf;  // LDS, sort_cap entries
  int sort_cap;               // power of two >= min(topk, capacity)
  SelectScratch* ss;          // LDS, histograms zeroed
  bool sorted;                // list the winners by descending score (ties: ascending index) as torch.topk does; else by
                              // ascending index, which needs no sort (the attention's sum does not care)
  const int32_t* table_lds;   // LDS copy of table[0 .. n_pages) (see prefetch_table), or null: look up in global memory
  bool digit0_counted;        // ss->hist[0] already holds the first digit of every candidate's key
};

// table_cap: entries reserved for the LDS copy of a page table (a multiple of 64, 0: none);
// it follows the sort buffer.
__host__ __device__ inline size_t select_lds_bytes(int kbar_pages, int sort_cap, int table_cap = 0) {
  return (size_t)((kbar_pages + 3) & ~3) * 4 + (size_t)sort_cap * 8 + (size_t)table_cap * 4;
}
__host__ __device__ inline size_t select_table_offset(int kbar_pages, int sort_cap) {
  return (size_t)((kbar_pages + 3) & ~3) * 4 + (size_t)sort_cap * 8;
}

// Largest page table that is copied to LDS (16 KiB); longer sequences translate through global memory.
constexpr int kMaxTableLds = 4096;
// Entries to reserve so that every sequence of up to max_pages pages gets the copy, capped at
// kMaxTableLds: a multiple of 64 (whole wave loads).  Whether a sequence fits is decided per sequence.
__host__ __device__ inline int select_table_cap(int max_pages) {
  const int want = (max_pages + 63) & ~63;
  return want < kMaxTableLds ? want : kMaxTableLds;
}

// Starts the copy of table[0 .. n_pages) to dst (LDS, room for table_cap entries) with LDS-direct
// loads (no registers are held while they are in flight) when n_pages fits; returns dst then, else
// null.  Every thread of the workgroup calls it.  The data may be read after
// every wave has waited for its loads (s_waitcnt vmcnt(0)) and a workgroup barrier.
template <int NT>
__device__ __forceinline__ const int32_t* prefetch_table(const int32_t* table, int n_pages, int32_t* dst, int table_cap) {
  if (n_pages > table_cap || n_pages <= 0) return nullptr;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const __amdgpu_buffer_rsrc_t r = make_rsrc(table, n_pages * 4);   // past the end: zeros, no traffic
  const int chunks = (n_pages + 63) >> 6;                            // 64 entries = 256 B per wave load
  for (int c = wave; c < chunks; c += NT / 64) {
    __attribute__((address_space(3))) unsigned char* d =
        (__attribute__((address_space(3))) unsigned char*)(dst + c * 64);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, d, 4, (c * 64 + lane) * 4, 0, 0, 0);
  }
  return dst;
}

__host__ __device__ inline int select_sort_cap(int topk, int kbar_pages) {
  const int need = topk < kbar_pages ? topk : kbar_pages;  // k_eff never exceeds either
  int cap = 2;
  while (cap < need) cap <<= 1;
  return cap;
}

// Splits a sequence of n_pages pages (the last one holding last_len tokens)
// into always-attended leading ("sink") pages, candidates and always-attended
// trailing ("local") pages.  The candidates are the whole pages between the sink
// pages and the newest local_tokens tokens, so the open page (local_tokens >= 1)
// is always local.  kbar_pages bounds the logical pages that have a mean key.
__host__ __device__ inline void split_pages(int n_pages, int last_len, int sink_pages, int local_tokens,
                                            int kbar_pages, int page_size, int& n_sink, int& n_cand, int& n_local) {
  last_len = last_len < 1 ? 1 : (last_len > page_size ? page_size : last_len);
  n_sink = sink_pages < n_pages - 1 ? sink_pages : n_pages - 1;
  const int between = (n_pages - 1 - n_sink) * page_size + last_len - local_tokens;  // tokens after the sink, before the local part
  n_cand = between > 0 ? between / page_size : 0;
  n_local = n_pages - n_sink - n_cand;
  const int cap = kbar_pages - n_sink;
  if (n_cand > cap) n_cand = cap > 0 ? cap : 0;
}

// One digit of a most-significant-digit-first radix select, run by ONE wave:
// hist[256] counts the keys that match the digits fixed so far, by their next
// digit; `remaining` of them are wanted, largest first.  Writes the digit that
// holds the threshold and how many keys of that digit are still wanted.
__device__ __forceinline__ void radix_pick_bin(const uint32_t* hist, uint32_t remaining, int lane, uint32_t* out_bin,
                                               uint32_t* out_remaining) {
  // Lane j owns bins 255-4j .. 252-4j (highest first); an inclusive scan over
  // lanes counts the keys in all bins at or above the lane's lowest.  The bin
  // where the running count first reaches `remaining` holds the threshold digit.
  const int top = 255 - 4 * lane;
  const uint32_t c0 = hist[top], c1 = hist[top - 1], c2 = hist[top - 2], c3 = hist[top - 3];
  const uint32_t mine = c0 + c1 + c2 + c3;
  uint32_t incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  uint32_t run = incl - mine;  // keys in bins above this lane's
  if (run < remaining && remaining <= incl) {
    int bin = top;
    uint32_t c = c0;
    if (run + c < remaining) { run += c; bin = top - 1; c = c1; }
    if (run + c < remaining) { run += c; bin = top - 2; c = c2; }
    if (run + c < remaining) { run += c; bin = top - 3; }
    *out_bin = (uint32_t)bin;
    *out_remaining = remaining - run;
  }
}

// The same digit pick made by EVERY wave that calls it (all 64 lanes), with the
// result in every lane: no shared variable, so no barrier after it.  exhausted:
// the keys wanted from the threshold bin are all the keys in it (every key with the
// digits fixed so far, this one included, is taken: no further digit is needed).
__device__ __forceinline__ void radix_pick_bin_uniform(const uint32_t* hist, uint32_t remaining, int lane, uint32_t& bin_out,
                                                       uint32_t& remaining_out, bool& exhausted) {
  const int top = 255 - 4 * lane;
  const uint32_t c0 = hist[top], c1 = hist[top - 1], c2 = hist[top - 2], c3 = hist[top - 3];
  const uint32_t mine = c0 + c1 + c2 + c3;
  const uint32_t incl = wave_inclusive_sum(mine);
  uint32_t run = incl - mine;  // keys in bins above this lane's
  const bool owner = run < remaining && remaining <= incl;
  uint32_t bin = 0, rem = 0, cnt = 0;
  if (owner) {
    bin = top;
    uint32_t c = c0;
    if (run + c < remaining) { run += c; bin = top - 1; c = c1; }
    if (run + c < remaining) { run += c; bin = top - 2; c = c2; }
    if (run + c < remaining) { run += c; bin = top - 3; c = c3; }
    rem = remaining - run;
    cnt = c;
  }
  // exactly one lane owns the threshold bin (1 <= remaining <= number of counted keys)
  const unsigned long long who = __ballot(owner);
  const int src = who ? __builtin_ctzll(who) : 0;
  bin_out = (uint32_t)__builtin_amdgcn_readlane((int)bin, src);
  remaining_out = (uint32_t)__builtin_amdgcn_readlane((int)rem, src);
  exhausted = (uint32_t)__builtin_amdgcn_readlane((int)cnt, src) == remaining_out;
}

// Scores the candidates r0 <= r < r1 of one (sequence, KV head) with the
// group-mean query and stores them as order-preserving keys in keys_out[r] (LDS
// or global memory) and, if a.scores_out is set, as fp32 in scores_out[r].
// Streams (r1 - r0) * 256 B; no barrier inside.  DEVICE_VISIBLE: keys_out is global
// memory that a workgroup on another XCD will read in this launch: the stores
// are made at device scope (past this XCD's L2).
// NT: threads of the workgroup (a multiple of 256, all of them call this).
// UNROLL: independent 16-byte loads each lane keeps in flight while streaming the
// mean keys (4 saturates HBM when thousands of workgroups run; a small grid
// needs more per workgroup).
// COUNT0: also count every key's first radix digit in a.ss->hist[0] (LDS atomics spread
// over the streaming, instead of a pass over the keys afterwards).
// HD: elements of a head row (128 or 64): HD / 8 lanes share a mean key, 16 bytes each.
template <int UNROLL, int NT, bool DEVICE_VISIBLE = false, bool F16 = false, bool COUNT0 = false, int HD = kHeadDim>
__device__ __forceinline__ void score_rows(const SelectArgs& a, int r0, int r1, uint32_t* keys_out) {
  constexpr int kUnroll = UNROLL;
  constexpr int kLanes = HD / 8;      // lanes per mean key
  constexpr int kRows = NT / kLanes;  // mean keys one pass of the workgroup covers
  constexpr int kRowB = HD * 2;       // bytes of a mean key
  const int tid = threadIdx.x;
  // Lane owns columns d = 8*c16 .. +7 of the mean query.
  const int c16 = tid & (kLanes - 1);
  // The group's query rows are requested four at a time (a loop of single loads would pay one memory
  // round trip per head), the first four before the first mean keys and averaged after those are
  // under way, so that the stream starts one round trip after the call.
  const uint16_t* qp = a.q_bh + 8 * c16;
  auto load_q_rows = [&](uint4 (&qv)[4], int g0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) qv[i] = *reinterpret_cast<const uint4*>(qp + (int64_t)min(g0 + i, a.G - 1) * HD);
  };
  auto add_q_rows = [&](float (&qm)[8], const uint4 (&qv)[4], int g0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (g0 + i < a.G) {
        const uint4 w = qv[i];
        qm[0] += elem_lo<F16>(w.x); qm[1] += elem_hi<F16>(w.x);
        qm[2] += elem_lo<F16>(w.y); qm[3] += elem_hi<F16>(w.y);
        qm[4] += elem_lo<F16>(w.z); qm[5] += elem_hi<F16>(w.z);
        qm[6] += elem_lo<F16>(w.w); qm[7] += elem_hi<F16>(w.w);
      }
    }
  };
  uint4 qv0[4];
  load_q_rows(qv0, 0);
  // The candidates of (b, h) are contiguous rows of 256 B (128 B for HD = 64).  They are read
  // through a buffer descriptor that ends after the last wanted row, so loads past
  // the end return zeros without touching memory and the loop needs no branches:
  // each lane keeps kUnroll 16-byte loads in flight, re-issuing slot j for the
  // next pass as soon as it has consumed it.  The hardware compares only the
  // per-lane (VGPR) offset with the descriptor's size -- the scalar offset operand
  // is added after the range check -- so the whole offset travels in the VGPR and
  // the scalar operand stays 0.
  constexpr int row_stride_b = kRowB;  // the list's mean keys are contiguous rows (head-major kbar)
  const int n = r1 > r0 ? r1 - r0 : 0;
  const char* kb = a.kb + (int64_t)r0 * row_stride_b;
  float* sc_out = a.scores_out;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(kb), 0, n > 0 ? (n - 1) * row_stride_b + kRowB : 0, 0x00020000);
  const int sub = tid / kLanes;  // which of the kRows rows of a slot this lane helps with
  const int lane_off = sub * row_stride_b + c16 * 16;
  u32x4 w[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j)
    w[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off + j * kRows * row_stride_b, 0, kStreamLoad);
  float qm[8];
  {
#pragma unroll
    for (int u = 0; u < 8; ++u) qm[u] = 0.f;
    add_q_rows(qm, qv0, 0);
    for (int g0 = 4; g0 < a.G; g0 += 4) {
      uint4 qv[4];
      load_q_rows(qv, g0);
      add_q_rows(qm, qv, g0);
    }
    const float inv = 1.0f / (float)a.G;
#pragma unroll
    for (int u = 0; u < 8; ++u) qm[u] *= inv;
  }
  KIN_STAMP(16);  // mean query in registers
  for (int base = 0; base < n; base += kRows * kUnroll) {
    const int next_off = lane_off + (base + kRows * kUnroll) * row_stride_b;
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
      const u32x4 x = w[j];
      w[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, next_off + j * kRows * row_stride_b, 0, kStreamLoad);
      float acc = 0.f;
      acc = fmaf(qm[0], elem_lo<F16>(x.x), acc); acc = fmaf(qm[1], elem_hi<F16>(x.x), acc);
      acc = fmaf(qm[2], elem_lo<F16>(x.y), acc); acc = fmaf(qm[3], elem_hi<F16>(x.y), acc);
      acc = fmaf(qm[4], elem_lo<F16>(x.z), acc); acc = fmaf(qm[5], elem_hi<F16>(x.z), acc);
      acc = fmaf(qm[6], elem_lo<F16>(x.w), acc); acc = fmaf(qm[7], elem_hi<F16>(x.w), acc);
      acc = row_sum<kLanes>(acc);
      const int row = base + j * kRows + sub;
      if (c16 == 0 && row < n) {
        const uint32_t key = order_key(acc);
        if (DEVICE_VISIBLE)
          __hip_atomic_store(keys_out + r0 + row, key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else
          keys_out[r0 + row] = key;
        if (COUNT0) atomicAdd(&a.ss->hist[0][key >> 24], 1u);
        if (sc_out) sc_out[r0 + row] = acc;
      }
    }
  }
}

// Copies the n keys that the workgroups sharing one list's scoring wrote to global
// memory (at device scope, 16-byte aligned) into LDS (16-byte aligned, room for n
// rounded up to 4): 16-byte device-scope loads, four per thread in flight -- one
// round trip for up to 16 * NT keys instead of one per key and thread.  The caller
// puts a barrier after it.
template <int NT>
__device__ __forceinline__ void load_shared_keys(const uint32_t* gkeys, int n, uint32_t* keys_lds) {
  const __amdgpu_buffer_rsrc_t r = make_rsrc(gkeys, n * 4);  // past n: zeros
  u32x4* dst = reinterpret_cast<u32x4*>(keys_lds);
  const int n4 = (n + 3) >> 2;
  for (int base = threadIdx.x; base < n4; base += 4 * NT) {
    u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b128(r, (base + u * NT) * 16, 0, kDeviceScope);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (base + u * NT < n4) dst[base + u * NT] = v[u];
  }
}

// Selects from the keys of the n_cand candidates in a.keys (LDS) and writes the
// page list to sel_lds (LDS, >= n_sink + topk + n_local entries): the sink
// pages, then the ordered physical ids of the k_eff winners, then the local
// pages (the open page last).  Returns the list length.  The caller has put a
// workgroup barrier between the last key write (and the last count into
// a.ss->hist[0], and the arrival of a.table_lds) and this call; it ends with one:
// sel_lds is visible to every thread and keys / sortbuf are free for reuse.
// a.ss->hist is left dirty: clear_select_scratch() before the next selection.
template <int NT>
__device__ __forceinline__ int select_from_keys(const SelectArgs& a, int32_t* sel_lds) {
  SelectScratch& ss = *a.ss;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n_cand = a.n_cand, n_pages = a.n_pages;
  const int k_eff = min(a.topk, n_cand);
  uint32_t* keys = a.keys;
  unsigned long long* sortbuf = a.sortbuf;

  // ---- phase 2: radix select of the k_eff-th largest key -------------------
  // One barrier per digit: the histograms are separate arrays zeroed together, and
  // every wave reads the digit's histogram for itself.  The loop stops as soon as the
  // threshold bin is wanted whole (usually after two or three digits).
  uint32_t prefix = 0, mask = 0;
  uint32_t remaining = (uint32_t)k_eff;  // how many keys equal to the threshold are taken
  uint32_t thr = 0;
  KIN_STAMP(20);  // select starts
  if (k_eff > 0 && k_eff < n_cand) {
    bool whole_bin = false;
    for (int pass = 0; pass < 4 && !whole_bin; ++pass) {
      const int shift = 24 - 8 * pass;
      if (pass > 0 || !a.digit0_counted) {
        for (int i = tid; i < n_cand; i += NT) {
          const uint32_t key = keys[i];
          if ((key & mask) == prefix) atomicAdd(&ss.hist[pass][(key >> shift) & 255u], 1u);
        }
        __syncthreads();
      }
      uint32_t bin;
      radix_pick_bin_uniform(ss.hist[pass], remaining, lane, bin, remaining, whole_bin);
      prefix |= bin << shift;
      mask |= 255u << shift;
      KIN_STAMP(21 + pass);  // digit fixed
    }
    if (whole_bin && prefix != 0) {
      // every key that starts with `prefix` is a winner: they all compare above prefix - 1,
      // and nothing else does except the keys of higher bins
      thr = prefix - 1u;
      remaining = 0;
    } else {
      thr = prefix;  // all 32 bits fixed (or prefix 0): `remaining` of the keys equal to thr are taken
    }
  }
  const bool take_all = (k_eff >= n_cand);
  // Logical -> physical page id: from the LDS copy of the table when there is one.  The copy is read
  // through a pointer typed as LDS: through a generic pointer the loads would be flat instructions,
  // which queue up behind the CU's global loads (microseconds under a saturated read stream).
  typedef const __attribute__((address_space(3))) int32_t* lds_table_t;
  const lds_table_t table_lds = (lds_table_t)a.table_lds;
  const bool have_lds_table = a.table_lds != nullptr;
  auto table = [&](int i) -> int32_t { return have_lds_table ? table_lds[i] : a.table[i]; };

  if (!a.sorted) {
    // ---- phase 3, listing by ascending index: an ordered compaction, no sort -------
    // Wave w owns the runs of 64 consecutive candidates w, w + NT/64, ...; it counts each run's
    // winners (low half: keys above the threshold; high half: keys equal to it), one wave turns
    // the counts into offsets, and every wave writes its winners in place.  Of the keys equal
    // to the threshold the `remaining` lowest-indexed count.
    const int runs = (n_cand + 63) >> 6;
    auto classify = [&](int i, bool& gt, bool& eq) {
      const uint32_t key = i < n_cand ? keys[i] : 0u;
      gt = i < n_cand && (take_all || key > thr);
      eq = i < n_cand && !take_all && remaining > 0 && key == thr;
    };
    if (k_eff > 0) {
      for (int r = wave; r < runs; r += NT / 64) {
        bool gt, eq;
        classify(r * 64 + lane, gt, eq);
        const uint32_t c = (uint32_t)__popcll(__ballot(gt)) | ((uint32_t)__popcll(__ballot(eq)) << 16);
        if (lane == 0) ss.run_cnt[r] = c;
      }
    }
    __syncthreads();
    if (k_eff > 0 && wave == 0) {
      // exclusive prefix over the runs, 64 at a time (halves add without carry: at most 16384 candidates)
      uint32_t carry = 0;
      for (int r0 = 0; r0 < runs; r0 += 64) {
        const uint32_t c = r0 + lane < runs ? ss.run_cnt[r0 + lane] : 0u;
        const uint32_t incl = wave_inclusive_sum(c);
        if (r0 + lane < runs) ss.run_cnt[r0 + lane] = carry + incl - c;
        carry += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
      }
    }
    __syncthreads();
    if (k_eff > 0) {
      for (int r = wave; r < runs; r += NT / 64) {
        bool gt, eq;
        const int i = r * 64 + lane;
        classify(i, gt, eq);
        const unsigned long long bg = __ballot(gt), be = __ballot(eq);
        const uint32_t before = ss.run_cnt[r];
        const uint32_t gt_before = (before & 0xffffu) + __builtin_amdgcn_mbcnt_hi((uint32_t)(bg >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bg, 0u));
        const uint32_t eq_before = (before >> 16) + __builtin_amdgcn_mbcnt_hi((uint32_t)(be >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)be, 0u));
        if (gt || (eq && eq_before < remaining))
          sel_lds[a.n_sink + gt_before + min(eq_before, remaining)] = table(a.n_sink + i);
      }
    }
    for (int i = tid; i < a.n_sink + a.n_local; i += NT) {
      if (i < a.n_sink)
        sel_lds[i] = table(i);
      else
        sel_lds[k_eff + i] = table(n_pages - a.n_local + (i - a.n_sink));
    }
    __syncthreads();
    return k_eff + a.n_sink + a.n_local;
  }

  // ---- phase 3: gather, sort, translate --------------------------------------
  const bool rank_sort = (k_eff <= kRankSortMax);
  if (!rank_sort)
    for (int i = tid; i < a.sort_cap; i += NT) sortbuf[i] = 0ull;
  if (tid == 0) ss.count = 0;
  __syncthreads();
  if (k_eff > 0) {
    // Keys above the threshold (or all of them): any order, the sort fixes it.  One slot
    // allocation per wave and step.
    for (int base = 0; base < n_cand; base += NT) {
      const int i = base + tid;
      const uint32_t key = i < n_cand ? keys[i] : 0u;
      const bool win = i < n_cand && (take_all || key > thr);
      const unsigned long long bal = __ballot(win);
      if (bal) {  // wave-uniform
        uint32_t slot0 = 0;
        if (lane == 0) slot0 = atomicAdd(&ss.count, (uint32_t)__popcll(bal));
        slot0 = __shfl(slot0, 0);
        const uint32_t before = __builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0u));
        if (win) sortbuf[slot0 + before] = ((unsigned long long)key << 32) | (uint32_t)(0xffffffffu - (uint32_t)i);
      }
    }
    if (!take_all && remaining > 0) {
      // Keys equal to the threshold: the `remaining` lowest indices, found by an ordered
      // count (every thread owns a run of consecutive candidates).  Only reached when the
      // threshold bin could not be taken whole, i.e. with exact ties at the threshold.
      const int per = (n_cand + NT - 1) / NT;
      const int lo = min(tid * per, n_cand), hi = min(lo + per, n_cand);
      uint32_t eq_cnt = 0;
      for (int i = lo; i < hi; ++i) eq_cnt += (keys[i] == thr) ? 1u : 0u;
      uint32_t incl = eq_cnt;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
      }
      if (lane == 63) ss.wave_tot[wave] = incl;
      __syncthreads();
      uint32_t before = 0;
      for (int wv = 0; wv < wave; ++wv) before += ss.wave_tot[wv];
      uint32_t rank = incl - eq_cnt + before;
      for (int i = lo; i < hi && rank < remaining; ++i) {
        const uint32_t key = keys[i];
        if (key == thr) {
          const uint32_t slot = atomicAdd(&ss.count, 1u);
          sortbuf[slot] = ((unsigned long long)key << 32) | (uint32_t)(0xffffffffu - (uint32_t)i);
          rank++;
        }
      }
    }
  }
  __syncthreads();
  KIN_STAMP(25);  // winners gathered
  if (rank_sort) {
    // Small k: every winner counts the winners that beat it (entries are
    // distinct, so the counts are a permutation) and writes itself to that slot.
    // All lanes read the same LDS word per step: a broadcast, no conflicts.
    for (int i = tid; i < k_eff; i += NT) {
      const unsigned long long mine = sortbuf[i];
      int rank = 0;
#pragma unroll 8
      for (int j = 0; j < k_eff; ++j) rank += (sortbuf[j] > mine) ? 1 : 0;
      const uint32_t logical = 0xffffffffu - (uint32_t)(mine & 0xffffffffull);
      sel_lds[a.n_sink + rank] = table(a.n_sink + logical);
      if (a.sel_logical) a.sel_logical[rank] = (int32_t)(a.n_sink + logical);
    }
  } else {
    // Large k: bitonic sort, descending, over sort_cap (power of two) 64-bit
    // entries; the zero padding sinks to the end.
    for (int size = 2; size <= a.sort_cap; size <<= 1) {
      for (int stride = size >> 1; stride > 0; stride >>= 1) {
        for (int i = tid; i < (a.sort_cap >> 1); i += NT) {
          const int lo_i = 2 * i - (i & (stride - 1));
          const int hi_i = lo_i + stride;
          const bool desc = ((lo_i & size) == 0);
          const unsigned long long x = sortbuf[lo_i], y = sortbuf[hi_i];
          if ((x < y) == desc) {
            sortbuf[lo_i] = y;
            sortbuf[hi_i] = x;
          }
        }
        __syncthreads();
      }
    }
    for (int i = tid; i < k_eff; i += NT) {
      const uint32_t logical = 0xffffffffu - (uint32_t)(sortbuf[i] & 0xffffffffull);
      sel_lds[a.n_sink + i] = table(a.n_sink + logical);
      if (a.sel_logical) a.sel_logical[i] = (int32_t)(a.n_sink + logical);
    }
  }
  for (int i = tid; i < a.n_sink + a.n_local; i += NT) {
    if (i < a.n_sink)
      sel_lds[i] = table(i);
    else
      sel_lds[k_eff + i] = table(n_pages - a.n_local + (i - a.n_sink));
  }
  __syncthreads();
  return k_eff + a.n_sink + a.n_local;
}

// score_rows() over every candidate into a.keys, then select_from_keys().
// a.ss->hist is zero and visible (clear_select_scratch + barrier); a.digit0_counted is
// ignored: the first digit is always counted on the fly here.
template <int UNROLL = 4, int NT = kThreads, bool F16 = false, int HD = kHeadDim>
__device__ __forceinline__ int score_select(SelectArgs& a, int32_t* sel_lds) {
  // Nothing to choose (topk == 0) and nobody asked for the scores: stream nothing.
  const int n_score = (min(a.topk, a.n_cand) > 0 || a.scores_out) ? a.n_cand : 0;
  KIN_STAMP(17);  // prologue over: the stream of mean keys starts
  score_rows<UNROLL, NT, false, F16, true, HD>(a, 0, n_score, a.keys);
  a.digit0_counted = true;
  // the page-table copy (LDS-direct loads) has landed in every wave before anyone reads it
  KIN_STAMP(18);  // this wave has consumed its last mean key
  __builtin_amdgcn_s_waitcnt(0);
  KIN_STAMP(19);  // ... and have landed
  __syncthreads();
  return select_from_keys<NT>(a, sel_lds);
}

}  // namespace kin
