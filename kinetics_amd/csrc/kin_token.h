// Device-side building blocks of token-level top-k sparse decode attention for
// one (sequence, KV head), run by one workgroup of NW waves:
//
//   token_score_select()  streams every key of the sequence once (the K half of
//       each page, 16-byte loads straight to registers; the mean over the
//       group's heads of q_g . k_t is (mean_g q_g) . k_t, one fp32 dot product
//       per token), turns the score of every token of the "dynamic" part
//       (after the sink tokens, before the local window) into an
//       order-preserving 32-bit key in an HBM scratch array, radix-selects the
//       k-th largest key and compacts the winners, in ascending token order,
//       into a token list in LDS: sink tokens, winners, local-window tokens;
//   attend_tokens()       attention over such a list: the page loop of
//       attend_list() with one address per token row instead of one per page.
//
// HBM-bound on the key stream: 256 B per context token, plus 512 B per listed
// token; the scratch keys (4 B per token, re-read by the select passes) stay in
// the cache hierarchy for the most part.
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
  int32_t* list;         // LDS, >= n_sink + min(topk, n_dyn) + n_local entries
  int32_t* sel_tokens;   // HBM, the listed tokens' positions in the sequence, or null
};

// Physical token id (page * 16 + slot) of cache slot c of the sequence.
__device__ __forceinline__ int phys_token(const int32_t* table, int c) {
  return table[c >> 4] * kPageSize + (c & (kPageSize - 1));
}

// LDS scratch of the two functions below.
struct KeySelectShared {
  uint32_t hist[256];
  uint32_t wave_gt[16], wave_eq[16];
  uint32_t bin, remaining;
};

// Most-significant-digit-first radix select over n_keys (a multiple of 16) 32-bit
// keys in global memory, run by a workgroup of NW waves: finds the k-th largest
// non-zero key (zero keys are "not a candidate"; at least k keys are non-zero).
// thr receives it, remaining how many keys equal to thr belong to the k largest.
// first_digit_counted: sh->hist already holds the histogram of the top byte of
// the non-zero keys (counted while they were produced).  The keys are written by
// this workgroup; a barrier separates their last write from this call.
template <int NW>
__device__ __forceinline__ void radix_threshold(const uint32_t* keys, int n_keys, uint32_t k, bool first_digit_counted,
                                                KeySelectShared* sh, uint32_t& thr, uint32_t& remaining) {
  constexpr int NT = NW * 64;
  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63;
  uint32_t prefix = 0, mask = 0;
  remaining = k;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (shift != 24 || !first_digit_counted) {
      if (tid < 256) sh->hist[tid] = 0;
      __syncthreads();
      // 4 independent 16-byte loads per thread in flight: the keys come from L2 / HBM
      for (int base = tid * 4; base < n_keys; base += NT * 16) {
        uint4 kk[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = base + u * NT * 4;
          kk[u] = (i < n_keys) ? *reinterpret_cast<const uint4*>(keys + i) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t k4[4] = {kk[u].x, kk[u].y, kk[u].z, kk[u].w};
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (k4[j] && (k4[j] & mask) == prefix) atomicAdd(&sh->hist[(k4[j] >> shift) & 255u], 1u);
        }
      }
      __syncthreads();
    }
    if (w == 0) radix_pick_bin(sh->hist, remaining, l, &sh->bin, &sh->remaining);
    __syncthreads();
    prefix |= sh->bin << shift;
    mask |= 255u << shift;
    remaining = sh->remaining;
  }
  thr = prefix;  // >= 1
}

// Calls emit(pos, index) for every key above thr and for the `remaining` lowest-
// indexed keys equal to it, pos = 0, 1, ... in ascending index order.  Each wave
// owns a contiguous run of indices and walks it 256 at a time (4 consecutive keys
// per lane, two such loads in flight).  n_keys is a multiple of 16.
template <int NW, typename Emit>
__device__ __forceinline__ void compact_winners(const uint32_t* keys, int n_keys, uint32_t thr, uint32_t remaining,
                                                KeySelectShared* sh, Emit emit) {
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63;
  const int seg = ((n_keys + NW - 1) / NW + 255) & ~255;
  const int seg_lo = min(w * seg, n_keys), seg_hi = min(seg_lo + seg, n_keys);  // multiples of 16
  auto load4 = [&](int c) { return (c < seg_hi) ? *reinterpret_cast<const uint4*>(keys + c) : make_uint4(0u, 0u, 0u, 0u); };
  uint32_t gt = 0, eq = 0;
  for (int i = seg_lo; i < seg_hi; i += 1024) {
    uint4 kk[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) kk[u] = load4(i + u * 256 + 4 * l);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
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
  uint32_t run = 0, eq_run = 0;  // winners / threshold-equal keys in the runs before this wave's
  for (int wv = 0; wv < w; ++wv) {
    const uint32_t e = sh->wave_eq[wv];
    const uint32_t left = remaining > eq_run ? remaining - eq_run : 0u;
    run += sh->wave_gt[wv] + min(e, left);
    eq_run += e;
  }
  const unsigned long long below = (1ull << l) - 1ull;
  for (int i = seg_lo; i < seg_hi; i += 512) {
    uint4 kk[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) kk[u] = load4(i + u * 256 + 4 * l);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c0 = i + u * 256 + 4 * l;  // this lane's 4 consecutive indices
      const uint32_t k4[4] = {kk[u].x, kk[u].y, kk[u].z, kk[u].w};
      // Keys equal to the threshold are rare: rank them (lane-major, then j) only when there are any.
      bool is_eq[4];
      uint32_t eq_mine = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        is_eq[j] = k4[j] == thr;
        eq_mine += is_eq[j] ? 1u : 0u;
      }
      uint32_t eq_before = eq_run;  // equal keys at lower indices
      uint32_t eq_total = 0;
      if (__ballot(eq_mine != 0) != 0ull) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned long long be = __ballot(is_eq[j]);
          eq_before += __popcll(be & below);
          eq_total += __popcll(be);
        }
      }
      bool take[4];
      uint32_t mine_eq_seen = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        take[j] = k4[j] > thr || (is_eq[j] && eq_before + mine_eq_seen < remaining);
        mine_eq_seen += is_eq[j] ? 1u : 0u;
      }
      uint32_t pos = run, total = 0;  // winners at lower indices
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const unsigned long long bt = __ballot(take[j]);
        pos += __popcll(bt & below);
        total += __popcll(bt);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (take[j]) {
          emit((int)pos, c0 + j);
          ++pos;
        }
      }
      run += total;
      eq_run += eq_total;
    }
  }
}

// Streams the K plane of every page of the sequence once and calls
// emit(c, score) -- from one lane per key row -- with score = (mean_g q_g) . k_c
// in fp32 for every cache slot c of those pages (slots past the last token
// included).  16-byte loads straight to registers, kU of them in flight per
// lane; no LDS, no barrier.
template <int NW, typename Emit>
__device__ __forceinline__ void stream_token_scores(const TokenArgs& a, Emit emit) {
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, kg = l >> 4, c16 = l & 15;
  const int G = a.G;
  const int n_pages = a.n_pages;
  const int32_t* table = a.table;
  // The mean over the group's heads of q_g . k_t is (mean_g q_g) . k_t: one dot
  // product per token.  Lane owns columns d = 8*(lane%16) .. +7 of the mean query;
  // 16 lanes share a key row, a wave covers 4 rows, 4 waves one page.
  float qm[8];
  {
#pragma unroll
    for (int u = 0; u < 8; ++u) qm[u] = 0.f;
    const uint16_t* qp = a.q_bh + 8 * c16;
    for (int g = 0; g < G; ++g) {
      const uint4 x = *reinterpret_cast<const uint4*>(qp + (int64_t)g * kHeadDim);
      qm[0] += bf16_lo(x.x); qm[1] += bf16_hi(x.x);
      qm[2] += bf16_lo(x.y); qm[3] += bf16_hi(x.y);
      qm[4] += bf16_lo(x.z); qm[5] += bf16_hi(x.z);
      qm[6] += bf16_lo(x.w); qm[7] += bf16_hi(x.w);
    }
    const float inv = 1.0f / (float)G;
#pragma unroll
    for (int u = 0; u < 8; ++u) qm[u] *= inv;
  }
  constexpr int kPP = NW / 4;   // pages one pass of the workgroup covers
  constexpr int kU = 16;        // passes (16-byte loads per lane) kept in flight
  const __attribute__((address_space(4))) int32_t* tab_c =
      reinterpret_cast<const __attribute__((address_space(4))) int32_t*>(reinterpret_cast<uintptr_t>(table));
  const int row = 4 * (w & 3) + kg;                 // key row of the page this lane helps with
  const int voff = row * a.row_bytes + c16 * 16;
  const int k_span = kPageSize * a.row_bytes - (a.span < a.page_bytes ? a.page_bytes - a.span : 0);  // K plane only
  auto load_page = [&](int p) -> u32x4 {
    // Pages past the end (or with an id outside the cache) are read through an
    // empty descriptor: zeros, no memory traffic.
    const bool in = p < n_pages;
    const int id = tab_c[in ? p : 0];
    const bool ok = in && id >= 0 && (int64_t)id < a.num_pages;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(a.kvb + (int64_t)(ok ? id : 0) * a.page_bytes, ok ? k_span : 0);
    return __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, kStreamLoad);
  };
  const int p_first = w >> 2;  // this wave's page within a pass
  u32x4 x[kU];
#pragma unroll
  for (int u = 0; u < kU; ++u) x[u] = load_page(p_first + u * kPP);
  for (int base = 0; base < n_pages; base += kU * kPP) {
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const u32x4 kx = x[u];
      const int p = base + u * kPP + p_first;
      x[u] = load_page(p + kU * kPP);
      float acc = 0.f;
      acc = fmaf(qm[0], bf16_lo(kx.x), acc); acc = fmaf(qm[1], bf16_hi(kx.x), acc);
      acc = fmaf(qm[2], bf16_lo(kx.y), acc); acc = fmaf(qm[3], bf16_hi(kx.y), acc);
      acc = fmaf(qm[4], bf16_lo(kx.z), acc); acc = fmaf(qm[5], bf16_hi(kx.z), acc);
      acc = fmaf(qm[6], bf16_lo(kx.w), acc); acc = fmaf(qm[7], bf16_hi(kx.w), acc);
      acc = row16_sum(acc);
      const int c = p * kPageSize + row;
      if (c16 == 0 && p < n_pages) emit(c, acc);
    }
  }
}

// Token-level top-k: writes the token list (physical token ids) to a.list and
// returns its length.  Every thread of the workgroup calls this; it ends with a
// workgroup barrier.
template <int NG, int NW>
__device__ __forceinline__ int token_score_select(const TokenArgs& a) {
  constexpr int NT = NW * 64;
  __shared__ KeySelectShared sh_store;
  KeySelectShared* sh = &sh_store;
  uint32_t* hist = sh->hist;

  const int tid = threadIdx.x;
  const int n_pages = a.n_pages;
  const int k_eff = min(a.topk, a.n_dyn);
  const int dyn_lo = a.pad + a.n_sink, dyn_hi = dyn_lo + a.n_dyn;  // cache slots of the candidates
  const int n_keys = n_pages * kPageSize;
  int32_t* list = a.list;
  const int32_t* table = a.table;

  if (k_eff > 0 && k_eff < a.n_dyn) {
    // ---- phase 1: group-mean logit of every token -> keys[], first radix digit counted on the fly
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    stream_token_scores<NW>(a, [&](int c, float score) {
      // 0 marks "not a candidate" (order_key is never 0 for a finite score)
      const uint32_t key = (c >= dyn_lo && c < dyn_hi) ? order_key(score) : 0u;
      a.keys[c] = key;
      if (key) atomicAdd(&hist[key >> 24], 1u);
    });
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // keys[] and hist[] complete and visible to the whole workgroup

    // ---- phases 2 and 3: threshold, then the winners in ascending token order ----
    uint32_t thr, remaining;
    radix_threshold<NW>(a.keys, n_keys, (uint32_t)k_eff, true, sh, thr, remaining);
    compact_winners<NW>(a.keys, n_keys, thr, remaining, sh, [&](int pos, int c) {
      list[a.n_sink + pos] = phys_token(table, c);
      if (a.sel_tokens) a.sel_tokens[a.n_sink + pos] = c - a.pad;
    });
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
  float* scores;         // HBM scratch, n_pages * 16 entries
  uint32_t* block_keys;  // HBM scratch, >= n_pages * 16 entries, 16-byte aligned
  uint32_t* bitmap;      // LDS, one bit per candidate token: (n_dyn + 31) / 32 words
};

// Strided overlapping-block top-k: block i covers the candidate tokens
// [i*stride, i*stride + block); the min(2*topk_blocks, num_blocks) blocks with the
// largest mean score are chosen, their tokens united, and the topk_blocks*block
// lowest-positioned of those kept.  With fewer candidates than one block every
// token is listed.  Writes the token list to a.list (sink tokens, kept tokens in
// ascending order, local tokens) and returns its length; ends with a barrier.
template <int NG, int NW>
__device__ __forceinline__ int strided_score_select(const TokenArgs& a, const StridedArgs& sa) {
  constexpr int NT = NW * 64;
  __shared__ KeySelectShared sh_store;
  __shared__ uint32_t wave_cnt[NW];
  KeySelectShared* sh = &sh_store;
  uint32_t* hist = sh->hist;

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
    // ---- token scores -> HBM ------------------------------------------------
    stream_token_scores<NW>(a, [&](int c, float score) { sa.scores[c] = score; });
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    // ---- block means -> keys (padded with "no candidate" to a multiple of 16) --
    const int nb_pad = (num_blocks + 15) & ~15;
    const float inv = 1.0f / (float)sa.block;
    for (int i = tid; i < nb_pad; i += NT) {
      uint32_t key = 0u;
      if (i < num_blocks) {
        const float* sp = sa.scores + dyn_lo + i * sa.stride;
        float sum = 0.f;
        for (int t = 0; t < sa.block; ++t) sum += sp[t];
        key = order_key(sum * inv);
        atomicAdd(&hist[key >> 24], 1u);
      }
      sa.block_keys[i] = key;
    }
    __builtin_amdgcn_s_waitcnt(0);
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
      uint32_t thr, remaining;
      radix_threshold<NW>(sa.block_keys, nb_pad, (uint32_t)k_blocks, true, sh, thr, remaining);
      compact_winners<NW>(sa.block_keys, nb_pad, thr, remaining, sh, [&](int, int i) { mark_block(i); });
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
        list[a.n_sink + pos] = phys_token(table, dyn_lo + t);
        if (a.sel_tokens) a.sel_tokens[a.n_sink + pos] = a.n_sink + t;
        ++pos;
      }
    }
    kept = (int)min(total, (uint32_t)budget);
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
template <int NG, int NW, typename Emit>
__device__ __forceinline__ void attend_tokens(const AttendArgs& a, const int32_t* list, unsigned char* lds,
                                              float (*sm_m)[4 * NG], float (*sm_l)[4 * NG], Emit emit) {
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, kg = l >> 4, c16 = l & 15, gq = l & 3;
  const int G = a.G;
  const int n = a.n;

  bf16x8 qB[NG][4];
#pragma unroll
  for (int half = 0; half < NG; ++half) {
    const int g = min(4 * half + gq, G - 1);
    const uint16_t* qp = a.q_bh + (int64_t)g * kHeadDim + 8 * kg;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      qB[half][c] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(qp + 32 * c));
  }

  const int row_bytes = a.row_bytes;
  const int page_bytes = a.page_bytes;
  const char* kvb = a.kvb;
  const int64_t max_tok = a.num_pages * kPageSize;
  unsigned char* kl = lds + w * (2 * 4096);
  int kchunk[4], lds_r[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int row = 4 * c + kg;                       // K row this lane helps to fetch with load c
    kchunk[c] = ((c16 ^ row) & 15) * 16;              // the chunk that belongs at its LDS position
    lds_r[c] = c16 * 256 + (((4 * c + kg) ^ c16) & 15) * 16;
  }
  const int vchunk = kPageSize * row_bytes + c16 * 16;  // V plane of the page, this lane's columns

  float m_run[NG], l_run[NG];
  floatx4 O[NG][8];
#pragma unroll
  for (int half = 0; half < NG; ++half) {
    m_run[half] = kNegInf;
    l_run[half] = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) O[half][u] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // This wave takes the 16-entry groups w, w+NW, ...  Entries past the end (and
  // ids outside the cache) read token 0 of the cache and are masked.
  const int groups = (n + kPageSize - 1) / kPageSize;
  const int iters = (groups > w) ? (groups - w + NW - 1) / NW : 0;
  auto row_ptr = [&](int tok) -> const char* {
    const bool ok = tok >= 0 && (int64_t)tok < max_tok;
    const int t = ok ? tok : 0;
    return kvb + (int64_t)(t >> 4) * page_bytes + (t & (kPageSize - 1)) * row_bytes;
  };
  struct Ids { int k[4], v[4], valid; };
  auto fetch_ids = [&](int it) {
    Ids ids;
    const int base = (w + NW * it) * kPageSize;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e = base + 4 * c + kg;
      ids.k[c] = (e < n) ? list[e] : -1;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = base + 4 * kg + r;
      ids.v[r] = (e < n) ? list[e] : -1;
    }
    ids.valid = max(0, min(kPageSize, n - base));
    return ids;
  };
  auto issue_v = [&](const Ids& ids, u32x4 (&vv)[4]) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      vv[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row_ptr(ids.v[r]) + vchunk));
  };
  auto issue_k = [&](const Ids& ids, int stage) {
    __attribute__((address_space(3))) unsigned char* dst =
        (__attribute__((address_space(3))) unsigned char*)(kl + stage * 4096);
#pragma unroll
    for (int c = 0; c < 4; ++c)
      __builtin_amdgcn_global_load_lds(
          reinterpret_cast<const __attribute__((address_space(1))) void*>(
              reinterpret_cast<uintptr_t>(row_ptr(ids.k[c]) + kchunk[c])),
          dst + c * 1024, 16, 0, kStreamLoad);
  };
  auto read_k = [&](int stage, uint4 (&ka)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) ka[c] = *reinterpret_cast<const uint4*>(kl + stage * 4096 + lds_r[c]);
  };

  // Same explicit wait as in attend_list(): when it executes, exactly the 4 V
  // loads issued just before it may be outstanding.
  if (iters > 0) {
    u32x4 vA[4], vB[4];
    uint4 ka[4];
    float pr[NG][4];
    Ids idA = fetch_ids(0), idB;
    issue_k(idA, 0);
    issue_v(idA, vA);
    for (int it = 0; it < iters; it += 2) {
      {
        idB = fetch_ids(it + 1);
        __builtin_amdgcn_sched_barrier(0);
        issue_v(idB, vB);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitVm4);
        __builtin_amdgcn_sched_barrier(0);
        read_k(0, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(idB, 1);
        __builtin_amdgcn_sched_barrier(0);
        page_scores<NG>(ka, qB, m_run, l_run, O, pr, a.scale_log2, 0, idA.valid, kg);
        if (idA.valid != kPageSize) clear_unused_v_rows(vA, 0, idA.valid, kg);
        page_pv<NG>(vA, pr, O);
      }
      {
        idA = fetch_ids(it + 2);
        __builtin_amdgcn_sched_barrier(0);
        issue_v(idA, vA);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitVm4);
        __builtin_amdgcn_sched_barrier(0);
        read_k(1, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(idA, 0);
        __builtin_amdgcn_sched_barrier(0);
        page_scores<NG>(ka, qB, m_run, l_run, O, pr, a.scale_log2, 0, idB.valid, kg);
        if (idB.valid != kPageSize) clear_unused_v_rows(vB, 0, idB.valid, kg);
        page_pv<NG>(vB, pr, O);
      }
    }
  }
  attend_finish<NG, NW>(m_run, l_run, O, G, lds, sm_m, sm_l, emit);
}

}  // namespace kin
