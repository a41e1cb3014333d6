// Paged gather-attention for one decode token per sequence (sparse page lists
// from the selector, or the full page table for the dense baseline).
//
// Work decomposition: one 256-thread workgroup per (sequence, KV head, split);
// its 4 waves take the list's pages round-robin, one 8 KiB page (16 keys +
// 16 values of 128 bf16) per wave per iteration, and keep private online-softmax
// state that is merged once at the end (wave -> workgroup -> optional split-K
// merge kernel).  HBM-bound: every K/V byte is read exactly once.
//
// Per page and wave (lane l, row group kg = l/16, 16-byte column chunk c = l%16):
//   K  4 x 16-byte loads, each instruction covering 4 whole 256-byte rows;
//      staged through wave-private LDS (XOR-swizzled 16-byte chunks) to turn
//      "row = l/16" into the MFMA operand layout "row = l%16".
//   S  = K q^T with 4 x v_mfma_f32_16x16x32_bf16; the 16 output columns hold
//      the (<=4) query heads of the group replicated 4x, so lane l ends up with
//      S[g = l%4][t = 4*kg + r] (r = 0..3) and no cross-lane traffic is needed.
//   softmax state (m, l) is kept per (row group, head): 4 independent partial
//      softmaxes per wave, so the running max needs no cross-lane reduction.
//   V  4 x 16-byte loads straight into registers: load r fetches row 4*kg + r.
//   O += P V with v_mfma_f32_4x4x1_16B_f32 (16 independent 4x4 outer products):
//      block = 4 lanes = one token row, A = p[g][t] (lane%4 = g), B = V[t][d]
//      (d = 8*c + u), so values feed the matrix unit in the layout they were
//      loaded in; P and V stay fp32.
// Query groups larger than 4 run NG = 2 passes of the S / PV tiles per page.
#include <cmath>

#include "kin_common.h"

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
  int num_q_heads, num_kv_heads, group;
  int list_stride, num_splits;
  int64_t num_pages;
  float scale_log2;  // sm_scale * log2(e)
};

// s_waitcnt immediate for "vmcnt <= 4, no wait on expcnt / lgkmcnt" (gfx9 encoding:
// vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]).
constexpr int kWaitVm4 = 4 | (7 << 4) | (15 << 8);

constexpr float kNegInf = -INFINITY;
constexpr float kLn2 = 0.6931471805599453f;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Buffer descriptor covering `bytes` bytes from `base` (0 bytes: every load
// through it returns zeros without touching memory).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// One page for one wave, first half: scores and the online softmax update.
// ka: this lane's 4 K chunks in MFMA A layout.  Leaves the probabilities of
// this lane's 4 tokens in pr.
template <int NG>
__device__ __forceinline__ void page_scores(const uint4 (&ka)[4], const bf16x8 (&qB)[NG][4], float (&m_run)[NG],
                                            float (&l_run)[NG], floatx4 (&O)[NG][8], float (&pr)[NG][4],
                                            float scale_log2, int valid_tokens, int kg) {
  floatx4 S[NG];
#pragma unroll
  for (int half = 0; half < NG; ++half) S[half] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const bf16x8 a = __builtin_bit_cast(bf16x8, ka[c]);
#pragma unroll
    for (int half = 0; half < NG; ++half)
      S[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qB[half][c], S[half], 0, 0, 0);
  }
#pragma unroll
  for (int half = 0; half < NG; ++half) {
    float s[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) s[r] = (4 * kg + r < valid_tokens) ? S[half][r] * scale_log2 : kNegInf;
    const float m_new = fmaxf(m_run[half], fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
    if (__any(m_new > m_run[half])) {
      const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
      const float alpha = fast_exp2(m_run[half] - m_safe);
      l_run[half] *= alpha;
      const float a0 = quad_bcast<0>(alpha), a1 = quad_bcast<1>(alpha);
      const float a2 = quad_bcast<2>(alpha), a3 = quad_bcast<3>(alpha);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        O[half][u][0] *= a0;
        O[half][u][1] *= a1;
        O[half][u][2] *= a2;
        O[half][u][3] *= a3;
      }
      m_run[half] = m_new;
    }
    const float m_use = (m_run[half] == kNegInf) ? 0.f : m_run[half];
#pragma unroll
    for (int r = 0; r < 4; ++r) pr[half][r] = fast_exp2(s[r] - m_use);
    l_run[half] += (pr[half][0] + pr[half][1]) + (pr[half][2] + pr[half][3]);
  }
}

// Second half: O += P V.  vr: this lane's 4 V rows (row 4*kg + r).
template <int NG>
__device__ __forceinline__ void page_pv(const u32x4 (&vr)[4], const float (&pr)[NG][4], floatx4 (&O)[NG][8]) {
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const u32x4 vv = vr[r];
    const float vf[8] = {bf16_lo(vv.x), bf16_hi(vv.x), bf16_lo(vv.y), bf16_hi(vv.y),
                         bf16_lo(vv.z), bf16_hi(vv.z), bf16_lo(vv.w), bf16_hi(vv.w)};
#pragma unroll
    for (int u = 0; u < 8; ++u) {
#pragma unroll
      for (int half = 0; half < NG; ++half)
        O[half][u] = __builtin_amdgcn_mfma_f32_4x4x1f32(pr[half][r], vf[u], O[half][u], 0, 0, 0);
    }
  }
}

template <int NG>
__global__ __launch_bounds__(256, 2) void paged_decode_kernel(DecodeParams p) {
  // 2 x 4 KiB of K staging per wave; reused as the [wave][head][128] merge buffer.
  __shared__ __attribute__((aligned(16))) unsigned char lds[32768];
  __shared__ float sm_m[4][4 * NG];
  __shared__ float sm_l[4][4 * NG];

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, kg = l >> 4, c16 = l & 15, gq = l & 3;
  const int list = blockIdx.x, split = blockIdx.y;
  const int b = list / p.num_kv_heads, h = list - b * p.num_kv_heads;
  const int G = p.group;

  const int32_t* __restrict__ pl;
  int n;
  if (p.list_indptr) {
    const int s = p.list_indptr[b];
    pl = p.page_ids + s;
    n = p.list_indptr[b + 1] - s;
  } else {
    pl = p.page_ids + (int64_t)list * p.list_stride;
    n = p.list_count[list];
  }
  n = max(n, 0);
  const int last_len = p.last_page_len[b];
  const int per_split = (n + p.num_splits - 1) / p.num_splits;
  const int p0 = min(split * per_split, n), p1 = min(n, p0 + per_split);

  // Query operands: B[k][j], j = l%16 -> head 4*half + l%4, k-chunk = l/16.
  bf16x8 qB[NG][4];
#pragma unroll
  for (int half = 0; half < NG; ++half) {
    const int g = min(4 * half + gq, G - 1);
    const uint16_t* qp = p.q + ((int64_t)b * p.num_q_heads + (int64_t)h * G + g) * kHeadDim + 8 * kg;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      qB[half][c] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(qp + 32 * c));
  }

  const int row_bytes = p.num_kv_heads * kRowBytes;
  const int page_bytes = 2 * kPageSize * row_bytes;
  const int span = page_bytes - h * kRowBytes;  // bytes addressable from this head's first row
  const char* kvb = reinterpret_cast<const char*>(p.kv) + (int64_t)h * kRowBytes;
  int voff[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) voff[c] = (kPageSize + 4 * kg + c) * row_bytes + c16 * 16;
  // K staging: two 4 KiB stages per wave, filled by LDS-direct buffer loads
  // (no VGPRs while in flight).  Load c brings rows 4c..4c+3: lane (kg, c16)
  // lands at LDS row 4c+kg, position c16, and fetches the chunk that belongs
  // there under the XOR swizzle (position p of row R holds chunk p ^ R).
  unsigned char* kl = lds + w * (2 * 4096);
  int kdma_off[4], lds_r[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int row = 4 * c + kg;
    kdma_off[c] = row * row_bytes + ((c16 ^ row) & 15) * 16;
    const int chunk_r = 4 * c + kg;  // chunk of row c16 that MFMA c wants from this lane
    lds_r[c] = c16 * 256 + ((chunk_r ^ c16) & 15) * 16;
  }

  float m_run[NG], l_run[NG];
  floatx4 O[NG][8];
#pragma unroll
  for (int half = 0; half < NG; ++half) {
    m_run[half] = kNegInf;
    l_run[half] = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) O[half][u] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // This wave takes list entries my_first, my_first+4, ...  The loop below is
  // branch-free: a page past the end (or with an id outside the cache) is read
  // through an empty buffer descriptor -- zeros, no memory traffic -- and all
  // of its tokens are masked.
  const int my_first = p0 + w;
  const int iters = (p1 > my_first) ? (p1 - my_first + 3) / 4 : 0;
  const int n_last = n - 1;
  // Page ids come through scalar loads issued one half-step before they are
  // needed.  The list is read-only for the whole kernel; the constant address
  // space makes the uniform load a scalar one (off the vector-memory counter
  // that the page prefetch relies on).
  const __attribute__((address_space(4))) int32_t* pl_c =
      reinterpret_cast<const __attribute__((address_space(4))) int32_t*>(reinterpret_cast<uintptr_t>(pl));
  auto load_id = [&](int it) -> int {
    const int idx = my_first + 4 * it;
    return pl_c[idx < p1 ? idx : 0];
  };
  auto page_rsrc = [&](int it, int id, int& valid_tokens) {
    const int idx = my_first + 4 * it;
    const bool ok = idx < p1 && id >= 0 && (int64_t)id < p.num_pages;
    valid_tokens = ok ? (idx == n_last ? last_len : kPageSize) : 0;
    return make_rsrc(kvb + (int64_t)(ok ? id : 0) * page_bytes, ok ? span : 0);
  };
  auto issue_v = [&](__amdgpu_buffer_rsrc_t r, u32x4 (&vv)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) vv[c] = __builtin_amdgcn_raw_buffer_load_b128(r, voff[c], 0, kStreamLoad);
  };
  auto issue_k = [&](__amdgpu_buffer_rsrc_t r, int stage) {
    __attribute__((address_space(3))) unsigned char* dst =
        (__attribute__((address_space(3))) unsigned char*)(kl + stage * 4096);
#pragma unroll
    for (int c = 0; c < 4; ++c)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, dst + c * 1024, 16, kdma_off[c], 0, 0, kStreamLoad);
  };
  auto read_k = [&](int stage, uint4 (&ka)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) ka[c] = *reinterpret_cast<const uint4*>(kl + stage * 4096 + lds_r[c]);
  };

  // The compiler does not order LDS reads after LDS-direct loads by itself, so
  // the wait is explicit: when it executes, exactly the 4 V loads issued just
  // before it are allowed to be outstanding, which means the K stage about to
  // be read (and the V registers about to be used) have landed.  The scheduling
  // fences keep the instruction order this count relies on.
  if (iters > 0 && n > 0) {
    u32x4 vA[4], vB[4];
    uint4 ka[4];
    float pr[NG][4];
    int validA, validB;
    {
      const __amdgpu_buffer_rsrc_t r0 = page_rsrc(0, load_id(0), validA);
      issue_k(r0, 0);
      issue_v(r0, vA);
    }
    int id_next = load_id(1);
    for (int it = 0; it < iters; it += 2) {
      {
        const __amdgpu_buffer_rsrc_t r1 = page_rsrc(it + 1, id_next, validB);
        __builtin_amdgcn_sched_barrier(0);
        issue_v(r1, vB);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitVm4);
        __builtin_amdgcn_sched_barrier(0);
        read_k(0, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(r1, 1);
        __builtin_amdgcn_sched_barrier(0);
        page_scores<NG>(ka, qB, m_run, l_run, O, pr, p.scale_log2, validA, kg);
        __builtin_amdgcn_sched_barrier(0);
        id_next = load_id(it + 2);  // lands while the P V products run
        page_pv<NG>(vA, pr, O);
      }
      {
        const __amdgpu_buffer_rsrc_t r2 = page_rsrc(it + 2, id_next, validA);
        __builtin_amdgcn_sched_barrier(0);
        issue_v(r2, vA);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitVm4);
        __builtin_amdgcn_sched_barrier(0);
        read_k(1, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(r2, 0);
        __builtin_amdgcn_sched_barrier(0);
        page_scores<NG>(ka, qB, m_run, l_run, O, pr, p.scale_log2, validB, kg);
        __builtin_amdgcn_sched_barrier(0);
        id_next = load_id(it + 3);
        page_pv<NG>(vB, pr, O);
      }
    }
  }
  // LDS-direct loads that are still in flight (masked tail pages) must land
  // before the staging area is reused below.
  __builtin_amdgcn_s_waitcnt(0);

  // ---- merge the 4 row groups of the wave (lanes l, l^16, l^32, l^48) --------
  float m_w[NG], l_w[NG];
#pragma unroll
  for (int half = 0; half < NG; ++half) {
    float mm = m_run[half];
    mm = fmaxf(mm, __shfl_xor(mm, 16));
    mm = fmaxf(mm, __shfl_xor(mm, 32));
    const float m_safe = (mm == kNegInf) ? 0.f : mm;
    const float sc = fast_exp2(m_run[half] - m_safe);
    float ll = l_run[half] * sc;
    ll += __shfl_xor(ll, 16);
    ll += __shfl_xor(ll, 32);
    m_w[half] = mm;
    l_w[half] = ll;
    const float s0 = quad_bcast<0>(sc), s1 = quad_bcast<1>(sc), s2 = quad_bcast<2>(sc), s3 = quad_bcast<3>(sc);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      float x0 = O[half][u][0] * s0, x1 = O[half][u][1] * s1, x2 = O[half][u][2] * s2, x3 = O[half][u][3] * s3;
      x0 += __shfl_xor(x0, 16); x1 += __shfl_xor(x1, 16); x2 += __shfl_xor(x2, 16); x3 += __shfl_xor(x3, 16);
      x0 += __shfl_xor(x0, 32); x1 += __shfl_xor(x1, 32); x2 += __shfl_xor(x2, 32); x3 += __shfl_xor(x3, 32);
      O[half][u] = floatx4{x0, x1, x2, x3};
    }
  }
  __syncthreads();  // every wave is done with its K staging area
  float* ow = reinterpret_cast<float*>(lds);  // [4 waves][4*NG heads][128]
  if (kg == 0) {
#pragma unroll
    for (int half = 0; half < NG; ++half) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float* dst = ow + ((w * 4 * NG + 4 * half + i) * kHeadDim + 8 * c16);
        *reinterpret_cast<float4*>(dst) = make_float4(O[half][0][i], O[half][1][i], O[half][2][i], O[half][3][i]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(O[half][4][i], O[half][5][i], O[half][6][i], O[half][7][i]);
      }
      if (l < 4) {
        sm_m[w][4 * half + l] = m_w[half];
        sm_l[w][4 * half + l] = l_w[half];
      }
    }
  }
  __syncthreads();

  // ---- merge the 4 waves and write out -----------------------------------------
#pragma unroll
  for (int j = 0; j < 2 * NG; ++j) {
    const int idx = tid + 256 * j;
    const int g = idx >> 7, d = idx & 127;
    if (g < G) {
      float mm = fmaxf(fmaxf(sm_m[0][g], sm_m[1][g]), fmaxf(sm_m[2][g], sm_m[3][g]));
      const float m_safe = (mm == kNegInf) ? 0.f : mm;
      float num = 0.f, den = 0.f;
#pragma unroll
      for (int wv = 0; wv < 4; ++wv) {
        const float sc = fast_exp2(sm_m[wv][g] - m_safe);
        num += ow[(wv * 4 * NG + g) * kHeadDim + d] * sc;
        den += sm_l[wv][g] * sc;
      }
      const float o = (den > 0.f) ? num / den : 0.f;
      const float lse2 = (den > 0.f) ? mm + fast_log2(den) : kNegInf;
      const int64_t hq = (int64_t)b * p.num_q_heads + (int64_t)h * G + g;
      if (p.num_splits == 1) {
        p.out[hq * kHeadDim + d] = (uint16_t)f32_to_bf16(o);
        if (p.lse && d == 0) p.lse[hq] = lse2 * kLn2;
      } else {
        p.ws_o[(hq * p.num_splits + split) * kHeadDim + d] = o;
        if (d == 0) p.ws_lse[hq * p.num_splits + split] = lse2;
      }
    }
  }
}

// Split-K merge: one 128-thread block per (sequence, query head).
__global__ __launch_bounds__(128) void merge_splits_kernel(const float* __restrict__ ws_o,
                                                           const float* __restrict__ ws_lse,
                                                           uint16_t* __restrict__ out, float* __restrict__ lse,
                                                           int num_splits) {
  const int64_t hq = blockIdx.x;
  const int d = threadIdx.x;
  const float* l2 = ws_lse + hq * num_splits;
  float mm = kNegInf;
  for (int s = 0; s < num_splits; ++s) mm = fmaxf(mm, l2[s]);
  const float m_safe = (mm == kNegInf) ? 0.f : mm;
  float num = 0.f, den = 0.f;
  for (int s = 0; s < num_splits; ++s) {
    const float wgt = fast_exp2(l2[s] - m_safe);
    num += ws_o[(hq * num_splits + s) * kHeadDim + d] * wgt;
    den += wgt;
  }
  out[hq * kHeadDim + d] = (uint16_t)f32_to_bf16(den > 0.f ? num / den : 0.f);
  if (lse && d == 0) lse[hq] = (den > 0.f) ? (mm + fast_log2(den)) * kLn2 : kNegInf;
}

static int auto_splits(int batch, int num_kv_heads, int max_pages_per_list) {
  // Aim for >= 4 workgroups per CU (256 CUs) without cutting lists below 4
  // pages (one per wave) per split.
  const int64_t lists = (int64_t)batch * num_kv_heads;
  if (lists <= 0) return 1;
  const int64_t target = 1024;
  if (lists >= target) return 1;
  int64_t want = (target + lists - 1) / lists;
  int64_t cap = max_pages_per_list / 4;
  if (cap < 1) cap = 1;
  if (want > cap) want = cap;
  if (want > 64) want = 64;
  return (int)want;
}

static size_t workspace_bytes_for(int batch, int num_q_heads, int splits) {
  if (splits <= 1) return 0;
  return (size_t)batch * num_q_heads * splits * (kHeadDim + 1) * sizeof(float);
}

static int launch_decode(const char* fn, DecodeParams& p, int batch, void* workspace, size_t workspace_bytes,
                         int max_pages_per_list, int num_splits, hipStream_t stream) {
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
    p.ws_lse = p.ws_o + (size_t)batch * p.num_q_heads * splits * kHeadDim;
  } else {
    p.ws_o = nullptr;
    p.ws_lse = nullptr;
  }
  const int64_t lists = (int64_t)batch * p.num_kv_heads;
  if (lists > 0x7fffffffLL) return fail(KIN_ERR_UNSUPPORTED, "%s: batch*num_kv_heads too large", fn);
  dim3 grid((unsigned)lists, (unsigned)splits);
  if (p.group <= 4)
    paged_decode_kernel<1><<<grid, 256, 0, stream>>>(p);
  else
    paged_decode_kernel<2><<<grid, 256, 0, stream>>>(p);
  int st = check_hip(hipGetLastError(), "paged_decode_kernel launch");
  if (st) return st;
  if (splits > 1) {
    merge_splits_kernel<<<(unsigned)((int64_t)batch * p.num_q_heads), 128, 0, stream>>>(p.ws_o, p.ws_lse, p.out,
                                                                                         p.lse, splits);
    st = check_hip(hipGetLastError(), "merge_splits_kernel launch");
  }
  return st;
}

static int check_decode_args(const char* fn, const void* q, const void* kv_cache, const void* last_page_len,
                             const void* out, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                             int page_size, int64_t num_pages, int num_splits) {
  if (!q || !kv_cache || !last_page_len || !out) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_common_dims(fn, batch, num_q_heads, num_kv_heads, head_dim, page_size);
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

int kin_sparse_paged_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache, const int32_t* sel_pages,
                            const int32_t* sel_count, const int32_t* last_page_len, kin_bf16_t* out, float* lse,
                            void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                            int head_dim, int page_size, int64_t num_pages, int sel_stride, float sm_scale,
                            int num_splits, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_sparse_paged_decode";
  if (!sel_pages || !sel_count) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_decode_args(fn, q, kv_cache, last_page_len, out, batch, num_q_heads, num_kv_heads, head_dim,
                             page_size, num_pages, num_splits);
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
  const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim);
  p.scale_log2 = scale * 1.4426950408889634f;
  return launch_decode(fn, p, batch, workspace, workspace_bytes, sel_stride, num_splits,
                       static_cast<hipStream_t>(stream));
}

int kin_dense_paged_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache, const int32_t* page_indices,
                           const int32_t* page_indptr, const int32_t* last_page_len, kin_bf16_t* out, float* lse,
                           void* workspace, size_t workspace_bytes, int batch, int num_q_heads, int num_kv_heads,
                           int head_dim, int page_size, int64_t num_pages, int max_pages_per_seq, float sm_scale,
                           int num_splits, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_dense_paged_decode";
  if (!page_indices || !page_indptr) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  int st = check_decode_args(fn, q, kv_cache, last_page_len, out, batch, num_q_heads, num_kv_heads, head_dim,
                             page_size, num_pages, num_splits);
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
  const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim);
  p.scale_log2 = scale * 1.4426950408889634f;
  return launch_decode(fn, p, batch, workspace, workspace_bytes, max_pages_per_seq, num_splits,
                       static_cast<hipStream_t>(stream));
}

}  // extern "C"
