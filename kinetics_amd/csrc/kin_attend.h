// Device-side building block: attention of one decode token over a list of
// KV pages, for one (sequence, KV head, split) handled by one workgroup of NW
// waves (4 in the stand-alone kernel; the fused step uses up to 16 when few
// lists have to fill the GPU).  Shared by the stand-alone paged decode kernel and the fused
// decode-step kernel.
//
// Work decomposition: the workgroup's NW waves take the list's tiles round-robin,
// one tile (16 keys + 16 values of 128 bf16: 8 KiB) per wave per iteration, and
// keep private online-softmax state that is merged once at the end.  A page of
// 16 tokens is one tile; pages of 32 or 64 tokens are 2 or 4 tiles, each a run of
// 16 rows of the page's K plane and the matching 16 rows of its V plane.
//
// Per page and wave (lane l, row group kg = l/16, 16-byte column chunk c = l%16):
//   K  4 x 16-byte LDS-direct buffer loads, each instruction covering 4 whole
//      256-byte rows, into a wave-private, XOR-swizzled staging area (two
//      stages); read back in the MFMA operand layout "row = l%16".
//   S  = K q^T with 4 x v_mfma_f32_16x16x32_bf16 (_f16 for half caches); the 16 output columns hold
//      the (<=4) query heads of the group replicated 4x, so lane l ends up with
//      S[g = l%4][t = 4*kg + r] (r = 0..3) and no cross-lane traffic is needed.
//   softmax state (m, l) is kept per (row group, head): 4 independent partial
//      softmaxes per wave, so the running max needs no cross-lane reduction.
//   V  4 x 16-byte buffer loads straight into registers: load r fetches row 4*kg + r.
//   O += P V with v_mfma_f32_4x4x1_16B_f32 (16 independent 4x4 outer products):
//      block = 4 lanes = one token row, A = p[g][t] (lane%4 = g), B = V[t][d]
//      (d = 8*c + u), so values feed the matrix unit in the layout they were
//      loaded in; P and V stay fp32.
// Query groups larger than 4 run the "wide" form NG = 4 (up to 16 heads, see
// page_scores_wide): the 16 columns of the S tile are 16 different heads and O += P V
// runs on v_mfma_f32_16x16x4_f32, whose K dimension adds the wave's four row groups up
// inside the matrix unit (same registers per lane as the narrow form, four times the
// matrix cycles).
//
// Head rows of 64 elements (HD = 64, 128 bytes): a tile is 2 KiB of keys and 2 KiB of values.  K arrives in
// 2 LDS-direct loads of 8 rows each and S takes 2 matrix instructions.  In the narrow form a lane fetches
// 2 V rows -- the 16 lanes of a row group split into two halves of 8 chunks, the lower half taking tokens
// 4*kg + 0..1 and the upper half 4*kg + 2..3 -- and the two halves' partial outputs are added at the end;
// the wide form keeps 4 V rows per lane with both halves fetching the same chunks (its P V instruction
// shares one probability between all 16 columns) and lets the halves take the even and the odd elements
// of a chunk (see page_pv_wide).
#pragma once

#include <cmath>

#include "kin_common.h"

namespace kin {

// s_waitcnt immediate for "vmcnt <= n (n < 16), no wait on expcnt / lgkmcnt" (gfx9 encoding:
// vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]).
constexpr int wait_vm_imm(int n) { return n | (7 << 4) | (15 << 8); }

// XOR swizzle of the K staging area: position p of row R holds the row's 16-byte chunk p ^ attend_swizzle(R),
// so that the 16 lanes that read one chunk column of 16 different rows hit different banks.  Rows of
// 256 bytes: R itself; rows of 128 bytes (two rows per 64 banks): rows 8..15 get the odd patterns.
template <int HD>
__device__ __forceinline__ int attend_swizzle(int row) {
  if constexpr (HD == 128) return row & 15;
  else return (row ^ (row >> 3)) & 7;
}
// V rows a lane fetches per tile: 4, or 2 in the narrow form with 128-byte rows.
template <int NG, int HD>
constexpr int attend_v_loads() { return (NG == 1 && HD == 64) ? 2 : 4; }

constexpr float kNegInf = -INFINITY;
constexpr float kLn2 = 0.6931471805599453f;

// One tile for one wave, first half: scores and the online softmax update, for
// groups of up to 4 heads (NG = 1).
// ka: this lane's 4 K chunks in MFMA A layout.  Leaves the probabilities of
// this lane's 4 tokens in pr.  Requires 0 <= first_token <= 16 and
// 0 <= valid_tokens <= 16 (an empty range masks the whole tile).
template <bool F16 = false, int KC = 4>
__device__ __forceinline__ void page_scores(const uint4 (&ka)[KC], const uint4 (&qB)[KC], float& m_run, float& l_run,
                                            floatx4 (&O)[8], float (&pr)[4], float scale_log2, int first_token,
                                            int valid_tokens, int kg) {
  floatx4 S = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < KC; ++c) S = mfma_16x16x32<F16>(ka[c], qB[c], S);
  float s[4];
#pragma unroll
  for (int r = 0; r < 4; ++r)  // token slots [first_token, valid_tokens) of the tile count
    s[r] = ((unsigned)(4 * kg + r - first_token) < (unsigned)(valid_tokens - first_token)) ? S[r] * scale_log2 : kNegInf;
  const float m_new = fmaxf(m_run, fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
  if (__any(m_new > m_run)) {
    const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    l_run *= alpha;
    const float a0 = quad_bcast<0>(alpha), a1 = quad_bcast<1>(alpha);
    const float a2 = quad_bcast<2>(alpha), a3 = quad_bcast<3>(alpha);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      O[u][0] *= a0;
      O[u][1] *= a1;
      O[u][2] *= a2;
      O[u][3] *= a3;
    }
    m_run = m_new;
  }
  const float m_use = (m_run == kNegInf) ? 0.f : m_run;
#pragma unroll
  for (int r = 0; r < 4; ++r) pr[r] = fast_exp2(s[r] - m_use);
  l_run += (pr[0] + pr[1]) + (pr[2] + pr[3]);
}

// Second half: O += P V.  vr: this lane's NV V rows (row 4*kg + r; with NV = 2: row 4*kg + 2*half + r, where
// half says which of the two 8-chunk halves of its row group the lane is in).
template <bool F16 = false, int NV = 4>
__device__ __forceinline__ void page_pv(const u32x4 (&vr)[NV], const float (&pr4)[4], floatx4 (&O)[8], int half) {
  float pr[NV];
  if constexpr (NV == 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) pr[r] = pr4[r];
  } else {
    pr[0] = half ? pr4[2] : pr4[0];
    pr[1] = half ? pr4[3] : pr4[1];
  }
#pragma unroll
  for (int r = 0; r < NV; ++r) {
    const u32x4 vv = vr[r];
    const float vf[8] = {elem_lo<F16>(vv.x), elem_hi<F16>(vv.x), elem_lo<F16>(vv.y), elem_hi<F16>(vv.y),
                         elem_lo<F16>(vv.z), elem_hi<F16>(vv.z), elem_lo<F16>(vv.w), elem_hi<F16>(vv.w)};
#pragma unroll
    for (int u = 0; u < 8; ++u) O[u] = __builtin_amdgcn_mfma_f32_4x4x1f32(pr[r], vf[u], O[u], 0, 0, 0);
  }
}


// Zeroes the V rows of token slots outside [first_token, valid_tokens): their
// probabilities are 0, but 0 * NaN would still poison the accumulator when an
// unused cache slot happens to hold a NaN or Inf bit pattern.
// row0: the tile row of vr[0] (4*kg, or 4*kg + 2*half with two rows per lane).
template <int NV>
__device__ __forceinline__ void clear_unused_v_rows(u32x4 (&vr)[NV], int first_token, int valid_tokens, int row0) {
#pragma unroll
  for (int r = 0; r < NV; ++r)
    if (!((unsigned)(row0 + r - first_token) < (unsigned)(valid_tokens - first_token))) vr[r] = u32x4{0u, 0u, 0u, 0u};
}

// NG names the kernel variant by the heads it holds, 4 * NG: 1 (narrow) or 4 (wide).
template <int NG>
constexpr bool attend_variant_ok() { return NG == 1 || NG == 4; }

// The wide form of page_scores(): qB holds head min(l%16, G-1) in column l%16, so
// lane (kg, c16) ends up with S[head c16][token 4*kg + r].  The running maximum of a
// head is kept equal in the four lanes (kg = 0..3) that share it, because the P V
// product below adds their tokens up inside one matrix instruction: it moves only
// when some token of the tile exceeds it (rare once a list is under way), and only
// then do the lanes exchange their maxima and rescale O.
template <bool F16 = false, int KC = 4>
__device__ __forceinline__ void page_scores_wide(const uint4 (&ka)[KC], const uint4 (&qB)[KC], float& m_run, float& l_run,
                                                 floatx4 (&O)[8], float (&pr)[4], float scale_log2, int first_token,
                                                 int valid_tokens, int kg) {
  floatx4 S = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < KC; ++c) S = mfma_16x16x32<F16>(ka[c], qB[c], S);
  float s[4];
#pragma unroll
  for (int r = 0; r < 4; ++r)
    s[r] = ((unsigned)(4 * kg + r - first_token) < (unsigned)(valid_tokens - first_token)) ? S[r] * scale_log2 : kNegInf;
  const float m_loc = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
  if (__any(m_loc > m_run)) {
    float mt = fmaxf(m_loc, __shfl_xor(m_loc, 16));
    mt = fmaxf(mt, __shfl_xor(mt, 32));
    const float m_new = fmaxf(m_run, mt);
    const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    l_run *= alpha;
    // This lane's O rows are heads 4*kg + 0..3; their factors sit in the lanes whose column is that head.
    const int src = (threadIdx.x & 48) + 4 * kg;
    const float a0 = __shfl(alpha, src), a1 = __shfl(alpha, src + 1);
    const float a2 = __shfl(alpha, src + 2), a3 = __shfl(alpha, src + 3);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      O[u][0] *= a0;
      O[u][1] *= a1;
      O[u][2] *= a2;
      O[u][3] *= a3;
    }
    m_run = m_new;
  }
  const float m_use = (m_run == kNegInf) ? 0.f : m_run;
#pragma unroll
  for (int r = 0; r < 4; ++r) pr[r] = fast_exp2(s[r] - m_use);
  l_run += (pr[0] + pr[1]) + (pr[2] + pr[3]);
}

// O += P V, wide form: A[i = head l%16][k = l/16] = p of token 4*kg + r, B[k = l/16][j = l%16] =
// V[token 4*kg + r][8*(l%16) + u]; the instruction's K = 4 adds the four row groups, so lane
// (kg, c16) accumulates O[head 4*kg + reg][d = 8*c16 + u] over all 16 tokens of the tile.
//
// With 64-element rows (HD = 64) a row has 8 chunks and the 16 columns carry two elements of a chunk instead:
// lane (kg, c16) with c8 = c16 % 8 and hi = c16 / 8 supplies V[token 4*kg + r][8*c8 + 2*uu + hi] (both halves hold
// chunk c8; `shift` = 16 * hi picks the element of dword uu), so a tile takes 16 instructions instead of 32 and the
// lane accumulates O[uu][reg] = out[head 4*kg + reg][8*c8 + 2*uu + hi], uu = 0..3.
template <bool F16 = false, int HD = kHeadDim>
__device__ __forceinline__ void page_pv_wide(const u32x4 (&vr)[4], const float (&pr)[4], floatx4 (&O)[8], int shift) {
  if constexpr (HD == 64) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const u32x4 vv = vr[r];
      const float vf[4] = {elem_lo<F16>(vv.x >> shift), elem_lo<F16>(vv.y >> shift), elem_lo<F16>(vv.z >> shift),
                           elem_lo<F16>(vv.w >> shift)};
#pragma unroll
      for (int uu = 0; uu < 4; ++uu) O[uu] = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[r], vf[uu], O[uu], 0, 0, 0);
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const u32x4 vv = vr[r];
    const float vf[8] = {elem_lo<F16>(vv.x), elem_hi<F16>(vv.x), elem_lo<F16>(vv.y), elem_hi<F16>(vv.y),
                         elem_lo<F16>(vv.z), elem_hi<F16>(vv.z), elem_lo<F16>(vv.w), elem_hi<F16>(vv.w)};
#pragma unroll
    for (int u = 0; u < 8; ++u) O[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[r], vf[u], O[u], 0, 0, 0);
  }
}

// Wave-uniform description of one list for attend_list().
struct AttendArgs {
  const uint16_t* q_bh;  // the group's G query rows (contiguous, HD elements each)
  const char* kvb;       // kv_cache base + h * HD * 2 bytes
  int row_bytes;         // bytes between token rows of a page (H_kv * HD * 2)
  int page_bytes;        // 2 * page_size * row_bytes
  int span;              // bytes addressable from kvb within one page
  int page_size;         // tokens per page: 16, 32, 64 or 128
  int64_t num_pages;
  int G;
  float scale_log2;      // sm_scale * log2(e)
  int n;                 // list length
  int p0, p1;            // this workgroup's part of the list [p0, p1)
  int last_len;          // tokens in the list's final page
  int first_skip;        // leading token slots of list entry 0 that hold no token (0 .. page_size-1)
  unsigned rotate;       // long parts start at tile (rotate mod tiles) and wrap around; 0: in list order
};

// Long lists that many workgroups walk in step -- dense decode over a cache whose pages are numbered
// p * batch + b, as the reference lays them out -- are all at the same page at the same time and
// read one narrow window of the cache (1024 sequences: 81 % of peak against 85-87 % for any other
// numbering).  Every list therefore starts at its own tile and wraps around; the sum over tiles does
// not care about the order.  Only with at least two lists per CU (512 sequences: 74 % in list order,
// 82 % rotated; with fewer, neighbours reading neighbouring pages helps: 256 lists lose 3 % when
// rotated, 384 lists 1 %) and only parts of at least
// kRotateMinTiles tiles.  The rule depends on the batch alone, so the fused step and the stand-alone
// kernel visit a list's tiles in the same order.
constexpr int kRotateMinTiles = 512;
__host__ __device__ inline bool attend_rotates(int64_t lists) { return lists >= 2 * kNumCus; }
__device__ __forceinline__ unsigned attend_rotation(int list, int split) {
  return ((unsigned)list * 2654435761u >> 8) + 977u * (unsigned)split;
}

// K tiles a wave keeps staged in LDS in attend_list(): the one being read and the one in flight.
constexpr int kAttendStages = 2;
// K staging for NW waves of kAttendStages stages of 4 KiB each (2 KiB with 64-element rows); the same 8 KiB per wave hold the
// merge buffer [NW][4*NG][HD] fp32 afterwards (up to 2 KiB per wave for NG = 1, 8 KiB for the wide form).
constexpr int attend_lds_bytes(int nw) { return nw * kAttendStages * 4096; }

// Common tail of the attention loops: merges the wave's 4 row groups, then the
// workgroup's NW waves through LDS, and hands out the normalised results.
// m_run / l_run / O: this lane's online-softmax state (see page_scores).
template <int NG, int NW, int HD, typename Emit>
__device__ __forceinline__ void attend_finish(float m_run, float l_run, floatx4 (&O)[8], int G, unsigned char* lds,
                                              float (*sm_m)[4 * NG], float (*sm_l)[4 * NG], Emit emit) {
  static_assert(attend_variant_ok<NG>(), "NG is 1 (up to 4 heads) or 4 (up to 16)");
  static_assert(HD == 128 || HD == 64, "head rows of 128 or 64 elements");
  constexpr int CPR = HD / 8;  // 16-byte chunks of a head row
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, kg = l >> 4, c16 = l & 15, cc = c16 & (CPR - 1);
  // LDS-direct loads that are still in flight (masked tail pages) must land
  // before the staging area is reused below.
  __builtin_amdgcn_s_waitcnt(0);
  float* ow = reinterpret_cast<float*>(lds);  // [NW waves][4*NG heads][HD]

  if constexpr (NG == 4) {
    // Wide form: O is already summed over the row groups; the lanes of a head share m
    // and hold partial sums l.
    float ll = l_run;
    ll += __shfl_xor(ll, 16);
    ll += __shfl_xor(ll, 32);
    __syncthreads();  // every wave is done with its K staging area
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int h = 4 * kg + i;
      if (h < G) {
        if constexpr (HD == 64) {  // this lane's columns are 8*cc + 2*uu + (c16 >> 3), see page_pv_wide
          float* dst = ow + ((w * 16 + h) * HD + 8 * cc + (c16 >> 3));
#pragma unroll
          for (int uu = 0; uu < 4; ++uu) dst[2 * uu] = O[uu][i];
        } else {
          float* dst = ow + ((w * 16 + h) * HD + 8 * cc);
          *reinterpret_cast<float4*>(dst) = make_float4(O[0][i], O[1][i], O[2][i], O[3][i]);
          *reinterpret_cast<float4*>(dst + 4) = make_float4(O[4][i], O[5][i], O[6][i], O[7][i]);
        }
      }
    }
    if (l < 16) {
      sm_m[w][l] = m_run;
      sm_l[w][l] = ll;
    }
  } else {
    // ---- merge the 4 row groups of the wave (lanes l, l^16, l^32, l^48) --------
    float mm = m_run;
    mm = fmaxf(mm, __shfl_xor(mm, 16));
    mm = fmaxf(mm, __shfl_xor(mm, 32));
    const float m_safe = (mm == kNegInf) ? 0.f : mm;
    const float sc = fast_exp2(m_run - m_safe);
    float ll = l_run * sc;
    ll += __shfl_xor(ll, 16);
    ll += __shfl_xor(ll, 32);
    const float s0 = quad_bcast<0>(sc), s1 = quad_bcast<1>(sc), s2 = quad_bcast<2>(sc), s3 = quad_bcast<3>(sc);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      float x0 = O[u][0] * s0, x1 = O[u][1] * s1, x2 = O[u][2] * s2, x3 = O[u][3] * s3;
      if constexpr (HD == 64) {  // the two halves of a row group took different tokens of it
        x0 += __shfl_xor(x0, 8); x1 += __shfl_xor(x1, 8); x2 += __shfl_xor(x2, 8); x3 += __shfl_xor(x3, 8);
      }
      x0 += __shfl_xor(x0, 16); x1 += __shfl_xor(x1, 16); x2 += __shfl_xor(x2, 16); x3 += __shfl_xor(x3, 16);
      x0 += __shfl_xor(x0, 32); x1 += __shfl_xor(x1, 32); x2 += __shfl_xor(x2, 32); x3 += __shfl_xor(x3, 32);
      O[u] = floatx4{x0, x1, x2, x3};
    }
    __syncthreads();  // every wave is done with its K staging area
    if (kg == 0 && c16 < CPR) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float* dst = ow + ((w * 4 + i) * HD + 8 * cc);
        *reinterpret_cast<float4*>(dst) = make_float4(O[0][i], O[1][i], O[2][i], O[3][i]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(O[4][i], O[5][i], O[6][i], O[7][i]);
      }
      if (l < 4) {
        sm_m[w][l] = mm;
        sm_l[w][l] = ll;
      }
    }
  }
  __syncthreads();

  // ---- merge the NW waves and hand the results out ------------------------------
  for (int idx = tid; idx < 4 * NG * HD; idx += NW * 64) {
    const int g = idx / HD, d = idx & (HD - 1);
    if (g < G) {
      float mm = kNegInf;
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) mm = fmaxf(mm, sm_m[wv][g]);
      const float m_safe = (mm == kNegInf) ? 0.f : mm;
      float num = 0.f, den = 0.f;
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) {
        const float sc = fast_exp2(sm_m[wv][g] - m_safe);
        num += ow[(wv * 4 * NG + g) * HD + d] * sc;
        den += sm_l[wv][g] * sc;
      }
      const float o = (den > 0.f) ? num / den : 0.f;
      const float lse2 = (den > 0.f) ? mm + fast_log2(den) : kNegInf;
      emit(g, d, o, lse2);
    }
  }
}

// id_at(i) returns the (wave-uniform) physical page id of list entry i, 0 <= i < n.
// emit(g, d, o, lse2) receives, once per (head g < G, column d), the normalised
// output and the base-2 log-sum-exp (-inf and o = 0 for an empty part).
// lds: attend_lds_bytes(NW), 16-byte aligned; sm_m / sm_l: NW x
// (4*NG) floats each.
// Every one of the workgroup's NW*64 threads calls this.
template <int NG, int NW, bool F16 = false, int HD = kHeadDim, typename IdAt, typename Emit>
__device__ __forceinline__ void attend_list(const AttendArgs& a, IdAt id_at, unsigned char* lds,
                                            float (*sm_m)[4 * NG], float (*sm_l)[4 * NG], Emit emit) {
  static_assert(HD == 128 || HD == 64, "head rows of 128 or 64 elements");
  constexpr int CPR = HD / 8;                      // 16-byte chunks of a head row: 16 or 8
  constexpr int KC = HD / 32;                      // matrix steps over the head dimension = LDS-direct loads per K tile: 4 or 2
  constexpr int RPI = 64 / CPR;                    // K rows one LDS-direct load brings: 4 or 8
  constexpr int NV = attend_v_loads<NG, HD>();     // V rows per lane and tile
  constexpr int kStage = kPageSize * HD * 2;       // bytes of one K stage (a tile's keys)
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l = tid & 63, kg = l >> 4, c16 = l & 15, gq = l & 3, cc = c16 & (CPR - 1);
  const int half = NV == 2 ? (c16 >> 3) : 0;       // which half of its row group's tokens this lane's V rows cover
  const int vrow0 = 4 * kg + 2 * half;             // tile row of this lane's first V row
  const int G = a.G;
  const int n = a.n, p0 = a.p0, p1 = a.p1, last_len = a.last_len;

  // Query operands: B[k][j], j = l%16 -> head l%4 (wide form: head l%16), k-chunk = l/16.
  uint4 qB[KC];
  {
    const int g = min(NG == 4 ? c16 : gq, G - 1);
    const uint16_t* qp = a.q_bh + (int64_t)g * HD + 8 * kg;
#pragma unroll
    for (int c = 0; c < KC; ++c) qB[c] = *reinterpret_cast<const uint4*>(qp + 32 * c);
  }

  const int row_bytes = a.row_bytes;
  const int page_bytes = a.page_bytes;
  const int span = a.span;
  const char* kvb = a.kvb;
  // A tile's rows are addressed from its first K row: its V rows lie one K plane
  // (page_size rows) further.
  const int tshift = page_tile_shift(a.page_size), tmask = (1 << tshift) - 1;
  int voff[NV];
#pragma unroll
  for (int r = 0; r < NV; ++r) voff[r] = (a.page_size + vrow0 + r) * row_bytes + cc * 16;
  // K staging: kAttendStages stages of one tile's keys per wave, filled by LDS-direct buffer loads
  // (no VGPRs while in flight).  Load c brings rows RPI*c .. RPI*c + RPI-1, one kilobyte: lane l
  // lands at LDS row RPI*c + l / CPR, position l % CPR, and fetches the chunk that belongs
  // there under the XOR swizzle (see attend_swizzle).
  unsigned char* kl = lds + w * (kAttendStages * kStage);
  int kdma_off[KC], lds_r[KC];
#pragma unroll
  for (int c = 0; c < KC; ++c) {
    const int row = RPI * c + l / CPR;
    kdma_off[c] = row * row_bytes + ((cc ^ attend_swizzle<HD>(row)) & (CPR - 1)) * 16;
    const int chunk_r = 4 * c + kg;  // chunk of row c16 that MFMA c wants from this lane
    lds_r[c] = c16 * (HD * 2) + ((chunk_r ^ attend_swizzle<HD>(c16)) & (CPR - 1)) * 16;
  }

  float m_run = kNegInf, l_run = 0.f;
  floatx4 O[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) O[u] = floatx4{0.f, 0.f, 0.f, 0.f};
  auto scores = [&](const uint4 (&ka)[KC], float (&pr)[4], int valid) {
    if constexpr (NG == 4)
      page_scores_wide<F16, KC>(ka, qB, m_run, l_run, O, pr, a.scale_log2, valid >> 8, valid & 255, kg);
    else
      page_scores<F16, KC>(ka, qB, m_run, l_run, O, pr, a.scale_log2, valid >> 8, valid & 255, kg);
  };
  auto pv = [&](const u32x4 (&vr)[NV], const float (&pr)[4]) {
    if constexpr (NG == 4)
      page_pv_wide<F16, HD>(vr, pr, O, 16 * (c16 >> 3));
    else
      page_pv<F16, NV>(vr, pr, O, half);
  };

  // This wave takes the tiles my_first, my_first+NW, ... of the list entries p0 .. p1-1
  // (entry e owns the tiles e << tshift ..; of the list's final page only the tiles
  // that hold tokens count).  The loop below is branch-free: a tile past the end (or
  // of a page with an id outside the cache) is read through an empty buffer
  // descriptor -- zeros, no memory traffic -- and all of its tokens are masked.
  const int n_last = n - 1;
  const int n_tiles = n > 0 ? (n_last << tshift) + ((min(max(last_len, 1), a.page_size) + kPageSize - 1) >> 4) : 0;
  const int t0 = p0 << tshift, t1 = min(p1 << tshift, n_tiles);
  const int my_first = t0 + w;
  const int iters = (t1 > my_first) ? (t1 - my_first + NW - 1) / NW : 0;
  // The it-th tile of this wave: my_first + NW * it, shifted by the part's rotation (see attend_rotates()).
  const int span_t = t1 - t0;
  const int rot = span_t >= kRotateMinTiles ? (int)(a.rotate % (unsigned)span_t) : 0;
  auto tile_at = [&](int it) -> int {
    const int i = my_first + NW * it;
    if (i >= t1) return i;  // past the end: stays past the end
    const int r = i - t0 + rot;
    return t0 + (r >= span_t ? r - span_t : r);
  };
  // Page ids are fetched one half-step before they are needed.
  auto load_id = [&](int it) -> int {
    const int idx = tile_at(it);
    return id_at((idx < t1 ? idx : t0) >> tshift);
  };
  const int first_skip = a.first_skip;
  auto page_rsrc = [&](int it, int id, int& valid_tokens) {
    const int idx = tile_at(it);
    const int e = idx >> tshift, sub16 = (idx & tmask) * kPageSize;  // list entry, first token slot of the tile in its page
    const bool ok = idx < t1 && id >= 0 && (int64_t)id < a.num_pages;
    // The token slots of the page that count are [lo_p, hi_p); the tile's share of
    // them is folded into one number: bits 8.. hold the first counted slot of the
    // tile, bits 0..7 one past the last.
    const int hi_p = e == n_last ? last_len : a.page_size;
    const int lo_p = e == 0 ? min(first_skip, hi_p) : 0;
    const int hi = min(max(hi_p - sub16, 0), kPageSize);
    const int lo = min(max(lo_p - sub16, 0), hi);
    valid_tokens = ok ? (hi | (lo << 8)) : 0;
    const int tile_off = sub16 * row_bytes;
    return make_rsrc(kvb + (int64_t)(ok ? id : 0) * page_bytes + tile_off, ok ? span - tile_off : 0);
  };
  auto issue_v = [&](__amdgpu_buffer_rsrc_t r, u32x4 (&vv)[NV]) {
#pragma unroll
    for (int c = 0; c < NV; ++c) vv[c] = __builtin_amdgcn_raw_buffer_load_b128(r, voff[c], 0, kStreamLoad);
  };
  auto issue_k = [&](__amdgpu_buffer_rsrc_t r, int stage) {
    __attribute__((address_space(3))) unsigned char* dst =
        (__attribute__((address_space(3))) unsigned char*)(kl + stage * kStage);
#pragma unroll
    for (int c = 0; c < KC; ++c)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, dst + c * 1024, 16, kdma_off[c], 0, 0, kStreamLoad);
  };
  auto read_k = [&](int stage, uint4 (&ka)[KC]) {
#pragma unroll
    for (int c = 0; c < KC; ++c) ka[c] = *reinterpret_cast<const uint4*>(kl + stage * kStage + lds_r[c]);
  };

  // The compiler does not order LDS reads after LDS-direct loads by itself, so
  // the wait is explicit: when it executes, exactly the NV V loads issued just
  // before it are allowed to be outstanding, which means the K stage about to
  // be read (and the V registers about to be used) have landed.  The scheduling
  // fences keep the instruction order this count relies on.
  if (iters > 0 && n > 0) {
    u32x4 vA[NV], vB[NV];
    uint4 ka[KC];
    float pr[4];
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
        __builtin_amdgcn_s_waitcnt(wait_vm_imm(NV));
        __builtin_amdgcn_sched_barrier(0);
        read_k(0, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(r1, 1);
        __builtin_amdgcn_sched_barrier(0);
        scores(ka, pr, validA);
        __builtin_amdgcn_sched_barrier(0);
        id_next = load_id(it + 2);  // lands while the P V products run
        if (validA != kPageSize) clear_unused_v_rows<NV>(vA, validA >> 8, validA & 255, vrow0);  // partial page: rare
        pv(vA, pr);
      }
      {
        const __amdgpu_buffer_rsrc_t r2 = page_rsrc(it + 2, id_next, validA);
        __builtin_amdgcn_sched_barrier(0);
        issue_v(r2, vA);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(wait_vm_imm(NV));
        __builtin_amdgcn_sched_barrier(0);
        read_k(1, ka);
        __builtin_amdgcn_sched_barrier(0);
        issue_k(r2, 0);
        __builtin_amdgcn_sched_barrier(0);
        scores(ka, pr, validB);
        __builtin_amdgcn_sched_barrier(0);
        id_next = load_id(it + 3);
        if (validB != kPageSize) clear_unused_v_rows<NV>(vB, validB >> 8, validB & 255, vrow0);
        pv(vB, pr);
      }
    }
  }
  attend_finish<NG, NW, HD>(m_run, l_run, O, G, lds, sm_m, sm_l, emit);
}

// Merges the `parts` partial results that the workgroups sharing one list left in
// global memory (ws_po [lists, parts, G, HD] normalised outputs, ws_plse [lists, parts, G]
// base-2 log-sum-exps, both fp32 bits written at device scope) and writes the list's G output
// rows (out_bh) and, if lse_bh is set, their natural-log log-sum-exps.  Run by the workgroup
// that counted in last, all NT threads; lds: room for (parts + 1) * G floats, free for reuse.
// The log-sum-exps first become weights in LDS, then every thread sums its output element over
// the parts with independent device-scope loads (the arithmetic of merge_splits_kernel).
template <int NT, bool F16, int HD = kHeadDim>
__device__ __forceinline__ void merge_list_parts(unsigned char* lds, const uint32_t* ws_po, const uint32_t* ws_plse, int item,
                                                 int parts, int G, uint16_t* out_bh, float* lse_bh) {
  const int tid = threadIdx.x;
  float* wl = reinterpret_cast<float*>(lds);  // [parts][G] weights, then [G] denominators
  float* den_g = wl + parts * G;
  const int64_t first_row = (int64_t)item * parts * G;
  const __amdgpu_buffer_rsrc_t rl = make_rsrc(ws_plse + first_row, parts * G * (int)sizeof(float));
  for (int i = tid; i < parts * G; i += NT)
    wl[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rl, i * 4, 0, kDeviceScope));
  __syncthreads();
  if (tid < G) {
    float mm = kNegInf;
    for (int sp = 0; sp < parts; ++sp) mm = fmaxf(mm, wl[sp * G + tid]);
    const float m_safe = (mm == kNegInf) ? 0.f : mm;
    float den = 0.f;
    for (int sp = 0; sp < parts; ++sp) {
      const float wgt = fast_exp2(wl[sp * G + tid] - m_safe);
      wl[sp * G + tid] = wgt;
      den += wgt;
    }
    den_g[tid] = den;
    if (lse_bh) lse_bh[tid] = (den > 0.f) ? (mm + fast_log2(den)) * kLn2 : kNegInf;
  }
  __syncthreads();
  const __amdgpu_buffer_rsrc_t ro = make_rsrc(ws_po + first_row * HD, parts * G * HD * (int)sizeof(float));
  for (int idx = tid; idx < G * HD; idx += NT) {
    const int g = idx / HD, d = idx & (HD - 1);
    float num = 0.f;
#pragma unroll 8
    for (int sp = 0; sp < parts; ++sp)
      num += __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ro, ((sp * G + g) * HD + d) * 4, 0, kDeviceScope)) *
             wl[sp * G + g];
    const float den = den_g[g];
    out_bh[g * HD + d] = (uint16_t)f32_to_elem<F16>(den > 0.f ? num / den : 0.f);
  }
}

}  // namespace kin
