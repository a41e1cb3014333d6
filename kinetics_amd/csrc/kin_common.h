// Shared host/device helpers for the gfx950 block top-k decode kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kinetics_amd.h"

namespace kin {

constexpr int kHeadDim = 128;    // elements per head row (256 B in bf16): the default, and the largest, head dimension
constexpr int kHeadDimSmall = 64;  // the second head dimension the page path is built for (128-byte rows)
constexpr int kPageSize = 16;    // tokens of one attention tile (an MFMA tile is 16 keys); the smallest page
constexpr int kMaxPageSize = 128; // pages hold 16, 32, 64 or 128 tokens: 1, 2, 4 or 8 tiles
constexpr int kRowBytes = kHeadDim * 2;
constexpr int kMaxGroup = 16;    // largest supported num_q_heads / num_kv_heads
constexpr int kMaxTopk = 2048;
constexpr int kMaxCandidates = 16384;
constexpr int kNumCus = 256;     // compute units of the target GPU (MI355X)
constexpr int kNumXcds = 8;      // accelerator dies, each with its own L2

// Workgroups to launch for one list per (sequence, KV head) under xcd_list_of().
inline int64_t xcd_grid_size(int batch, int num_kv_heads) {
  if (num_kv_heads == 1) return batch;
  return ((int64_t)batch + kNumXcds - 1) / kNumXcds * kNumXcds * num_kv_heads;
}
constexpr int kMaxFixedPages = 64;  // most sink / local pages that can be pinned into every list
constexpr int kMaxLocalTokens = (kMaxFixedPages - 1) * kPageSize + 1;

// Most trailing pages that local_tokens always-attended trailing tokens can span
// (for 16-token pages; larger pages need no more).
__host__ __device__ inline int max_local_pages(int local_tokens) { return 1 + (local_tokens + kPageSize - 2) / kPageSize; }

inline bool supported_page_size(int ps) { return ps == 16 || ps == 32 || ps == 64 || ps == 128; }
inline bool supported_head_dim(int hd) { return hd == kHeadDim || hd == kHeadDimSmall; }
// log2(page_size / 16): a page is 1 << page_tile_shift(ps) tiles of 16 tokens.
__host__ __device__ inline int page_tile_shift(int ps) { return ps >= 128 ? 3 : (ps >= 64 ? 2 : (ps >= 32 ? 1 : 0)); }

// Cache-policy bits for buffer loads of read-once data (K/V pages, mean keys):
// the non-temporal hint keeps streams from displacing each other in L2/MALL and
// measurably raises achieved HBM read bandwidth (about 6.3 -> 7.0 TB/s on a
// plain streaming read).
constexpr int kStreamLoad = 2;  // "nt"
// Cache-policy bit for buffer loads and stores at device scope ("sc1", what a
// relaxed agent-scope atomic access uses): the access bypasses the XCD-private
// L2, so workgroups on different XCDs can hand data to each other through
// memory inside one launch without cache maintenance.
constexpr int kDeviceScope = 16;

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte access: 8 bf16

// ---- host side: status + thread-local message -----------------------------
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int check_hip(hipError_t e, const char* what);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Shape rules every entry point shares.  Returns KIN_OK or records an error.
// small_head_dim_built: the entry point also has kernels for head_dim 64 (the page path has, the
// token-granular policies and the layer's row kernels have not).
int check_common_dims(const char* fn, int batch, int num_q_heads, int num_kv_heads,
                      int head_dim, int page_size, bool small_head_dim_built = false);
// Range rules for the always-attended parts of a page list.
int check_fixed_pages(const char* fn, int sink_pages, int local_tokens);
// first_page_offset: padding slots at the start of every sequence's first page.
int check_first_page_offset(const char* fn, int first_page_offset, int page_size = kPageSize);
// The token-granular policies address single token rows and are built for 16-token pages only.
int check_page_size_16(const char* fn, int page_size);

// Split scoring of the page selector (few, long lists): workgroups per list.  1
// unless the lists are at most a quarter of the CUs and long, then enough to put
// a workgroup on every CU, each with at least 256 candidates.
inline int score_chunks(int batch, int num_kv_heads, int kbar_pages) {
  const int64_t items = (int64_t)batch * num_kv_heads;
  if (items <= 0 || items * 4 > kNumCus || kbar_pages < 2048) return 1;
  int64_t c = kNumCus / items;
  const int64_t by_rows = kbar_pages / 256;
  if (c > by_rows) c = by_rows;
  return c < 2 ? 1 : (int)c;
}
// Bytes of the per-list arrival counters in front of the shared key array.
inline size_t score_count_bytes(int64_t items) { return ((size_t)items * sizeof(int32_t) + 255) & ~(size_t)255; }
// Keys per list in the shared key array: a multiple of 4, so that every list starts 16-byte aligned.
__host__ __device__ inline int score_key_stride(int kbar_pages) { return (kbar_pages + 3) & ~3; }
// Workspace of split scoring: counters, then score_key_stride() keys per list.
inline size_t score_workspace_bytes(int64_t items, int kbar_pages) {
  return score_count_bytes(items) + (size_t)items * score_key_stride(kbar_pages) * sizeof(uint32_t);
}

// Row of kbar[batch, num_kv_heads, kbar_pages, head_dim] that holds the mean key
// of logical page `page` of (sequence b, KV head h): head-major, so the
// candidates of one list are one contiguous run of 256-byte rows.
__host__ __device__ inline int64_t kbar_row_index(int b, int h, int page, int num_kv_heads, int kbar_pages) {
  return ((int64_t)b * num_kv_heads + h) * kbar_pages + page;
}

// ---- device side -----------------------------------------------------------
#if defined(__HIPCC__)

// Row block of kbar that holds the mean keys of sequence b: b itself, or slot_ids[b] when the
// caller keeps kbar by cache slot (a serving engine's active batch is a changing subset of its
// slots, and q, k, v, out and the page table follow the batch while the mean keys stay with
// the slot).  -1 for an id outside [0, num_slots): such a sequence has no mean keys.
__device__ __forceinline__ int kbar_block_of(const int32_t* slot_ids, int num_slots, int b) {
  const int s = slot_ids ? slot_ids[b] : b;
  return (unsigned)s < (unsigned)num_slots ? s : -1;
}

// Workgroups are handed to the GPU's 8 XCDs round-robin by index; every XCD has
// its own L2 and address-translation caches.  The lists of one sequence's KV
// heads read different parts of the same KV pages and the same page-table
// entries, so they go to workgroups of ONE XCD: with t = bid / 8 and x = bid % 8,
// workgroup bid handles head t % hkv of sequence (t / hkv) * 8 + x.  The grid
// is xcd_grid_size(batch, hkv) workgroups; false marks a padding workgroup.
__device__ __forceinline__ bool xcd_list_of(int bid, int batch, int hkv, int& b, int& h) {
  if (hkv == 1) {
    b = bid;
    h = 0;
    return true;
  }
  const int t = bid / kNumXcds, x = bid - t * kNumXcds;
  const int tb = t / hkv;
  h = t - tb * hkv;
  b = tb * kNumXcds + x;
  return b < batch;
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> bf16 bits, round-to-nearest-even, NaN kept quiet.
__device__ __forceinline__ uint32_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

// ---- element formats --------------------------------------------------------
// q, k, v, kv_cache, kbar and out hold bfloat16 (F16 = false) or IEEE half
// (F16 = true, the reference's --dtype float16); everything is accumulated in fp32.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// The two elements packed in one dword, widened to fp32 (exact).
template <bool F16>
__device__ __forceinline__ float elem_lo(uint32_t w) {
  if constexpr (F16) return (float)__builtin_bit_cast(f16x2, w).x;
  else return bf16_lo(w);
}
template <bool F16>
__device__ __forceinline__ float elem_hi(uint32_t w) {
  if constexpr (F16) return (float)__builtin_bit_cast(f16x2, w).y;
  else return bf16_hi(w);
}
// fp32 -> element bits (low 16 bits of the result), round-to-nearest-even.
template <bool F16>
__device__ __forceinline__ uint32_t f32_to_elem(float f) {
  if constexpr (F16) return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
  else return f32_to_bf16(f);
}
// 16 keys x 32 columns times 32 columns x 16 queries on the matrix unit, 8 elements per lane and operand.
template <bool F16>
__device__ __forceinline__ floatx4 mfma_16x16x32(const uint4& a, const uint4& b, floatx4 c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// DPP lane permutes inside a row of 16 lanes (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
constexpr int kDppQuadXor1 = 0xB1;     // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;     // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // row_half_mirror: lane i <- 7-i (per 8)
constexpr int kDppMirror = 0x140;      // row_mirror:      lane i <- 15-i (per 16)

// Sum over each aligned group of 16 lanes; every lane of the group gets it.
__device__ __forceinline__ float row16_sum(float x) {
  x += dpp_f<kDppQuadXor1>(x);
  x += dpp_f<kDppQuadXor2>(x);
  x += dpp_f<kDppHalfMirror>(x);
  x += dpp_f<kDppMirror>(x);
  return x;
}
// Sum over each aligned group of LANES (8 or 16) lanes: the lanes that share one head row of LANES * 8 elements.
template <int LANES>
__device__ __forceinline__ float row_sum(float x) {
  static_assert(LANES == 8 || LANES == 16, "a head row is 8 or 16 chunks of 16 bytes");
  x += dpp_f<kDppQuadXor1>(x);
  x += dpp_f<kDppQuadXor2>(x);
  x += dpp_f<kDppHalfMirror>(x);
  if constexpr (LANES == 16) x += dpp_f<kDppMirror>(x);
  return x;
}

// Inclusive prefix sum over the 64 lanes of a wave on the DPP path (no LDS crossbar: about a
// tenth of the latency of six ds_bpermute steps): inside each row of 16 lanes by shifts of
// 1, 2, 3, then 4 and 8, then lane 15 of rows 0 and 2 is added to rows 1 and 3, and lane 31
// to rows 2 and 3.  A lane without a source takes 0.
template <int CTRL, int ROW_MASK, int BANK_MASK>
__device__ __forceinline__ uint32_t dpp_or_zero(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, ROW_MASK, BANK_MASK, false);
}
__device__ __forceinline__ uint32_t wave_inclusive_sum(uint32_t x) {
  uint32_t s = x + dpp_or_zero<0x111, 0xf, 0xf>(x) + dpp_or_zero<0x112, 0xf, 0xf>(x) + dpp_or_zero<0x113, 0xf, 0xf>(x);  // row_shr:1..3
  s += dpp_or_zero<0x114, 0xf, 0xe>(s);  // row_shr:4 into lanes 4..15 of each row
  s += dpp_or_zero<0x118, 0xf, 0xc>(s);  // row_shr:8 into lanes 8..15
  s += dpp_or_zero<0x142, 0xa, 0xf>(s);  // row_bcast:15 into rows 1 and 3
  s += dpp_or_zero<0x143, 0xc, 0xf>(s);  // row_bcast:31 into rows 2 and 3
  return s;
}

// Value of lane (quad base + I) broadcast to the 4 lanes of each quad.
template <int I>
__device__ __forceinline__ float quad_bcast(float x) {
  return dpp_f<(I) | (I << 2) | (I << 4) | (I << 6)>(x);
}

// Buffer descriptor covering `bytes` bytes from `base` (0 bytes: every load
// through it returns zeros without touching memory).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// Zeroes n int32 counters.  A kernel rather than a memset so that the launch
// sequences that use it can be captured into a HIP graph.  (static: every
// translation unit that launches it gets its own copy.)
static __global__ __attribute__((unused)) void fill_zero_i32_kernel(int32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

#ifdef KIN_TUNE
// Phase stamps of the diagnostic build (-DKIN_TUNE): per workgroup up to 64 (tag, 100 MHz clock) pairs, in
// arrays private to the translation unit; the accessor copies them out and empties them.
static __device__ long long g_stamps[1024 * 64 * 2];
static __device__ int g_nstamps[1024];
#define KIN_STAMP(tag)                                                          \
  do {                                                                          \
    if (threadIdx.x == 0 && blockIdx.x < 1024) {                                \
      const int k_ = g_nstamps[blockIdx.x];                                     \
      if (k_ < 64) {                                                            \
        g_stamps[(blockIdx.x * 64 + k_) * 2] = (tag);                           \
        g_stamps[(blockIdx.x * 64 + k_) * 2 + 1] = wall_clock64();              \
        g_nstamps[blockIdx.x] = k_ + 1;                                         \
      }                                                                         \
    }                                                                           \
  } while (0)
#define KIN_STAMP_RESET()                                                       \
  do {                                                                          \
    if (threadIdx.x == 0 && blockIdx.x < 1024) g_nstamps[blockIdx.x] = 0;       \
  } while (0)
#define KIN_STAMP_ACCESSOR(fn_name)                                                                                          \
  extern "C" int fn_name(long long* stamps, int* counts) {                                                                  \
    if (hipDeviceSynchronize() != hipSuccess) return 1;                                                                      \
    if (hipMemcpyFromSymbol(stamps, HIP_SYMBOL(kin::g_stamps), sizeof(long long) * 1024 * 64 * 2) != hipSuccess) return 2;   \
    if (hipMemcpyFromSymbol(counts, HIP_SYMBOL(kin::g_nstamps), sizeof(int) * 1024) != hipSuccess) return 3;                 \
    static const int zeros_[1024] = {};  /* the next reading starts empty, whatever grid wrote this one */                   \
    if (hipMemcpyToSymbol(HIP_SYMBOL(kin::g_nstamps), zeros_, sizeof(zeros_)) != hipSuccess) return 4;                       \
    return 0;                                                                                                                \
  }
#else
#define KIN_STAMP(tag) do { } while (0)
#define KIN_STAMP_RESET() do { } while (0)
#endif

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

#endif  // __HIPCC__

}  // namespace kin
