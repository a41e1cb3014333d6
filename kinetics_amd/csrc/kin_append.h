// Device-side building block: one wave appends one token's K and V rows for one
// (sequence, KV head) and refreshes the mean key of the page when the row fills
// it.  Shared by the stand-alone append kernel and the fused decode step.
#pragma once

#include "kin_common.h"

namespace kin {

// Mean of the page_size key rows of one page for one head, for this lane's
// two columns.  `krow` points at slot 0 of the page's K plane for that head
// (in dwords); `row_stride` is in dwords.  Sum order is slot 0, 1, ..., page_size-1.
template <bool F16 = false>
__device__ __forceinline__ uint32_t page_mean_dword(const uint32_t* krow, int row_stride, int lane, int page_size) {
  float s0 = 0.f, s1 = 0.f;
#pragma unroll 16
  for (int t = 0; t < page_size; ++t) {
    const uint32_t w = krow[(int64_t)t * row_stride + lane];
    s0 += elem_lo<F16>(w);
    s1 += elem_hi<F16>(w);
  }
  const float inv = 1.0f / (float)page_size;
  return f32_to_elem<F16>(s0 * inv) | (f32_to_elem<F16>(s1 * inv) << 16);
}

// The same mean for 8 columns at once: `kplane16` points at this lane's 16 bytes of
// slot 0 (lane c16 of 16 owns columns 8*c16 .. 8*c16+7), `row_stride16` is the
// distance between token rows in 16-byte units.  16 loads are in flight
// together (one tile of the page at a time); the sums run in slot order like
// page_mean_dword(), so both give the same bits.
template <bool F16 = false>
__device__ __forceinline__ u32x4 page_mean_16B(const u32x4* kplane16, int row_stride16, int page_size) {
  float acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = 0.f;
  for (int t0 = 0; t0 < page_size; t0 += kPageSize) {
    u32x4 x[kPageSize];
#pragma unroll
    for (int t = 0; t < kPageSize; ++t) x[t] = __builtin_nontemporal_load(kplane16 + (int64_t)(t0 + t) * row_stride16);
#pragma unroll
    for (int t = 0; t < kPageSize; ++t) {
      acc[0] += elem_lo<F16>(x[t].x); acc[1] += elem_hi<F16>(x[t].x);
      acc[2] += elem_lo<F16>(x[t].y); acc[3] += elem_hi<F16>(x[t].y);
      acc[4] += elem_lo<F16>(x[t].z); acc[5] += elem_hi<F16>(x[t].z);
      acc[6] += elem_lo<F16>(x[t].w); acc[7] += elem_hi<F16>(x[t].w);
    }
  }
  const float inv = 1.0f / (float)page_size;
  u32x4 m;
  m.x = f32_to_elem<F16>(acc[0] * inv) | (f32_to_elem<F16>(acc[1] * inv) << 16);
  m.y = f32_to_elem<F16>(acc[2] * inv) | (f32_to_elem<F16>(acc[3] * inv) << 16);
  m.z = f32_to_elem<F16>(acc[4] * inv) | (f32_to_elem<F16>(acc[5] * inv) << 16);
  m.w = f32_to_elem<F16>(acc[6] * inv) | (f32_to_elem<F16>(acc[7] * inv) << 16);
  return m;
}

// Run by the 64 lanes of one wave (lane = 0..63, 4 bytes each = one 256-byte row; with HD = 64 the
// first 32 lanes move the 128-byte row and the others do nothing).
// k_row / v_row: the new token's rows for this (sequence, head), in dwords.
// The row lands in slot last_len-1 of the sequence's last page (physical id
// last_pid).  If that fills the page and the page has a slot in kbar
// (n_pages-1 < kbar_pages, kbar may be null), its mean key goes to
// kbar_page_row, the dword address of kbar[b, h, n_pages-1, 0]: the earlier rows are
// read from the cache, the last row is taken from the register, so the result does not
// depend on store visibility.  Metadata outside its contract would write
// outside the cache: the row is skipped.
template <bool F16 = false, int HD = kHeadDim>
__device__ __forceinline__ void append_token_row(const uint32_t* k_row, const uint32_t* v_row, uint32_t* kv_cache,
                                                 uint32_t* kbar_page_row, int64_t last_pid, int last_len, int n_pages,
                                                 int kbar_pages, int h, int num_kv_heads, int64_t num_pages, int lane,
                                                 int page_size) {
  const int pos = last_len - 1;
  if (pos < 0 || pos >= page_size || last_pid < 0 || last_pid >= num_pages) return;
  if (HD < 128 && lane >= HD / 2) return;
  const int row_stride = num_kv_heads * (HD / 2);            // dwords per token row
  const int64_t page_dwords = 2LL * page_size * row_stride;  // K plane + V plane
  uint32_t* kplane = kv_cache + last_pid * page_dwords + h * (HD / 2);
  uint32_t* vplane = kplane + (int64_t)page_size * row_stride;
  const uint32_t kw = k_row[lane];
  const uint32_t vw = v_row[lane];
  kplane[(int64_t)pos * row_stride + lane] = kw;
  vplane[(int64_t)pos * row_stride + lane] = vw;
  if (kbar_page_row != nullptr && pos == page_size - 1 && n_pages - 1 < kbar_pages) {
    float s0 = 0.f, s1 = 0.f;
#pragma unroll 15
    for (int t = 0; t < page_size - 1; ++t) {
      const uint32_t w = kplane[(int64_t)t * row_stride + lane];
      s0 += elem_lo<F16>(w);
      s1 += elem_hi<F16>(w);
    }
    s0 += elem_lo<F16>(kw);
    s1 += elem_hi<F16>(kw);
    const float inv = 1.0f / (float)page_size;
    kbar_page_row[lane] = f32_to_elem<F16>(s0 * inv) | (f32_to_elem<F16>(s1 * inv) << 16);
  }
}

}  // namespace kin
