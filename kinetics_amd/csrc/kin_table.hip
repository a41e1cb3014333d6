// Page-table metadata for slot-based caches: each slot owns a fixed run of
// `pages_per_slot` physical pages (page id = slot * pages_per_slot + p), as a
// paged stand-in for a contiguous [max_batch, H_kv, max_len, D] cache.  From
// the per-sequence token counts this builds the CSR table the kernels read.
#include "kin_common.h"

namespace kin {

// One 1024-thread workgroup: n_pages, last_page_len and the exclusive scan.
__global__ __launch_bounds__(1024) void slot_table_scan_kernel(const int32_t* __restrict__ seq_lens, int batch,
                                                               int pages_per_slot, int page_size,
                                                               int32_t* __restrict__ page_indptr,
                                                               int32_t* __restrict__ last_page_len) {
  __shared__ int wave_sum[16];
  __shared__ int carry_sh;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) {
    carry_sh = 0;
    page_indptr[0] = 0;
  }
  __syncthreads();
  for (int base = 0; base < batch; base += 1024) {
    const int b = base + tid;
    int n = 0;
    if (b < batch) {
      const int len = max(seq_lens[b], 0);
      n = min((len + page_size - 1) / page_size, pages_per_slot);
      const int tokens = min(len, n * page_size);
      last_page_len[b] = (n > 0) ? tokens - (n - 1) * page_size : 1;
    }
    int incl = n;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry_sh;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    if (b < batch) page_indptr[b + 1] = before + incl;
    __syncthreads();
    if (tid == 1023) carry_sh = before + incl;
    __syncthreads();
  }
}

// grid = (ceil(pages_per_slot / 256), batch)
__global__ __launch_bounds__(256) void slot_table_fill_kernel(const int32_t* __restrict__ slot_ids,
                                                              const int32_t* __restrict__ page_indptr,
                                                              int pages_per_slot, int32_t* __restrict__ page_indices) {
  const int b = blockIdx.y;
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int s = page_indptr[b], n = page_indptr[b + 1] - s;
  if (p >= n) return;
  const int slot = slot_ids ? slot_ids[b] : b;
  page_indices[s + p] = slot * pages_per_slot + p;
}

}  // namespace kin

extern "C" int kin_build_slot_page_table(const int32_t* slot_ids, const int32_t* seq_lens, int batch,
                                         int pages_per_slot, int page_size, int32_t* page_indices,
                                         int32_t* page_indptr, int32_t* last_page_len, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_build_slot_page_table";
  if (!seq_lens || !page_indices || !page_indptr || !last_page_len)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (batch < 0 || pages_per_slot < 1 || page_size < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: batch=%d pages_per_slot=%d page_size=%d", fn, batch, pages_per_slot, page_size);
  if (batch > 65535) return fail(KIN_ERR_UNSUPPORTED, "%s: batch=%d exceeds 65535", fn, batch);
  if ((int64_t)batch * pages_per_slot > 0x7fffffffLL)
    return fail(KIN_ERR_UNSUPPORTED, "%s: batch*pages_per_slot overflows int32 page ids", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (batch == 0) {
    // nothing to fill, but indptr[0] must still be valid
    fill_zero_i32_kernel<<<1, 64, 0, s>>>(page_indptr, 1);
    return check_hip(hipGetLastError(), "fill_zero_i32_kernel launch");
  }
  slot_table_scan_kernel<<<1, 1024, 0, s>>>(seq_lens, batch, pages_per_slot, page_size, page_indptr, last_page_len);
  int st = check_hip(hipGetLastError(), "slot_table_scan_kernel launch");
  if (st) return st;
  dim3 grid((unsigned)((pages_per_slot + 255) / 256), (unsigned)batch);
  slot_table_fill_kernel<<<grid, 256, 0, s>>>(slot_ids, page_indptr, pages_per_slot, page_indices);
  return check_hip(hipGetLastError(), "slot_table_fill_kernel launch");
}
