// Page-table metadata for slot-based caches, as a paged stand-in for a
// contiguous [max_batch, H_kv, max_len, D] cache: each slot either owns a fixed
// run of `pages_per_slot` physical pages (page id = slot * pages_per_slot + p), or
// draws its pages from a pool through a free list kept on the device.  From the
// per-sequence token counts this builds the CSR table the kernels read.
#include "kin_common.h"

namespace kin {

// One 1024-thread workgroup: n_pages, last_page_len and the exclusive scan.
// slot_npages (may be null): pages slot s really owns.  A sequence that its slot cannot hold
// -- longer than pages_per_slot pages, or than the pages the slot owns because a reserve
// failed -- gets an EMPTY page list: the kernels then write nothing for it and return
// zeros, instead of appending into the wrong token slot of a truncated list.  So does a
// sequence whose slot id lies outside [0, max_slots).
__global__ __launch_bounds__(1024) void slot_table_scan_kernel(const int32_t* __restrict__ seq_lens, int batch,
                                                               int pages_per_slot, int page_size,
                                                               int32_t* __restrict__ page_indptr,
                                                               int32_t* __restrict__ last_page_len,
                                                               const int32_t* __restrict__ slot_ids = nullptr,
                                                               const int32_t* __restrict__ slot_npages = nullptr,
                                                               int max_slots = 0x7fffffff) {
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
      n = (len + page_size - 1) / page_size;
      const int slot = slot_ids ? slot_ids[b] : b;
      const bool slot_ok = (unsigned)slot < (unsigned)max_slots;
      const int owned = !slot_ok ? 0 : (slot_npages ? min(slot_npages[slot], pages_per_slot) : pages_per_slot);
      if (n > owned) n = 0;
      last_page_len[b] = (n > 0) ? len - (n - 1) * page_size : 1;
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

// grid = (ceil(pages_per_slot / 256), batch).  slot_table == null: slot s owns the
// fixed run s*pages_per_slot ..; else page p of slot s is slot_table[s*pages_per_slot + p].
__global__ __launch_bounds__(256) void slot_table_fill_kernel(const int32_t* __restrict__ slot_ids,
                                                              const int32_t* __restrict__ page_indptr,
                                                              const int32_t* __restrict__ slot_table,
                                                              int pages_per_slot, int32_t* __restrict__ page_indices) {
  const int b = blockIdx.y;
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int s = page_indptr[b], n = page_indptr[b + 1] - s;
  if (p >= n) return;
  const int slot = slot_ids ? slot_ids[b] : b;  // (in range: the scan gave other sequences an empty list)
  const int64_t e = (int64_t)slot * pages_per_slot + p;
  page_indices[s + p] = slot_table ? slot_table[e] : (int32_t)e;
}

// ---- page pool: a free list on the device -------------------------------------
// pool_state[0] = pages on the free stack, pool_state[1] = status bits.
constexpr int kPoolExhausted = 1;   // a reserve call wanted more pages than were free: it reserved nothing
constexpr int kPoolSlotTooLong = 2; // a sequence wanted more than pages_per_slot pages: its slot got pages_per_slot
constexpr int kPoolBadSlot = 4;     // a slot id outside [0, max_slots), or listed twice in one call: that entry was skipped
constexpr int kPoolMark = 1 << 24;  // added to slot_npages[s] while a reserve call checks its ids for repeats

__global__ __launch_bounds__(256) void pool_init_kernel(int32_t* __restrict__ free_stack, int32_t* __restrict__ pool_state,
                                                        int32_t* __restrict__ slot_npages, int num_pool_pages,
                                                        int max_slots) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < num_pool_pages) free_stack[i] = num_pool_pages - 1 - i;  // pops hand out 0, 1, 2, ...
  if (i < max_slots) slot_npages[i] = 0;
  if (i == 0) {
    pool_state[0] = num_pool_pages;
    pool_state[1] = 0;
  }
}

// Sum over the workgroup's 1024 threads; every thread gets it.  `red` holds 16 ints.
__device__ __forceinline__ int block_sum_1024(int x, int* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off);
  __syncthreads();  // red may still be read from a previous call
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
  __syncthreads();
  int t = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) t += red[w];
  return t;
}

// One 1024-thread workgroup grows every listed slot to ceil(seq_lens[b] / page_size)
// pages (never shrinks one), all or nothing: if the free stack cannot cover the
// whole call, nothing is reserved and kPoolExhausted is raised.  Entries whose slot id is
// out of range, or that name a slot an earlier entry of the same call named, are skipped
// (kPoolBadSlot): every entry first adds kPoolMark to its slot's page count, and whoever
// finds the mark already there is a repeat.
__global__ __launch_bounds__(1024) void pool_reserve_kernel(const int32_t* __restrict__ slot_ids,
                                                            const int32_t* __restrict__ seq_lens, int batch,
                                                            int pages_per_slot, int page_size,
                                                            int32_t* __restrict__ slot_table,
                                                            int32_t* __restrict__ slot_npages,
                                                            const int32_t* __restrict__ free_stack,
                                                            int32_t* __restrict__ pool_state, int max_slots) {
  __shared__ int red[16];
  __shared__ int wave_sum[16];
  __shared__ int carry_sh;
  __shared__ uint32_t skip_bits[2048];  // one bit per entry of the call (batch <= 65535)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 2048; i += 1024) skip_bits[i] = 0;
  __syncthreads();
  int bad = 0;
  for (int b = tid; b < batch; b += 1024) {
    const int slot = slot_ids ? slot_ids[b] : b;
    bool skip = (unsigned)slot >= (unsigned)max_slots;
    if (!skip) skip = atomicAdd(&slot_npages[slot], kPoolMark) >= kPoolMark;
    if (skip) {
      atomicOr(&skip_bits[b >> 5], 1u << (b & 31));
      bad = 1;
    }
  }
  __syncthreads();
  auto skipped = [&](int b) -> bool { return (skip_bits[b >> 5] >> (b & 31)) & 1u; };
  auto demand = [&](int b, int& slot, int& have) -> int {
    slot = slot_ids ? slot_ids[b] : b;
    if (skipped(b)) {
      have = 0;
      return 0;
    }
    have = slot_npages[slot] & (kPoolMark - 1);
    const int len = max(seq_lens[b], 0);
    const int need = min((len + page_size - 1) / page_size, pages_per_slot);
    return max(need - have, 0);
  };
  int mine = 0, too_long = 0;
  for (int b = tid; b < batch; b += 1024) {
    int slot, have;
    mine += demand(b, slot, have);
    too_long |= (max(seq_lens[b], 0) > pages_per_slot * page_size) ? 1 : 0;
  }
  const int total = block_sum_1024(mine, red);
  const int any_long = block_sum_1024(too_long, red);
  const int any_bad = block_sum_1024(bad, red);
  const int free_top = pool_state[0];
  __syncthreads();  // everybody has read free_top before thread 0 may change it
  if (tid == 0 && (any_long || any_bad || total > free_top))
    pool_state[1] |= (any_long ? kPoolSlotTooLong : 0) | (any_bad ? kPoolBadSlot : 0) | (total > free_top ? kPoolExhausted : 0);
  const bool grow = total <= free_top && total > 0;
  if (tid == 0) carry_sh = 0;
  __syncthreads();
  for (int base = 0; base < batch; base += 1024) {
    const int b = base + tid;
    int slot = 0, have = 0, extra = 0;
    const bool live = b < batch && !skipped(b);
    if (b < batch) extra = demand(b, slot, have);
    if (!grow) extra = 0;
    int incl = extra;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry_sh;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    const int first = before + incl - extra;  // this slot takes entries first .. first+extra-1 from the top
    for (int j = 0; j < extra; ++j)
      slot_table[(int64_t)slot * pages_per_slot + have + j] = free_stack[free_top - 1 - (first + j)];
    if (live) slot_npages[slot] = have + extra;  // (also takes the mark off)
    __syncthreads();
    if (tid == 1023) carry_sh = before + incl;
    __syncthreads();
  }
  if (tid == 0 && grow) pool_state[0] = free_top - total;
}

// One 256-thread workgroup pushes the pages of the listed slots back, slot after slot.
__global__ __launch_bounds__(256) void pool_release_kernel(const int32_t* __restrict__ slot_ids, int count,
                                                           int pages_per_slot, const int32_t* __restrict__ slot_table,
                                                           int32_t* __restrict__ slot_npages,
                                                           int32_t* __restrict__ free_stack,
                                                           int32_t* __restrict__ pool_state, int num_pool_pages,
                                                           int max_slots) {
  int top = pool_state[0];
  for (int i = 0; i < count; ++i) {
    const int slot = slot_ids[i];
    if ((unsigned)slot >= (unsigned)max_slots) {  // (uniform: every thread reads the same id)
      if (threadIdx.x == 0) pool_state[1] |= kPoolBadSlot;
      continue;
    }
    const int n = slot_npages[slot];
    __syncthreads();  // everybody has read n before it is cleared
    for (int j = threadIdx.x; j < n; j += 256)
      if (top + j < num_pool_pages) free_stack[top + j] = slot_table[(int64_t)slot * pages_per_slot + j];
    if (threadIdx.x == 0) slot_npages[slot] = 0;
    top = min(top + n, num_pool_pages);
    __syncthreads();  // a slot listed twice is empty the second time
  }
  __syncthreads();
  if (threadIdx.x == 0) pool_state[0] = top;
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
  slot_table_fill_kernel<<<grid, 256, 0, s>>>(slot_ids, page_indptr, nullptr, pages_per_slot, page_indices);
  return check_hip(hipGetLastError(), "slot_table_fill_kernel launch");
}

extern "C" int kin_page_pool_init(int32_t* free_stack, int32_t* pool_state, int32_t* slot_npages,
                                  int num_pool_pages, int max_slots, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_page_pool_init";
  if (!free_stack || !pool_state || !slot_npages) return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (num_pool_pages < 1 || max_slots < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: num_pool_pages=%d max_slots=%d must be >= 1", fn, num_pool_pages, max_slots);
  const int n = num_pool_pages > max_slots ? num_pool_pages : max_slots;
  pool_init_kernel<<<(unsigned)((n + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(free_stack, pool_state,
                                                                                              slot_npages, num_pool_pages,
                                                                                              max_slots);
  return check_hip(hipGetLastError(), "pool_init_kernel launch");
}

extern "C" int kin_page_pool_reserve(const int32_t* slot_ids, const int32_t* seq_lens, int batch,
                                     int pages_per_slot, int page_size, int32_t* slot_table, int32_t* slot_npages,
                                     const int32_t* free_stack, int32_t* pool_state, int max_slots,
                                     kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_page_pool_reserve";
  if (!seq_lens || !slot_table || !slot_npages || !free_stack || !pool_state)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (batch < 0 || pages_per_slot < 1 || page_size < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: batch=%d pages_per_slot=%d page_size=%d", fn, batch, pages_per_slot, page_size);
  if (batch > 65535) return fail(KIN_ERR_UNSUPPORTED, "%s: batch=%d exceeds 65535", fn, batch);
  if (max_slots < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: max_slots=%d must be >= 1", fn, max_slots);
  if (pages_per_slot >= kPoolMark) return fail(KIN_ERR_UNSUPPORTED, "%s: pages_per_slot=%d exceeds %d", fn, pages_per_slot, kPoolMark - 1);
  if (!slot_ids && batch > max_slots)
    return fail(KIN_ERR_BAD_SHAPE, "%s: batch=%d sequences but only max_slots=%d slots", fn, batch, max_slots);
  if (batch == 0) return KIN_OK;
  pool_reserve_kernel<<<1, 1024, 0, static_cast<hipStream_t>(stream)>>>(slot_ids, seq_lens, batch, pages_per_slot, page_size,
                                                                       slot_table, slot_npages, free_stack, pool_state, max_slots);
  return check_hip(hipGetLastError(), "pool_reserve_kernel launch");
}

extern "C" int kin_page_pool_release(const int32_t* slot_ids, int count, int pages_per_slot,
                                     const int32_t* slot_table, int32_t* slot_npages, int32_t* free_stack,
                                     int32_t* pool_state, int num_pool_pages, int max_slots, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_page_pool_release";
  if (!slot_ids || !slot_table || !slot_npages || !free_stack || !pool_state)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (count < 0 || pages_per_slot < 1 || num_pool_pages < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: count=%d pages_per_slot=%d num_pool_pages=%d", fn, count, pages_per_slot,
                num_pool_pages);
  if (max_slots < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: max_slots=%d must be >= 1", fn, max_slots);
  if (count == 0) return KIN_OK;
  pool_release_kernel<<<1, 256, 0, static_cast<hipStream_t>(stream)>>>(slot_ids, count, pages_per_slot, slot_table,
                                                                      slot_npages, free_stack, pool_state, num_pool_pages,
                                                                      max_slots);
  return check_hip(hipGetLastError(), "pool_release_kernel launch");
}

extern "C" int kin_build_pool_page_table(const int32_t* slot_ids, const int32_t* seq_lens, int batch,
                                         int pages_per_slot, int page_size, const int32_t* slot_table,
                                         const int32_t* slot_npages, int32_t* page_indices, int32_t* page_indptr,
                                         int32_t* last_page_len, int max_slots, kin_stream_t stream) {
  using namespace kin;
  const char* fn = "kin_build_pool_page_table";
  if (!seq_lens || !slot_table || !slot_npages || !page_indices || !page_indptr || !last_page_len)
    return fail(KIN_ERR_NULL_POINTER, "%s: null pointer argument", fn);
  if (batch < 0 || pages_per_slot < 1 || page_size < 1)
    return fail(KIN_ERR_BAD_SHAPE, "%s: batch=%d pages_per_slot=%d page_size=%d", fn, batch, pages_per_slot, page_size);
  if (batch > 65535) return fail(KIN_ERR_UNSUPPORTED, "%s: batch=%d exceeds 65535", fn, batch);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (batch == 0) {
    fill_zero_i32_kernel<<<1, 64, 0, s>>>(page_indptr, 1);
    return check_hip(hipGetLastError(), "fill_zero_i32_kernel launch");
  }
  if (max_slots < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: max_slots=%d must be >= 1", fn, max_slots);
  slot_table_scan_kernel<<<1, 1024, 0, s>>>(seq_lens, batch, pages_per_slot, page_size, page_indptr, last_page_len, slot_ids,
                                            slot_npages, max_slots);
  int st = check_hip(hipGetLastError(), "slot_table_scan_kernel launch");
  if (st) return st;
  dim3 grid((unsigned)((pages_per_slot + 255) / 256), (unsigned)batch);
  slot_table_fill_kernel<<<grid, 256, 0, s>>>(slot_ids, page_indptr, slot_table, pages_per_slot, page_indices);
  return check_hip(hipGetLastError(), "slot_table_fill_kernel launch");
}
