// Status handling, shared argument checks and the page-table checker.
#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "kin_common.h"
#include "kin_step.h"

namespace kin {

static std::atomic<int> g_team_spin_limit{kTeamSpinLimit};
int team_spin_limit() { return g_team_spin_limit.load(std::memory_order_relaxed); }

static thread_local char g_last_error[512] = {0};

int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return status;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return KIN_OK;
  return fail(KIN_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

int check_common_dims(const char* fn, int batch, int num_q_heads, int num_kv_heads,
                      int head_dim, int page_size, bool small_head_dim_built) {
  if (batch < 0) return fail(KIN_ERR_BAD_SHAPE, "%s: batch=%d is negative", fn, batch);
  if (num_kv_heads < 1) return fail(KIN_ERR_BAD_SHAPE, "%s: num_kv_heads=%d must be >= 1", fn, num_kv_heads);
  if (num_q_heads < 1 || num_q_heads % num_kv_heads != 0)
    return fail(KIN_ERR_BAD_SHAPE, "%s: num_q_heads=%d must be a positive multiple of num_kv_heads=%d", fn,
                num_q_heads, num_kv_heads);
  if (head_dim <= 0 || page_size <= 0)
    return fail(KIN_ERR_BAD_SHAPE, "%s: head_dim=%d and page_size=%d must be positive", fn, head_dim, page_size);
  if (head_dim != kHeadDim && !(small_head_dim_built && head_dim == kHeadDimSmall))
    return fail(KIN_ERR_UNSUPPORTED, "%s: head_dim=%d unsupported (kernels are built for %s%d)", fn, head_dim,
                small_head_dim_built ? "64 and " : "", kHeadDim);
  if (!supported_page_size(page_size))
    return fail(KIN_ERR_UNSUPPORTED, "%s: page_size=%d unsupported (kernels are built for 16, 32, 64 and 128)", fn, page_size);
  if (num_q_heads / num_kv_heads > kMaxGroup)
    return fail(KIN_ERR_UNSUPPORTED, "%s: GQA group %d unsupported (max %d)", fn, num_q_heads / num_kv_heads,
                kMaxGroup);
  return KIN_OK;
}

int check_fixed_pages(const char* fn, int sink_pages, int local_tokens) {
  if (sink_pages < 0 || sink_pages > kMaxFixedPages || local_tokens < 1 || local_tokens > kMaxLocalTokens)
    return fail(KIN_ERR_BAD_SHAPE, "%s: sink_pages=%d must be in [0, %d] and local_tokens=%d in [1, %d]", fn, sink_pages,
                kMaxFixedPages, local_tokens, kMaxLocalTokens);
  return KIN_OK;
}

int check_first_page_offset(const char* fn, int first_page_offset, int page_size) {
  if (first_page_offset < 0 || first_page_offset >= page_size)
    return fail(KIN_ERR_BAD_SHAPE, "%s: first_page_offset=%d must be in [0, page_size=%d)", fn, first_page_offset, page_size);
  return KIN_OK;
}

int check_page_size_16(const char* fn, int page_size) {
  if (page_size != kPageSize)
    return fail(KIN_ERR_UNSUPPORTED, "%s: page_size=%d unsupported (the token-granular policies are built for %d)", fn,
                page_size, kPageSize);
  return KIN_OK;
}

// One thread per sequence checks its indptr step, last_page_len and page ids.
__global__ void check_page_table_kernel(const int32_t* __restrict__ page_indices,
                                        const int32_t* __restrict__ page_indptr,
                                        const int32_t* __restrict__ last_page_len, int batch, int page_size,
                                        int64_t num_pages, int64_t nnz, int32_t* __restrict__ bad) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch) return;
  int errs = 0;
  const int s = page_indptr[b], e = page_indptr[b + 1];
  if (b == 0 && s != 0) errs++;
  if (e < s || s < 0 || (int64_t)e > nnz) {
    errs++;
  } else {
    if (e > s) {
      const int ll = last_page_len[b];
      if (ll < 1 || ll > page_size) errs++;
    }
    for (int i = s; i < e; ++i) {
      const int id = page_indices[i];
      if (id < 0 || (int64_t)id >= num_pages) errs++;
    }
  }
  if (errs) atomicAdd(bad, errs);
}

}  // namespace kin

extern "C" {

int kin_version(void) { return 30200; }

int kin_set_team_spin_limit(int polls) {
  return kin::g_team_spin_limit.exchange(polls < 0 ? kin::kTeamSpinLimit : polls, std::memory_order_relaxed);
}

int kin_sel_list_capacity(int topk, int sink_pages, int local_tokens) {
  if (topk < 0 || sink_pages < 0 || local_tokens < 1) return 0;
  return topk + sink_pages + kin::max_local_pages(local_tokens);
}

const char* kin_last_error(void) { return kin::g_last_error; }

const char* kin_status_string(int status) {
  switch (status) {
    case KIN_OK: return "KIN_OK";
    case KIN_ERR_NULL_POINTER: return "KIN_ERR_NULL_POINTER";
    case KIN_ERR_BAD_SHAPE: return "KIN_ERR_BAD_SHAPE";
    case KIN_ERR_UNSUPPORTED: return "KIN_ERR_UNSUPPORTED";
    case KIN_ERR_WORKSPACE: return "KIN_ERR_WORKSPACE";
    case KIN_ERR_LAUNCH: return "KIN_ERR_LAUNCH";
    case KIN_ERR_PAGE_TABLE: return "KIN_ERR_PAGE_TABLE";
    case KIN_ERR_MISALIGNED: return "KIN_ERR_MISALIGNED";
    default: return "KIN_ERR_UNKNOWN";
  }
}

int kin_check_page_table(const int32_t* page_indices, const int32_t* page_indptr, const int32_t* last_page_len,
                         int batch, int page_size, int64_t num_pages, int64_t nnz, int32_t* scratch,
                         kin_stream_t stream) {
  using namespace kin;
  if (!page_indices || !page_indptr || !last_page_len || !scratch)
    return fail(KIN_ERR_NULL_POINTER, "kin_check_page_table: null pointer argument");
  if (batch < 0 || page_size <= 0 || num_pages < 0 || nnz < 0)
    return fail(KIN_ERR_BAD_SHAPE, "kin_check_page_table: batch=%d page_size=%d num_pages=%lld nnz=%lld", batch,
                page_size, (long long)num_pages, (long long)nnz);
  if (batch == 0) return KIN_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int32_t zero = 0, bad = 0;
  int st = check_hip(hipMemcpyAsync(scratch, &zero, sizeof(zero), hipMemcpyHostToDevice, s), "clear scratch");
  if (st) return st;
  st = check_hip(hipStreamSynchronize(s), "sync");  // `zero` is a stack variable
  if (st) return st;
  const int threads = 256;
  check_page_table_kernel<<<(batch + threads - 1) / threads, threads, 0, s>>>(page_indices, page_indptr,
                                                                            last_page_len, batch, page_size,
                                                                            num_pages, nnz, scratch);
  st = check_hip(hipGetLastError(), "check_page_table_kernel launch");
  if (st) return st;
  st = check_hip(hipMemcpyAsync(&bad, scratch, sizeof(bad), hipMemcpyDeviceToHost, s), "read scratch");
  if (st) return st;
  st = check_hip(hipStreamSynchronize(s), "sync");
  if (st) return st;
  if (bad != 0) return fail(KIN_ERR_PAGE_TABLE, "kin_check_page_table: %d invalid page-table entries", bad);
  return KIN_OK;
}

}  // extern "C"
