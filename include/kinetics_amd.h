/*
 * kinetics_amd.h -- C ABI of the MI355X (gfx950) block top-k sparse paged
 * decode-attention path.
 *
 * Every entry point is extern "C", takes plain device pointers and sizes,
 * returns an int status (KIN_OK == 0), never throws, never allocates or frees
 * device memory and never synchronises the device (kin_check_page_table, a
 * debugging aid, is the one documented exception).  All work is enqueued on
 * the HIP stream passed as the last argument (NULL = the default stream).
 *
 * Citations "ref:" are file:line in the Infini-AI-Lab/Kinetics tree and name
 * the reference interface each entry point stands in for.
 *
 * Tensor conventions (all device memory, densely packed, row-major):
 *   bf16 tensors are passed as uint16_t* (raw bfloat16 bit patterns); the
 *   *_f16 entry points near the end take IEEE binary16 bits the same way.
 *   q, out        [batch, num_q_heads, head_dim]                    bf16
 *   k, v          [batch, num_kv_heads, head_dim]                   bf16
 *   kv_cache      [num_pages, 2, page_size, num_kv_heads, head_dim] bf16
 *                 ("NHD" paged layout, K plane then V plane per page;
 *                  ref: benchmark/blocktopk_decoder.py:161-164)
 *   kbar          [batch, num_kv_heads, kbar_pages, head_dim]       bf16
 *                 per-page representative (mean) key, indexed by LOGICAL page,
 *                 head-major: the candidates of one (sequence, KV head) are one
 *                 contiguous run of rows.  With one KV head this is the
 *                 reference's compressed_key_cache [batch, pages, head_dim]
 *                 (ref: benchmark/blocktopk_decoder.py:165-168, which asserts
 *                 one KV head).
 *   page_indices  [nnz] int32, page_indptr [batch+1] int32,
 *   last_page_len [batch] int32 in [1, page_size]
 *                 CSR page table: sequence b owns physical pages
 *                 page_indices[page_indptr[b] : page_indptr[b+1]] in logical
 *                 order and holds (n_pages-1)*page_size + last_page_len[b]
 *                 tokens (ref: benchmark/blocktopk_decoder.py:141-149).
 *   sel_pages     [batch, num_kv_heads, sel_stride] int32 physical page ids,
 *   sel_count     [batch, num_kv_heads] int32
 *                 per-(sequence, KV head) list of pages to attend to; the
 *                 final entry is always the sequence's last page
 *                 (ref: benchmark/blocktopk_decoder.py:143,217-221).
 *
 * Supported shapes: head_dim 128 or 64 (the reference reads it from the model
 * config, benchmark/blocktopk_decoder.py:104); page_size 16, 32, 64 or 128
 * (the reference's --page_size, benchmark/blocktopk.py:13; the token-granular
 * policies: 16 only);
 * num_q_heads % num_kv_heads == 0 and group size num_q_heads/num_kv_heads <= 16.
 * Where a comment below says "16" for a page it means page_size.
 */
#ifndef KINETICS_AMD_H
#define KINETICS_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t kin_bf16_t;  /* raw bfloat16 bits */
typedef uint16_t kin_f16_t;   /* raw IEEE binary16 bits */
typedef void* kin_stream_t;   /* a hipStream_t */

enum kin_status {
  KIN_OK = 0,
  KIN_ERR_NULL_POINTER = 1,  /* a required pointer argument is NULL */
  KIN_ERR_BAD_SHAPE = 2,     /* a size argument is out of range / inconsistent */
  KIN_ERR_UNSUPPORTED = 3,   /* valid request outside the compiled fast paths */
  KIN_ERR_WORKSPACE = 4,     /* workspace missing or too small */
  KIN_ERR_LAUNCH = 5,        /* the HIP runtime refused a launch / call */
  KIN_ERR_PAGE_TABLE = 6,    /* kin_check_page_table found an invalid entry */
  KIN_ERR_MISALIGNED = 7     /* a tensor pointer is not 16-byte aligned */
};

/* Library version (major*10000 + minor*100 + patch).  2.0.0: mean keys are stored
 * head-major ([batch, num_kv_heads, kbar_pages, 128]; 1.x had [batch, kbar_pages,
 * num_kv_heads, 128]), kin_block_score_topk takes the page size, pages of 32 and 64
 * tokens, float16 twins (kin_*_f16), groups of up to 16 query heads per KV head,
 * the page pool and kin_blocktopk_decode_step_static.  2.1.0: the decode step
 * attends few lists in parts (kin_step_workspace_bytes grows to up to 2.1 MB for
 * up to 128 lists; KIN_STATIC_SCRATCH_BYTES grows by 32 KiB less 256 B).  2.2.0:
 * few lists are handled by teams of workgroups that share the scoring and the
 * attention (kin_step_workspace_bytes covers keys and partial results;
 * KIN_STATIC_SCRATCH_BYTES doubles); without sel_pages the step attends the
 * winners in index order.  3.0.0: every entry point that touches kbar takes
 * slot_ids / num_slots in front of the stream (kbar laid out by cache slot).
 * 3.1.0: head_dim 64 in the page path (append, mean keys, selector, sparse and
 * dense decode, the fused step), in kin_qkv_norm_split and, for rows of 64
 * elements, in kin_rms_norm.  3.2.0: head_dim 64 in the token-granular
 * policies, pages of 128 tokens, teams (the fused step) or a launch of their
 * own (the token-granular policies) for the lists that a batch has beyond a
 * multiple of 256. */
int kin_version(void);

/* Human-readable text of the last non-OK status on the calling thread
 * (thread-local; empty string if none). */
const char* kin_last_error(void);

/* Static name of a status code ("KIN_OK", "KIN_ERR_BAD_SHAPE", ...). */
const char* kin_status_string(int status);

/*
 * (1) Paged KV append -- replaces mylib::update_kv ->
 * flashinfer.append_paged_kv_cache (ref: benchmark/blocktopk_decoder.py:23-46,
 * 209-213; semantics of LiteSys copy_to_cache,
 * ref: LiteSys/litesys/attention/cache_utils.py:5-51).
 *
 * The page table describes the cache AFTER the append: the new token of
 * sequence b is written at slot last_page_len[b]-1 of its last page.  When
 * that write fills the page (last_page_len[b] == page_size) and kbar != NULL,
 * kbar[b, h, n_pages-1, :] is set to the mean of the page's page_size keys
 * (fp32 sum in slot order, times 1/page_size, round-to-nearest-even to bf16).
 * Sequences with an empty page list are skipped.  kbar may be NULL.
 *
 * slot_ids / num_slots (here and in every entry point that touches kbar): the
 * reference's kernels take batch_idx and index the cache by slot while q, k, v
 * and the output follow the position in the active batch
 * (ref: LiteSys/litesys/attention/cache_utils.py:40-51,67-70,
 * LiteSys/litesys/attention/batch_cache.py:76-110).  Here the page table is
 * already per active sequence, so the one tensor left that is laid out by slot is
 * kbar: with slot_ids != NULL (int32 [batch], on the device), sequence b's mean
 * keys are kbar[slot_ids[b], ...] and kbar has num_slots row blocks; a sequence
 * whose id lies outside [0, num_slots) has no mean keys (nothing is written for
 * it, and it has no candidate pages).  slot_ids == NULL: kbar[b, ...], num_slots
 * is ignored.  Two sequences of one call must not share a slot.
 */
int kin_append_paged_kv(const kin_bf16_t* k, const kin_bf16_t* v,
                        kin_bf16_t* kv_cache, kin_bf16_t* kbar,
                        const int32_t* page_indices, const int32_t* page_indptr,
                        const int32_t* last_page_len,
                        int batch, int num_kv_heads, int head_dim, int page_size,
                        int64_t num_pages, int kbar_pages,
                        const int32_t* slot_ids, int num_slots, kin_stream_t stream);

/*
 * Representative keys for every FULL page of every sequence (what a prefill
 * has to leave behind for the scorer).  The reference fills
 * compressed_key_cache with random numbers and never maintains it
 * (ref: benchmark/blocktopk_decoder.py:166-168); this is the missing producer.
 * Same arithmetic as the append-time update.
 */
int kin_build_kbar(const kin_bf16_t* kv_cache, kin_bf16_t* kbar,
                   const int32_t* page_indices, const int32_t* page_indptr,
                   const int32_t* last_page_len,
                   int batch, int num_kv_heads, int head_dim, int page_size,
                   int64_t num_pages, int kbar_pages,
                   const int32_t* slot_ids, int num_slots, kin_stream_t stream);

/*
 * Ragged multi-token append -- the general form of
 * flashinfer.append_paged_kv_cache behind mylib::update_kv, whose signature
 * carries kv_append_indptr (ref: benchmark/blocktopk_decoder.py:23-46), and the
 * paged counterpart of LiteSys' prefill write
 * (ref: LiteSys/litesys/attention/batch_cache.py:112-131).
 *
 * k, v: [nnz, num_kv_heads, head_dim]; sequence b appends the rows
 * append_indptr[b] .. append_indptr[b+1]-1 (n_b of them).  The page table
 * describes the cache AFTER the append: row i of sequence b lands at token
 * position kv_len_b - n_b + i, kv_len_b = 16*(n_pages_b-1) + last_page_len[b].
 * When kbar is given, the mean key of every page the append completed is
 * (re)computed, with the arithmetic of kin_append_paged_kv.  max_append_len is
 * an upper bound on n_b, 0 <= max_append_len <= nnz (checked; the launches are
 * sized by nnz alone, so nnz is as good a value as any).  Sequences whose
 * metadata is out of contract are skipped.
 */
int kin_append_paged_kv_ragged(const kin_bf16_t* k, const kin_bf16_t* v,
                               const int32_t* append_indptr,
                               kin_bf16_t* kv_cache, kin_bf16_t* kbar,
                               const int32_t* page_indices, const int32_t* page_indptr,
                               const int32_t* last_page_len,
                               int batch, int64_t nnz, int max_append_len,
                               int num_kv_heads, int head_dim, int page_size,
                               int64_t num_pages, int kbar_pages,
                               const int32_t* slot_ids, int num_slots, kin_stream_t stream);

/*
 * (2)+(3) Page scoring and top-k page selection, fused -- replaces
 *   csim = einsum("b g d, b n d -> b g n", q, kbar).mean(1); topk(csim, k);
 *   logical->physical translation; cat(last page)
 * (ref: benchmark/blocktopk_decoder.py:216-221) and, per KV head, LiteSys
 * blockwise_topk_sparsity (ref: LiteSys/litesys/attention/sparsity_utils.py:24-47).
 *
 * With kv_len = 16*(n_pages-1) + last_page_len[b], the pages of sequence b
 * split into
 *   n_sink  = min(sink_pages, n_pages-1) leading pages, always attended,
 *   n_cand  = max(0, floor((kv_len - 16*n_sink - local_tokens) / 16)) candidate
 *             pages after them (the whole pages that lie before the newest
 *             local_tokens tokens), and
 *   n_local = n_pages - n_sink - n_cand trailing pages, always attended; the
 *             open page is one of them (local_tokens >= 1), even when full.
 * sink_pages = 0, local_tokens = 1 is the reference's rule ("top-k plus the
 * last page", blocktopk_decoder.py:220); local_tokens = 16*(L-1)+1 pins exactly
 * the last L pages.  sink_pages = 1 with the sequences stored 12 slots into
 * their first page (see first_page_offset below) and local_tokens = LiteSys'
 * `local` reproduces blockwise_topk_sparsity with its hard-wired 4 sink tokens
 * and 16-token blocks that start at token 4 (sparsity_utils.py:24-35).
 * score[p] = dot(mean_g q[b, h*G+g, :], kbar[b, h, p, :]) in fp32.
 * k_eff = min(topk, n_cand) candidates are selected: descending score, equal
 * scores by ascending logical index (deterministic).
 * Outputs, with n = n_sink + k_eff + n_local:
 *   sel_pages[b,h,0:n_sink]          physical ids of the sink pages
 *   sel_pages[b,h,n_sink:n_sink+k_eff]  the selected pages, in that order
 *   sel_pages[b,h,n_sink+k_eff:n]    the local pages (the open page last)
 *   sel_pages[b,h,n:]        -1
 *   sel_count[b,h]           n   (0 for an empty page list)
 *   sel_logical[b,h,0:k_eff] logical page indices (== n_sink +
 *                            torch.topk(...).indices), stride topk; may be NULL
 *   scores_out[b,h,p]        fp32 score of candidate page p (logical index),
 *                            stride kbar_pages; may be NULL (debug/parity only:
 *                            costs an HBM write)
 * Only logical pages below kbar_pages have a mean key: candidates at or beyond
 * kbar_pages are never selected (size kbar for the longest sequence).
 * Requires topk >= 0 (0: sink and local pages only, no key is read),
 * 0 <= sink_pages <= 64, 1 <= local_tokens <= 1009,
 * sel_stride >= kin_sel_list_capacity(topk, sink_pages, local_tokens),
 * topk <= 2048, kbar_pages <= 16384.
 * workspace: optional (NULL / 0 allowed), kin_step_workspace_bytes(batch,
 * num_kv_heads, kbar_pages) bytes, 16-byte aligned, any contents.  With it, few
 * long lists (that function returns non-zero for them) are scored by several
 * workgroups per list, which meet through this memory; a small kernel that zeroes
 * its counters is then launched first on the same stream.  Results do not depend
 * on it.
 */
int kin_block_score_topk(const kin_bf16_t* q, const kin_bf16_t* kbar,
                         const int32_t* page_indices, const int32_t* page_indptr,
                         const int32_t* last_page_len,
                         int topk, int sink_pages, int local_tokens,
                         int32_t* sel_pages, int32_t* sel_count,
                         int32_t* sel_logical, float* scores_out,
                         int batch, int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                         int kbar_pages, int sel_stride,
                         void* workspace, size_t workspace_bytes,
                         const int32_t* slot_ids, int num_slots, kin_stream_t stream);

/*
 * Longest page list the selector can write for these settings:
 * topk + sink_pages + 1 + ceil((local_tokens - 1) / 16) (the bound for 16-token
 * pages; larger pages never need more).  0 for arguments out of range.
 */
int kin_sel_list_capacity(int topk, int sink_pages, int local_tokens);

/*
 * Bytes of workspace kin_sparse_paged_decode / kin_dense_paged_decode need for
 * the given problem when num_splits is chosen automatically (0) or forced.
 * max_pages_per_list is an upper bound on any list length (sel_stride, or the
 * longest sequence's page count).  Returns 0 when no workspace is needed.
 */
size_t kin_decode_workspace_bytes(int batch, int num_q_heads, int num_kv_heads,
                                  int head_dim, int max_pages_per_list,
                                  int num_splits);

/* The split count the decode entry points use for num_splits == 0. */
int kin_decode_auto_splits(int batch, int num_kv_heads, int max_pages_per_list);

/*
 * (4) Sparse paged gather-attention -- replaces mylib::decode ->
 * flashinfer BatchDecodeWithPagedKVCacheWrapper.run over the k+1 listed pages
 * (ref: benchmark/blocktopk_decoder.py:171-184,223-225,255-265: NHD layout,
 * no positional encoding, sm_scale = 1/sqrt(head_dim) by default).
 *
 * out[b, hq, :] = softmax(sm_scale * q[b,hq,:] . K[tokens]) V[tokens] over the
 * tokens of the pages sel_pages[b,h,0:sel_count[b,h]], h = hq / G; every listed
 * page is full except the final one, which holds last_page_len[b] tokens.
 * Accumulation in fp32, output bf16.  lse (may be NULL) receives the natural-log
 * sum-exp of the scaled logits, [batch, num_q_heads] fp32.  sm_scale <= 0 means
 * 1/sqrt(head_dim).  num_splits: 0 = automatic, else the number of split-K
 * partitions per list (>1 needs workspace, see kin_decode_workspace_bytes).
 * An empty list yields out = 0, lse = -inf.
 * first_page_offset (0 .. page_size-1): the first that many token slots of the FIRST listed
 * page of every list hold no token and are skipped -- for caches that store
 * each sequence shifted into its first page so that pages line up with blocks
 * that do not start at token 0 (LiteSys' blocks start after 4 sink tokens,
 * sparsity_utils.py:24-35: offset page_size - 4, i.e. 12 for its default blocks of 16).  The offset is applied to list entry 0,
 * which is the sequence's first page only if the list was made with
 * sink_pages >= 1 (kin_block_score_topk then lists the first page first) or
 * the sequence has a single page: a caller that passes first_page_offset > 0
 * must have selected with sink_pages >= 1 (kin_blocktopk_decode_step checks
 * this pairing; here the list's origin is unknown and nothing can be checked).
 */
int kin_sparse_paged_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache,
                            const int32_t* sel_pages, const int32_t* sel_count,
                            const int32_t* last_page_len,
                            kin_bf16_t* out, float* lse,
                            void* workspace, size_t workspace_bytes,
                            int batch, int num_q_heads, int num_kv_heads,
                            int head_dim, int page_size, int64_t num_pages,
                            int sel_stride, int first_page_offset,
                            float sm_scale, int num_splits, kin_stream_t stream);

/*
 * Dense paged decode attention over every page of each sequence -- replaces
 * the dense layer's mylib::decode (ref: benchmark/dense_decoder.py:149-170,
 * 211-219).  Same arithmetic and kernel as kin_sparse_paged_decode; the page
 * list of sequence b is page_indices[page_indptr[b]:page_indptr[b+1]], shared
 * by all KV heads.  max_pages_per_seq bounds the longest list (used only to
 * choose the split count).  first_page_offset as above.
 */
int kin_dense_paged_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache,
                           const int32_t* page_indices, const int32_t* page_indptr,
                           const int32_t* last_page_len,
                           kin_bf16_t* out, float* lse,
                           void* workspace, size_t workspace_bytes,
                           int batch, int num_q_heads, int num_kv_heads,
                           int head_dim, int page_size, int64_t num_pages,
                           int max_pages_per_seq, int first_page_offset,
                           float sm_scale, int num_splits, kin_stream_t stream);

/*
 * The whole decode step in ONE launch -- replaces lines 209-225 of the
 * reference layer's forward (ref: benchmark/blocktopk_decoder.py:209-225):
 * append (kin_append_paged_kv), scoring + selection (kin_block_score_topk) and
 * attention over the selected pages (kin_sparse_paged_decode), with the same
 * arithmetic, results and argument meaning as those three calls in sequence.
 * One workgroup per (sequence, KV head) runs all phases, so the page list never
 * leaves the chip and phases of different sequences overlap.
 *
 * k and v may both be NULL (no append).  sel_pages / sel_count are optional
 * outputs (both NULL, or both given with sel_stride >=
 * kin_sel_list_capacity(...)); topk / sink_pages / local_tokens as in
 * kin_block_score_topk, first_page_offset as in kin_sparse_paged_decode (a
 * non-zero offset requires sink_pages >= 1: a padded page has no valid mean
 * key); lse is optional.  One workgroup walks a whole list, of 8 waves instead
 * of 4 with 256 lists or fewer; with lists for at most a third of the GPU's
 * compute units (half, for page lists of 384 tiles of 16 tokens or more) and a
 * workspace (optional, see kin_step_workspace_bytes), a team of workgroups
 * shares a list: each scores a slice of the candidates, the keys meet in the
 * workspace, and the members each select for themselves (identical results),
 * attend a part of the listed pages and leave a partial result that the last to
 * finish merges.  A batch of up to 96 lists more than a multiple of the GPU's
 * 256 compute units (257 .. 352 lists, 513 .. 608, ...) keeps one workgroup
 * per list for that multiple and forms teams of 2 to 4 for the others, so that
 * the launch does not end with a few compute units working on whole lists
 * while the others wait.  A member waits for its team's keys for a bounded time only
 * and then scores the list alone, so the launch never depends on which
 * workgroups run at the same time.  Without sel_pages the winners are attended
 * in index order instead of score order (no sort).  slot_lens (optional, int32
 * [num_slots], by slot like kbar; [batch] without slot_ids): a per-slot token
 * counter that the kernel advances by one for every sequence of the call when
 * k and v are given -- the reference's kv_offset[batch_idx] += 1 after its copy
 * (ref: LiteSys/litesys/attention/batch_cache.py:76-84) without a launch of its
 * own.  Any of this changes only the
 * fp32 summation order of the output, not the page lists or cache bytes.  At
 * least as fast as the three calls except for few lists of more than 4096 pages
 * with topk >= 256 and for 257..349 lists with topk > 768 (up to 1.3x and 1.2x
 * slower).
 */
int kin_blocktopk_decode_step(const kin_bf16_t* q, const kin_bf16_t* k, const kin_bf16_t* v,
                              kin_bf16_t* kv_cache, kin_bf16_t* kbar,
                              const int32_t* page_indices, const int32_t* page_indptr,
                              const int32_t* last_page_len, int topk,
                              int sink_pages, int local_tokens,
                              int32_t* sel_pages, int32_t* sel_count,
                              kin_bf16_t* out, float* lse,
                              int batch, int num_q_heads, int num_kv_heads,
                              int head_dim, int page_size, int64_t num_pages,
                              int kbar_pages, int sel_stride, int first_page_offset,
                              float sm_scale, void* workspace, size_t workspace_bytes,
                              const int32_t* slot_ids, int num_slots, int32_t* slot_lens,
                              kin_stream_t stream);

/*
 * Workspace kin_blocktopk_decode_step and kin_block_score_topk can use for the
 * given problem: 0 unless the lists are few, or up to 96 more than a multiple
 * of 256 (then for those lists).  Up to 128 lists (batch *
 * num_kv_heads) the step may hand a list to a team of workgroups that meet
 * through this memory: two arrival counters per list, 4 bytes per candidate
 * page and list for the keys, and the partial results of the members that
 * attend (up to 256 workgroups x 16 heads x 129 floats: 2.1 MB at most); the
 * figure returned covers any group size and page budget.  Up to 64 lists of
 * 2048 candidate pages or more the selector spreads the scoring of a list over
 * several workgroups the same way.  Contents need no initialisation and are of
 * no use afterwards; launches that overlap in time must not share a workspace.
 * Passing NULL or too little is allowed: a list is then shared by fewer
 * workgroups, or walked by a single one as for every other shape.
 */
size_t kin_step_workspace_bytes(int batch, int num_kv_heads, int kbar_pages);

/*
 * kin_blocktopk_decode_step for callers that cannot allocate -- code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference (which sizes a 128 MiB workspace up front,
 * benchmark/blocktopk_decoder.py:152).  Same arguments, arithmetic and results as
 * kin_blocktopk_decode_step given a full workspace, but the
 * workspace is an array of KIN_STATIC_SCRATCH_BYTES bytes inside the library's
 * device code: each GPU the library runs on holds its own copy until the
 * process ends.  The call allocates and frees nothing (no hipMalloc, no
 * hipFree, no allocating library routine); the arrival counters are zeroed by a
 * small kernel on `stream`, never by a memset.  The first call on a device looks
 * the array's address up (hipGetSymbolAddress, with that device current; make
 * that call outside graph capture); the stream must belong to the current
 * device.
 * Limit: shapes whose teams would need more than KIN_STATIC_SCRATCH_BYTES are
 * rejected with KIN_ERR_WORKSPACE -- besides the partial results (2.1 MB at
 * most) the array covers the keys of up to 524288 candidate pages in total over
 * all lists, e.g. 64 lists of 8192 pages or 32 of 16384; shapes that share no
 * list between workgroups (kin_step_workspace_bytes() returns 0) never touch
 * the array.
 * All calls on one GPU share the array: calls that overlap in time on the same
 * GPU (different streams, or different threads) race and must be serialised by
 * the caller; calls in one stream are ordered by the stream.
 */
#define KIN_STATIC_SCRATCH_BYTES (4u * 1024u * 1024u + 64u * 1024u)

/*
 * Patience of a team member (kin_blocktopk_decode_step, kin_token_topk_decode,
 * kin_strided_topk_decode with few lists): the workgroups that share one list
 * exchange their scores through the workspace, and a member polls at most `polls`
 * times (about a third of a microsecond each; default 300) for the others before
 * it scores the whole list for itself -- the same values, so results do not depend
 * on it.  0: never wait (every member scores everything: what tests use to walk
 * that path); negative: back to the default.  Process-wide, read at each launch.
 * Returns the previous value.  No counterpart in the reference.
 */
int kin_set_team_spin_limit(int polls);

size_t kin_static_scratch_bytes(void);

int kin_blocktopk_decode_step_static(const kin_bf16_t* q, const kin_bf16_t* k, const kin_bf16_t* v,
                                     kin_bf16_t* kv_cache, kin_bf16_t* kbar,
                                     const int32_t* page_indices, const int32_t* page_indptr,
                                     const int32_t* last_page_len, int topk,
                                     int sink_pages, int local_tokens,
                                     int32_t* sel_pages, int32_t* sel_count,
                                     kin_bf16_t* out, float* lse,
                                     int batch, int num_q_heads, int num_kv_heads,
                                     int head_dim, int page_size, int64_t num_pages,
                                     int kbar_pages, int sel_stride, int first_page_offset,
                                     float sm_scale,
                                     const int32_t* slot_ids, int num_slots, int32_t* slot_lens,
                                     kin_stream_t stream);

/*
 * Token-level top-k sparse decode attention in one launch -- LiteSys'
 * topk_sparsity policy (ref: LiteSys/litesys/attention/sparsity_utils.py:6-21)
 * inside BatchKVManager.decode (ref: LiteSys/litesys/attention/batch_cache.py:154-168),
 * on the paged cache.  Per (sequence, KV head): the logits of every token are
 * averaged over the query group; the first sink_tokens tokens and the newest
 * local_tokens tokens are always attended; of the tokens in between, the
 * topk_tokens with the largest mean logit (ties: lowest position) are attended
 * too; everything when the sequence has no more than sink + topk + local tokens.
 * Attention itself is that of kin_sparse_paged_decode.  The token just appended
 * must already be in the cache (kin_append_paged_kv first).
 *
 * A sequence of n_pages pages holds 16*(n_pages-1) + last_page_len[b] -
 * first_page_offset tokens; token t sits in cache slot t + first_page_offset.
 * Optional outputs: sel_tokens[b,h,0:n] (stride sel_stride >= topk + sink +
 * local) the attended token positions -- sink tokens, selected tokens in
 * ascending order, local tokens -- padded with -1, and sel_count[b,h] = n
 * (-1 for a sequence with more than max_pages_per_seq pages, which is skipped:
 * out = 0).  workspace: kin_token_topk_workspace_bytes(...) bytes of scratch
 * (4 bytes per cache slot and KV head, plus two arrival counters per list and,
 * for fewer than 128 lists, up to 2.4 MB of histograms and partial results; any
 * contents, 16-byte aligned; with 128 lists or more and max_pages_per_seq up
 * to ~2300 the per-token keys stay in on-chip memory and the scratch is not
 * touched, but its size is still checked).  Reads every key of the context
 * once: HBM traffic is about half of dense decode's.  When the lists are fewer than
 * the GPU's compute units, a team of workgroups shares a list: every member scores a run of
 * pages, the first members then select for themselves and attend a share of the
 * token list each, the last one merges (a workspace without the room for that part
 * gets the older scheme: the last workgroup to arrive selects and attends alone);
 * a small kernel that zeroes the counters is then launched first on the
 * same stream (no memset, so the call can be captured in a HIP graph).
 * A batch of up to 96 lists more than a multiple of the GPU's 256 compute units
 * (when that multiple is whole sequences) is two launches, one after the other
 * on the stream: the multiple, then the rest with the GPU to themselves.
 * Limits: topk_tokens <= 4096, sink_tokens <= 64, local_tokens <= 1024.
 */
size_t kin_token_topk_workspace_bytes(int batch, int num_kv_heads, int max_pages_per_seq);

int kin_token_topk_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache,
                          const int32_t* page_indices, const int32_t* page_indptr,
                          const int32_t* last_page_len,
                          int topk_tokens, int sink_tokens, int local_tokens,
                          int first_page_offset,
                          int32_t* sel_tokens, int32_t* sel_count,
                          kin_bf16_t* out, float* lse,
                          void* workspace, size_t workspace_bytes,
                          int batch, int num_q_heads, int num_kv_heads,
                          int head_dim, int page_size, int64_t num_pages,
                          int max_pages_per_seq, int sel_stride, float sm_scale,
                          kin_stream_t stream);
int kin_token_topk_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache,
                              const int32_t* page_indices, const int32_t* page_indptr,
                              const int32_t* last_page_len,
                              int topk_tokens, int sink_tokens, int local_tokens,
                              int first_page_offset,
                              int32_t* sel_tokens, int32_t* sel_count,
                              kin_f16_t* out, float* lse,
                              void* workspace, size_t workspace_bytes,
                              int batch, int num_q_heads, int num_kv_heads,
                              int head_dim, int page_size, int64_t num_pages,
                              int max_pages_per_seq, int sel_stride, float sm_scale,
                              kin_stream_t stream);

/*
 * Strided overlapping-block top-k decode attention in one launch -- LiteSys'
 * strided_blockwise_topk_sparsity policy
 * (ref: LiteSys/litesys/attention/sparsity_utils.py:49-105) inside
 * BatchKVManager.decode (ref: LiteSys/litesys/attention/batch_cache.py:154-168).
 * Per (sequence, KV head), with L candidate tokens between the sink tokens and
 * the local window: block i covers candidates [i*stride, i*stride + block_size),
 * i < (L - block_size) / stride + 1; the min(2*topk_blocks, num_blocks) blocks
 * with the largest mean group-mean logit are chosen, their tokens united, and
 * the topk_blocks * block_size lowest-positioned of those attended together with
 * the sink and local tokens.  Candidates no chosen block covers are dropped,
 * also when the budget would have room for them; with L < block_size every token
 * is attended.  Arguments, outputs and token layout as in kin_token_topk_decode
 * (sel_stride >= max(topk_blocks, 1) * block_size + sink + local).  workspace:
 * kin_strided_topk_workspace_bytes(...).  Limits: block_size <= 64,
 * topk_blocks * block_size <= 4096, sink_tokens <= 64, local_tokens <= 1024.
 */
size_t kin_strided_topk_workspace_bytes(int batch, int num_kv_heads, int max_pages_per_seq);

int kin_strided_topk_decode(const kin_bf16_t* q, const kin_bf16_t* kv_cache,
                            const int32_t* page_indices, const int32_t* page_indptr,
                            const int32_t* last_page_len,
                            int topk_blocks, int block_size, int stride,
                            int sink_tokens, int local_tokens, int first_page_offset,
                            int32_t* sel_tokens, int32_t* sel_count,
                            kin_bf16_t* out, float* lse,
                            void* workspace, size_t workspace_bytes,
                            int batch, int num_q_heads, int num_kv_heads,
                            int head_dim, int page_size, int64_t num_pages,
                            int max_pages_per_seq, int sel_stride, float sm_scale,
                            kin_stream_t stream);
int kin_strided_topk_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache,
                                const int32_t* page_indices, const int32_t* page_indptr,
                                const int32_t* last_page_len,
                                int topk_blocks, int block_size, int stride,
                                int sink_tokens, int local_tokens, int first_page_offset,
                                int32_t* sel_tokens, int32_t* sel_count,
                                kin_f16_t* out, float* lse,
                                void* workspace, size_t workspace_bytes,
                                int batch, int num_q_heads, int num_kv_heads,
                                int head_dim, int page_size, int64_t num_pages,
                                int max_pages_per_seq, int sel_stride, float sm_scale,
                                kin_stream_t stream);

/*
 * Page-table metadata for a slot-based cache -- the paged replacement of
 * LiteSys' contiguous per-slot caches and kv_offset counters
 * (ref: LiteSys/litesys/attention/batch_cache.py:40-62,76-84).  Slot s owns the
 * physical pages s*pages_per_slot .. (s+1)*pages_per_slot-1.  For sequence b
 * living in slot slot_ids[b] (NULL = identity) with seq_lens[b] tokens, writes
 *   page_indptr[0..batch]   CSR offsets (n_pages = ceil(len / page_size); 0
 *                           pages for len <= 0, and for a sequence longer than
 *                           its slot -- pages_per_slot pages -- can hold: the
 *                           kernels then write nothing for it and return
 *                           zeros, rather than append into a cut list)
 *   page_indices[...]       slot*pages_per_slot + p, packed per sequence
 *                           (capacity batch*pages_per_slot entries)
 *   last_page_len[b]        tokens in the final page (1 for empty sequences)
 * No host synchronisation, kernels only (capturable in a HIP graph).
 * batch <= 65535.
 */
int kin_build_slot_page_table(const int32_t* slot_ids, const int32_t* seq_lens, int batch,
                              int pages_per_slot, int page_size,
                              int32_t* page_indices, int32_t* page_indptr,
                              int32_t* last_page_len, kin_stream_t stream);

/*
 * Page pool for a slot-based cache -- the paged replacement of LiteSys'
 * per-slot contiguous caches that also gives memory back: LiteSys sizes
 * [max_batch, H_kv, max_len, D] per layer up front and clear_cache zeroes a
 * slot (ref: LiteSys/litesys/attention/batch_cache.py:40-62,147-152); here the
 * slots draw pages (of 16, 32, 64 or 128 tokens) from one pool of num_pool_pages pages through a
 * free list that lives on the device, so the pool can be smaller than
 * max_slots * pages_per_slot and a finished request returns its pages.  No host
 * synchronisation anywhere; every call is a single small kernel.
 *
 * Caller-owned device arrays (int32):
 *   free_stack  [num_pool_pages]  the free page ids; the top is the next to go
 *   pool_state  [2]               [0] = pages on the stack, [1] = status bits:
 *                                 1 = a reserve call wanted more pages than were
 *                                     free (that call reserved nothing),
 *                                 2 = a sequence wanted more than pages_per_slot
 *                                     pages (its slot got pages_per_slot),
 *                                 4 = a slot id outside [0, max_slots), or one
 *                                     that an earlier entry of the same call
 *                                     named (that entry was skipped)
 *   slot_table  [max_slots, pages_per_slot]  physical page of each logical page
 *   slot_npages [max_slots]       pages the slot owns
 * kin_page_pool_init fills the stack (pages are handed out 0, 1, 2, ...), and
 * clears the state and the slot counts.
 * kin_page_pool_reserve grows the slot of every sequence b (slot_ids[b], NULL =
 * identity; distinct and below max_slots: other entries are skipped and raise
 * status bit 4) to ceil(seq_lens[b] / page_size) pages, at most
 * pages_per_slot; it never shrinks a slot, so sequences with seq_lens[b] <= 0
 * are left alone and calling it again with the same lengths changes nothing.
 * All or nothing: if the stack cannot cover the whole call it reserves nothing
 * and raises status bit 1.  batch <= 65535.
 * kin_page_pool_release pushes every page of the `count` listed slots back and
 * empties them (clear_cache).
 * kin_build_pool_page_table is kin_build_slot_page_table with page ids taken
 * from slot_table; a sequence that needs more pages than its slot owns (a
 * reserve failed, or it outgrew pages_per_slot) gets an empty page list, so no
 * unowned entry is ever listed and nothing is appended into a cut list.
 * The status word is for the host to poll when it is convenient
 * (hipMemcpy of pool_state) and to clear once it has seen it (a store of 0 to
 * pool_state[1]); kernels cannot raise.
 */
int kin_page_pool_init(int32_t* free_stack, int32_t* pool_state, int32_t* slot_npages,
                       int num_pool_pages, int max_slots, kin_stream_t stream);

int kin_page_pool_reserve(const int32_t* slot_ids, const int32_t* seq_lens, int batch,
                          int pages_per_slot, int page_size,
                          int32_t* slot_table, int32_t* slot_npages,
                          const int32_t* free_stack, int32_t* pool_state, int max_slots,
                          kin_stream_t stream);

int kin_page_pool_release(const int32_t* slot_ids, int count, int pages_per_slot,
                          const int32_t* slot_table, int32_t* slot_npages,
                          int32_t* free_stack, int32_t* pool_state, int num_pool_pages,
                          int max_slots, kin_stream_t stream);

int kin_build_pool_page_table(const int32_t* slot_ids, const int32_t* seq_lens, int batch,
                              int pages_per_slot, int page_size,
                              const int32_t* slot_table, const int32_t* slot_npages,
                              int32_t* page_indices, int32_t* page_indptr,
                              int32_t* last_page_len, int max_slots, kin_stream_t stream);

/*
 * Debugging aid, SYNCHRONOUS (waits for the stream): verifies on the device
 * that page_indptr is non-decreasing from 0 and never exceeds nnz (the length
 * of page_indices), every page id lies in [0, num_pages), and every
 * last_page_len lies in [1, page_size] for non-empty sequences.  Returns KIN_ERR_PAGE_TABLE if not.  scratch must
 * point to at least 4 bytes of device memory (the caller's, not allocated
 * here).  The reference has no counterpart: flashinfer trusts its metadata.
 */
int kin_check_page_table(const int32_t* page_indices, const int32_t* page_indptr,
                         const int32_t* last_page_len, int batch, int page_size,
                         int64_t num_pages, int64_t nnz, int32_t* scratch,
                         kin_stream_t stream);

/* ---- float16 caches ----------------------------------------------------------
 * The reference benchmark takes --dtype (benchmark/blocktopk.py:18,
 * benchmark/dense.py) and allocates q, kv_cache and compressed_key_cache in it;
 * LiteSys' manager takes a dtype too (LiteSys/litesys/attention/batch_cache.py:21).
 * The entry points above are the bfloat16 path; each of the following is its
 * float16 twin: same arguments, same meaning, same fp32 accumulation, with q, k,
 * v, kv_cache, kbar and out holding IEEE binary16 (round-to-nearest-even on
 * every store; the mean key is the fp32 sum times 1/page_size rounded to
 * binary16).  The token-granular policies above and the row-wise layer kernels
 * further down have float16 twins too (the reference moves the whole layer to
 * --dtype).  Only the entry point with built-in scratch is bfloat16 only.
 */
int kin_append_paged_kv_f16(const kin_f16_t* k, const kin_f16_t* v,
                            kin_f16_t* kv_cache, kin_f16_t* kbar,
                            const int32_t* page_indices, const int32_t* page_indptr,
                            const int32_t* last_page_len,
                            int batch, int num_kv_heads, int head_dim, int page_size,
                            int64_t num_pages, int kbar_pages,
                            const int32_t* slot_ids, int num_slots, kin_stream_t stream);

int kin_build_kbar_f16(const kin_f16_t* kv_cache, kin_f16_t* kbar,
                       const int32_t* page_indices, const int32_t* page_indptr,
                       const int32_t* last_page_len,
                       int batch, int num_kv_heads, int head_dim, int page_size,
                       int64_t num_pages, int kbar_pages,
                       const int32_t* slot_ids, int num_slots, kin_stream_t stream);

int kin_append_paged_kv_ragged_f16(const kin_f16_t* k, const kin_f16_t* v,
                                   const int32_t* append_indptr,
                                   kin_f16_t* kv_cache, kin_f16_t* kbar,
                                   const int32_t* page_indices, const int32_t* page_indptr,
                                   const int32_t* last_page_len,
                                   int batch, int64_t nnz, int max_append_len,
                                   int num_kv_heads, int head_dim, int page_size,
                                   int64_t num_pages, int kbar_pages,
                                   const int32_t* slot_ids, int num_slots, kin_stream_t stream);

int kin_block_score_topk_f16(const kin_f16_t* q, const kin_f16_t* kbar,
                             const int32_t* page_indices, const int32_t* page_indptr,
                             const int32_t* last_page_len,
                             int topk, int sink_pages, int local_tokens,
                             int32_t* sel_pages, int32_t* sel_count,
                             int32_t* sel_logical, float* scores_out,
                             int batch, int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                             int kbar_pages, int sel_stride,
                             void* workspace, size_t workspace_bytes,
                             const int32_t* slot_ids, int num_slots, kin_stream_t stream);

int kin_sparse_paged_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache,
                                const int32_t* sel_pages, const int32_t* sel_count,
                                const int32_t* last_page_len,
                                kin_f16_t* out, float* lse,
                                void* workspace, size_t workspace_bytes,
                                int batch, int num_q_heads, int num_kv_heads,
                                int head_dim, int page_size, int64_t num_pages,
                                int sel_stride, int first_page_offset,
                                float sm_scale, int num_splits, kin_stream_t stream);

int kin_dense_paged_decode_f16(const kin_f16_t* q, const kin_f16_t* kv_cache,
                               const int32_t* page_indices, const int32_t* page_indptr,
                               const int32_t* last_page_len,
                               kin_f16_t* out, float* lse,
                               void* workspace, size_t workspace_bytes,
                               int batch, int num_q_heads, int num_kv_heads,
                               int head_dim, int page_size, int64_t num_pages,
                               int max_pages_per_seq, int first_page_offset,
                               float sm_scale, int num_splits, kin_stream_t stream);

int kin_blocktopk_decode_step_f16(const kin_f16_t* q, const kin_f16_t* k, const kin_f16_t* v,
                                  kin_f16_t* kv_cache, kin_f16_t* kbar,
                                  const int32_t* page_indices, const int32_t* page_indptr,
                                  const int32_t* last_page_len, int topk,
                                  int sink_pages, int local_tokens,
                                  int32_t* sel_pages, int32_t* sel_count,
                                  kin_f16_t* out, float* lse,
                                  int batch, int num_q_heads, int num_kv_heads,
                                  int head_dim, int page_size, int64_t num_pages,
                                  int kbar_pages, int sel_stride, int first_page_offset,
                                  float sm_scale, void* workspace, size_t workspace_bytes,
                                  const int32_t* slot_ids, int num_slots, int32_t* slot_lens,
                                  kin_stream_t stream);

/* ---- row-wise layer kernels around the attention path ---------------------
 * The reference's decoder layer (benchmark/blocktopk_decoder.py:187-240) calls
 * flashinfer's RMSNorm through its custom ops layer_norm and qk_norm
 * (benchmark/model_utils.py:4-25) and leaves the residual adds, the q/k/v split
 * and act(gate)*up to PyTorch.  These three entry points cover the same steps
 * with one pass over the data each.  All tensors are bf16 (float16 for the
 * kin_*_f16 twins, whose roundings are to float16 wherever the text below says
 * bf16); statistics are fp32.
 */

/*
 * RMSNorm over rows of `hidden` elements:
 *   out[r, :] = bf16( x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * weight[:] )
 * which is flashinfer.rmsnorm(x, weight, eps) as layer_norm and qk_norm call it
 * (benchmark/model_utils.py:8,19).  With residual != NULL ([rows, hidden],
 * contiguous) the add that precedes the norm in the layer
 * (benchmark/blocktopk_decoder.py:229-232: a bf16 tensor add, then layer_norm)
 * is folded in with exactly that arithmetic -- the sum is rounded to bf16
 * first and the ROUNDED value is normalised:
 *   residual[r, :] = bf16(x[r, :] + residual[r, :]);  out = RMSNorm(residual)
 * This is the layer's unfused add-then-norm, not flashinfer.fused_add_rmsnorm
 * (benchmark/model_utils.py:27-41), which is understood to keep the fp32 sum
 * for the statistics: the two can differ in the last bf16 place.
 * Row strides are in elements (multiples of 8, >= hidden); out may alias x.
 * hidden: a multiple of 512 up to 8192, a multiple of 128 up to 2048
 * (head_dim 128 rows for qk_norm), or 64 (head_dim 64 rows for qk_norm).
 */
int kin_rms_norm(const void* x, void* residual, const void* weight, void* out,
                 int64_t rows, int hidden, int64_t x_row_stride, int64_t out_row_stride,
                 float eps, kin_stream_t stream);
int kin_rms_norm_f16(const void* x, void* residual, const void* weight, void* out,
                     int64_t rows, int hidden, int64_t x_row_stride, int64_t out_row_stride,
                     float eps, kin_stream_t stream);

/*
 * The steps between the fused QKV projection and the attention path
 * (benchmark/blocktopk_decoder.py:196-207): split qkv[b, :] =
 * [num_q_heads*D | num_kv_heads*D | num_kv_heads*D] into heads, RMSNorm every q
 * head with q_weight[D] and every k head with k_weight[D] (qk_norm,
 * benchmark/model_utils.py:15-25), copy the v heads, and write contiguous
 * q[batch, num_q_heads, D], k[batch, num_kv_heads, D], v[batch, num_kv_heads, D].
 * qkv_row_stride in elements (multiple of 8).  head_dim (D) must be 128 or 64.
 */
int kin_qkv_norm_split(const void* qkv, int64_t qkv_row_stride, const void* q_weight,
                       const void* k_weight, float eps, void* q, void* k, void* v,
                       int batch, int num_q_heads, int num_kv_heads, int head_dim,
                       kin_stream_t stream);
int kin_qkv_norm_split_f16(const void* qkv, int64_t qkv_row_stride, const void* q_weight,
                           const void* k_weight, float eps, void* q, void* k, void* v,
                           int batch, int num_q_heads, int num_kv_heads, int head_dim,
                           kin_stream_t stream);

#define KIN_ACT_SILU 0
#define KIN_ACT_GELU 1 /* erf form */
#define KIN_ACT_RELU 2

/*
 * out[r, :] = bf16( bf16(act(gate[r, :])) * up[r, :] ), the gated MLP product
 * (benchmark/blocktopk_decoder.py:234-237) with the rounding of the two bf16
 * tensor operations it replaces.  gate and up may be the two halves of one
 * fused projection: row strides in elements (multiples of 8, >= inter); out is
 * contiguous [rows, inter]; inter a multiple of 8.
 */
int kin_gated_act(const void* gate, const void* up, void* out, int64_t rows, int inter,
                  int64_t gate_row_stride, int64_t up_row_stride, int act,
                  kin_stream_t stream);
int kin_gated_act_f16(const void* gate, const void* up, void* out, int64_t rows, int inter,
                      int64_t gate_row_stride, int64_t up_row_stride, int act,
                      kin_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KINETICS_AMD_H */
