"""CPU oracle for block top-k sparse paged decode attention.  TEST INFRASTRUCTURE.

This file is the checker, not the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  The shipped path (``kinetics_amd``) never does and fails loudly
when its HIP library is missing.

It restates, in numpy with float64 arithmetic on bfloat16-rounded inputs, the
algorithm of the reference's block top-k decoder path:

* append            benchmark/blocktopk_decoder.py:209-213 (flashinfer
                    append_paged_kv_cache; same effect as LiteSys
                    copy_to_cache, LiteSys/litesys/attention/cache_utils.py:40-51)
* page scores       benchmark/blocktopk_decoder.py:216
* top-k pages       benchmark/blocktopk_decoder.py:217; per KV head as in
                    LiteSys/litesys/attention/sparsity_utils.py:36-38
* page list         benchmark/blocktopk_decoder.py:218-221 (logical->physical,
                    last page always appended) -- applied ONCE; the reference
                    file applies the translation twice and never hands the
                    result to the decode kernel, which is a defect of that
                    timing harness, not behaviour to reproduce
* attention         benchmark/blocktopk_decoder.py:223-225,255-265 (NHD pages,
                    no positional encoding, scale 1/sqrt(D)); the arithmetic is
                    LiteSys/litesys/attention/cache_utils.py:54-169
                    (logits*scale, -inf mask past the length, fp32 softmax,
                    P.V) with the new token attended
                    (LiteSys/litesys/attention/batch_cache.py:154-168)
* dense baseline    benchmark/dense_decoder.py:211-219
* LiteSys' mask form LiteSys/litesys/attention/sparsity_utils.py:24-47 on a
                    contiguous cache (litesys_decode), the cross-check that the
                    page lists with sink_pages=1, local_tokens=local and a
                    12-slot first-page offset are the same function

* layer row steps   RMSNorm (benchmark/model_utils.py:4-41), q/k norm + split and
                    act(gate)*up (benchmark/blocktopk_decoder.py:196-207,229-237)

flashinfer 0.1.6 (the wheel the reference calls, README.md:81) is not in the
reference tree; its page-table convention is restated here: sequence b owns
``page_indices[page_indptr[b]:page_indptr[b+1]]`` and holds
``(n_pages-1)*page_size + last_page_len[b]`` tokens, the metadata describing
the cache AFTER the append.

Pinning (tests/test_oracle.py): the reference ships no tests or golden
vectors for this path, so each function is pinned by what the mathematics
fixes -- append: clone-and-compare of every byte; mean key: float64 mean
within one bf16 ulp; scores: mean_g(q_g.k) == (mean_g q_g).k and LiteSys'
group-mean/block-mean order up to the constant 1/sqrt(D); selection:
numpy/torch library top-k on the same scores plus hand-built tie cases;
attention: torch scaled_dot_product_attention on the de-paged K/V when every
page is selected, out == v for one token, out == V for constant V, q == 0 gives
the mean of V, permutation invariance of the page list, split-K merge
invariance, lse == logsumexp; layer row steps: torch's own rms_norm, silu, gelu,
relu and bf16 tensor add/mul on the CPU, constant rows, scale invariance.

bfloat16 tensors are numpy uint16 arrays of raw bit patterns throughout.
"""
from __future__ import annotations

import contextlib

import numpy as np

# ---------------------------------------------------------------------------
# bfloat16 <-> float32
# ---------------------------------------------------------------------------


# The page path (append, mean keys, scores, attention) works on one element
# format per call: bfloat16, or IEEE binary16 (the reference's --dtype float16,
# benchmark/blocktopk.py:18).  Tensors are uint16 bit arrays either way; the
# format in force is chosen with ``element_format``.
_ELEMENT_FORMAT = "bf16"


@contextlib.contextmanager
def element_format(name: str):
    """``with element_format("f16"):`` -- the page-path functions below read and
    write IEEE binary16 bit patterns inside the block (default: bfloat16)."""
    global _ELEMENT_FORMAT
    if name not in ("bf16", "f16"):
        raise ValueError(name)
    old, _ELEMENT_FORMAT = _ELEMENT_FORMAT, name
    try:
        yield
    finally:
        _ELEMENT_FORMAT = old


def elem_to_f32(bits: np.ndarray) -> np.ndarray:
    """Exact widening of the element format in force to float32."""
    if _ELEMENT_FORMAT == "f16":
        return np.ascontiguousarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)
    return bf16_to_f32(bits)


def f32_to_elem(x: np.ndarray) -> np.ndarray:
    """float32 -> bits of the element format in force, round-to-nearest-even."""
    if _ELEMENT_FORMAT == "f16":
        return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)
    return f32_to_bf16(x)


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    """Exact widening of bfloat16 bit patterns (uint16) to float32."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bits, round-to-nearest-even (NaN stays NaN)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounded = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    out = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), rounded)
    return out.astype(np.uint16)


# ---------------------------------------------------------------------------
# page-table helpers
# ---------------------------------------------------------------------------


def seq_pages(page_indices, page_indptr, b):
    """Physical page ids of sequence ``b`` in logical order (CSR convention of
    benchmark/blocktopk_decoder.py:141-147)."""
    return np.asarray(page_indices[int(page_indptr[b]) : int(page_indptr[b + 1])], dtype=np.int64)


def seq_len(page_indptr, last_page_len, b, page_size):
    n_pages = int(page_indptr[b + 1]) - int(page_indptr[b])
    return 0 if n_pages <= 0 else (n_pages - 1) * page_size + int(last_page_len[b])


# ---------------------------------------------------------------------------
# (1) append  -- benchmark/blocktopk_decoder.py:209-213
# ---------------------------------------------------------------------------


def page_mean_key(page_k_bits: np.ndarray) -> np.ndarray:
    """Representative key of full pages: ``page_k_bits`` is [..., page_size, D]
    bf16 bits; float32 sum in slot order, times 1/page_size, RNE to bf16.  The
    reference leaves compressed_key_cache random
    (benchmark/blocktopk_decoder.py:166-168); the block mean is what LiteSys ranks
    blocks by (sparsity_utils.py:37) up to the query projection."""
    rows = elem_to_f32(page_k_bits)
    ps = rows.shape[-2]
    acc = np.zeros(rows.shape[:-2] + rows.shape[-1:], dtype=np.float32)
    for t in range(ps):
        acc = (acc + rows[..., t, :]).astype(np.float32)
    return f32_to_elem(acc * np.float32(1.0 / ps))


def append_paged_kv(k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len):
    """benchmark/blocktopk_decoder.py:209-213 (LiteSys copy_to_cache,
    cache_utils.py:5-51).  In place.  k, v: [B, Hkv, D] bits; kv_cache: [P, 2, ps, Hkv, D] bits;
    kbar: [B, Hkv, kbar_pages, D] bits or None (head-major; [B, pages, D] of
    the reference, blocktopk_decoder.py:165-168, when Hkv == 1).  Writes the new token at slot
    ``last_page_len[b]-1`` of the last page; a page that becomes full gets its
    mean key stored at its logical index."""
    B, Hkv, _ = k.shape
    ps = kv_cache.shape[2]
    for b in range(B):
        pages = seq_pages(page_indices, page_indptr, b)
        if len(pages) == 0:
            continue
        pid, pos = int(pages[-1]), int(last_page_len[b]) - 1
        kv_cache[pid, 0, pos] = k[b]
        kv_cache[pid, 1, pos] = v[b]
        if kbar is not None and pos == ps - 1 and len(pages) - 1 < kbar.shape[2]:
            for h in range(Hkv):
                kbar[b, h, len(pages) - 1] = page_mean_key(kv_cache[pid, 0, :, h, :])


def append_paged_kv_ragged(k, v, append_indptr, kv_cache, kbar, page_indices, page_indptr, last_page_len):
    """flashinfer.append_paged_kv_cache in its general form (the call behind
    mylib::update_kv, benchmark/blocktopk_decoder.py:38-46, which carries
    kv_append_indptr): sequence b appends rows append_indptr[b]:append_indptr[b+1]
    of k / v [nnz, Hkv, D]; the page table describes the cache after the append,
    so row i lands at token position kv_len_b - n_b + i.  Same effect as LiteSys'
    prefill write into its contiguous cache (batch_cache.py:112-131).  The mean
    key of every page the append completed is recomputed.  In place."""
    ps = kv_cache.shape[2]
    B = len(page_indptr) - 1
    for b in range(B):
        a0, a1 = int(append_indptr[b]), int(append_indptr[b + 1])
        pages = seq_pages(page_indices, page_indptr, b)
        if a1 <= a0 or len(pages) == 0:
            continue
        kv_len = (len(pages) - 1) * ps + int(last_page_len[b])
        first = kv_len - (a1 - a0)
        for i in range(a1 - a0):
            pos = first + i
            kv_cache[pages[pos // ps], 0, pos % ps] = k[a0 + i]
            kv_cache[pages[pos // ps], 1, pos % ps] = v[a0 + i]
        if kbar is not None:
            for p in range(first // ps, kv_len // ps):
                if p < kbar.shape[2]:
                    kbar[b, :, p] = page_mean_key(kv_cache[pages[p], 0].transpose(1, 0, 2))


def build_kbar(kv_cache, kbar, page_indices, page_indptr, last_page_len):
    """Mean key of every FULL page of every sequence (in place on ``kbar``)."""
    B = len(page_indptr) - 1
    ps = kv_cache.shape[2]
    for b in range(B):
        pages = seq_pages(page_indices, page_indptr, b)
        if len(pages) == 0:
            continue
        n_full = len(pages) if int(last_page_len[b]) >= ps else len(pages) - 1
        n_full = min(n_full, kbar.shape[2])
        if n_full > 0:
            # [n_full, ps, Hkv, D] -> [Hkv, n_full, ps, D]
            kbar[b, :, :n_full] = page_mean_key(kv_cache[pages[:n_full], 0].transpose(2, 0, 1, 3))


# ---------------------------------------------------------------------------
# (2) scores  -- benchmark/blocktopk_decoder.py:216
# ---------------------------------------------------------------------------


def split_pages(n_pages, last_len, sink_pages, local_tokens, kbar_pages, page_size=16):
    """(n_sink, n_cand, n_local).  The first ``sink_pages`` pages (never the
    open page) and the pages that hold the newest ``local_tokens`` tokens are
    always attended; the candidates are the whole pages in between.  sink 0 /
    local 1 is the reference's rule (benchmark/blocktopk_decoder.py:220).  With
    the sequence stored 12 slots into its first page, sink 1 / local = LiteSys'
    ``local`` is LiteSys/litesys/attention/sparsity_utils.py:31-33:
    ``_n_dynamic = (seq_len - local - sink) // block_size * block_size`` with
    sink = 4, the rest of the tokens being the local part.  Candidates beyond
    ``kbar_pages`` have no mean key and are dropped.  ``page_size``: tokens per
    page (the reference's --page_size, benchmark/blocktopk.py:13)."""
    ps = int(page_size)
    n_sink = min(sink_pages, n_pages - 1)
    kv_len = (n_pages - 1) * ps + min(max(int(last_len), 1), ps)
    n_cand = max(0, (kv_len - ps * n_sink - local_tokens) // ps)
    n_local = n_pages - n_sink - n_cand
    n_cand = max(0, min(n_cand, kbar_pages - n_sink))
    return n_sink, n_cand, n_local


def block_scores(q, kbar, page_indptr, last_page_len, sink_pages=0, local_tokens=1, page_size=16):
    """score[b][h][n] = mean_g q[b, h*G+g, :] . kbar[b, h, n_sink + n, :] in
    float64 over the candidate pages.  Returns a list (b) of lists (h) of
    float64 arrays."""
    B, Hq, D = q.shape
    Hkv = kbar.shape[1]
    G = Hq // Hkv
    qf = elem_to_f32(q).astype(np.float64)
    out = []
    for b in range(B):
        n_pages = int(page_indptr[b + 1]) - int(page_indptr[b])
        if n_pages <= 0:
            out.append([np.zeros(0) for _ in range(Hkv)])
            continue
        n_sink, n_cand, _ = split_pages(n_pages, last_page_len[b], sink_pages, local_tokens, kbar.shape[2], page_size)
        kb = elem_to_f32(kbar[b, :, n_sink : n_sink + n_cand]).astype(np.float64)  # [Hkv, n, D]
        per_head = []
        for h in range(Hkv):
            per_q = np.einsum("gd,nd->gn", qf[b, h * G : (h + 1) * G], kb[h])  # [G, n]
            per_head.append(per_q.mean(axis=0))
        out.append(per_head)
    return out


# ---------------------------------------------------------------------------
# (3) selection  -- benchmark/blocktopk_decoder.py:217-221
# ---------------------------------------------------------------------------


def select_topk(scores: np.ndarray, k: int) -> np.ndarray:
    """benchmark/blocktopk_decoder.py:217 / sparsity_utils.py:38 (torch.topk).
    Indices of the min(k, n) largest scores: descending score, equal scores by
    ascending index."""
    n = len(scores)
    order = np.lexsort((np.arange(n), -np.asarray(scores, dtype=np.float64)))
    return order[: min(k, n)].astype(np.int64)


def sel_list_capacity(topk, sink_pages=0, local_tokens=1):
    """Longest list block_score_topk can produce (for 16-token pages; larger pages need no more)."""
    return topk + sink_pages + 1 + (local_tokens + 14) // 16


def block_score_topk(q, kbar, page_indices, page_indptr, last_page_len, topk, sel_stride=None, sink_pages=0,
                     local_tokens=1, page_size=16):
    """Returns (sel_pages [B,Hkv,stride] int32 padded with -1, sel_count [B,Hkv],
    sel_logical list[b][h] of logical page index arrays, scores list[b][h] over
    the candidates).  List order: sink pages, winners (descending score), local
    pages with the open page last."""
    B = q.shape[0]
    Hkv = kbar.shape[1]
    stride = sel_list_capacity(topk, sink_pages, local_tokens) if sel_stride is None else sel_stride
    scores = block_scores(q, kbar, page_indptr, last_page_len, sink_pages, local_tokens, page_size)
    sel_pages = np.full((B, Hkv, stride), -1, dtype=np.int32)
    sel_count = np.zeros((B, Hkv), dtype=np.int32)
    sel_logical = []
    for b in range(B):
        pages = seq_pages(page_indices, page_indptr, b)
        row = []
        for h in range(Hkv):
            if len(pages) == 0:
                row.append(np.zeros(0, dtype=np.int64))
                continue
            n_sink, _, n_local = split_pages(len(pages), last_page_len[b], sink_pages, local_tokens, kbar.shape[2], page_size)
            idx = n_sink + select_topk(scores[b][h], topk)
            full = np.concatenate([pages[:n_sink], pages[idx], pages[len(pages) - n_local :]])
            sel_pages[b, h, : len(full)] = full
            sel_count[b, h] = len(full)
            row.append(idx)
        sel_logical.append(row)
    return sel_pages, sel_count, sel_logical, scores


# ---------------------------------------------------------------------------
# (4) attention  -- benchmark/blocktopk_decoder.py:223-225
# ---------------------------------------------------------------------------


def attend_pages(q_bh, kv_cache, pages, h, last_len, sm_scale, first_skip=0):
    """LiteSys cache_utils.py:54-169 restated for pages: logits * scale, softmax in
    one pass over the valid tokens, P.V.
    Softmax attention of the G query rows ``q_bh`` ([G, D] float64) over the
    tokens of ``pages`` for KV head ``h``; every page full except the final one
    (``last_len`` tokens); the first ``first_skip`` token slots of the first
    listed page are padding.  Returns (out [G, D] float64, lse [G] float64,
    natural log)."""
    G, D = q_bh.shape
    if len(pages) == 0:
        return np.zeros((G, D)), np.full(G, -np.inf)
    ps = kv_cache.shape[2]
    K = elem_to_f32(kv_cache[np.asarray(pages), 0, :, h, :]).astype(np.float64).reshape(-1, D)
    V = elem_to_f32(kv_cache[np.asarray(pages), 1, :, h, :]).astype(np.float64).reshape(-1, D)
    n_tok = (len(pages) - 1) * ps + int(last_len)
    K, V = K[first_skip:n_tok], V[first_skip:n_tok]
    if len(K) == 0:
        return np.zeros((G, D)), np.full(G, -np.inf)
    logits = (q_bh @ K.T) * sm_scale  # [G, n_tok]
    m = logits.max(axis=1, keepdims=True)
    p = np.exp(logits - m)
    s = p.sum(axis=1, keepdims=True)
    return (p / s) @ V, (m + np.log(s))[:, 0]


def sparse_paged_decode(q, kv_cache, sel_pages, sel_count, last_page_len, sm_scale=None, first_page_offset=0):
    """benchmark/blocktopk_decoder.py:223-225.  out [B, Hq, D] float64 and lse
    [B, Hq] float64 over the listed pages."""
    B, Hq, D = q.shape
    Hkv = kv_cache.shape[3]
    G = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if sm_scale is None else sm_scale
    qf = elem_to_f32(q).astype(np.float64)
    out = np.zeros((B, Hq, D))
    lse = np.full((B, Hq), -np.inf)
    for b in range(B):
        for h in range(Hkv):
            pages = sel_pages[b, h, : int(sel_count[b, h])]
            o, l = attend_pages(qf[b, h * G : (h + 1) * G], kv_cache, pages, h, last_page_len[b], scale, first_page_offset)
            out[b, h * G : (h + 1) * G] = o
            lse[b, h * G : (h + 1) * G] = l
    return out, lse


def dense_paged_decode(q, kv_cache, page_indices, page_indptr, last_page_len, sm_scale=None, first_page_offset=0):
    """Attention over every page of each sequence -- benchmark/dense_decoder.py:211-219."""
    B, Hq, D = q.shape
    Hkv = kv_cache.shape[3]
    G = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if sm_scale is None else sm_scale
    qf = elem_to_f32(q).astype(np.float64)
    out = np.zeros((B, Hq, D))
    lse = np.full((B, Hq), -np.inf)
    for b in range(B):
        pages = seq_pages(page_indices, page_indptr, b)
        for h in range(Hkv):
            o, l = attend_pages(qf[b, h * G : (h + 1) * G], kv_cache, pages, h, last_page_len[b], scale, first_page_offset)
            out[b, h * G : (h + 1) * G] = o
            lse[b, h * G : (h + 1) * G] = l
    return out, lse


def merge_partials(outs, lses):
    """Online-softmax merge of partial attention results over disjoint token
    sets (what LiteSys' split-K partial sums amount to, cache_utils.py:193-212):
    outs [S, ..., D], lses [S, ...] (natural log)."""
    lses = np.asarray(lses, dtype=np.float64)
    m = lses.max(axis=0)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    w = np.exp(lses - m_safe)
    den = w.sum(axis=0)
    num = (np.asarray(outs) * w[..., None]).sum(axis=0)
    with np.errstate(invalid="ignore", divide="ignore"):
        out = np.where(den[..., None] > 0, num / den[..., None], 0.0)
        lse = np.where(den > 0, m_safe + np.log(den), -np.inf)
    return out, lse


# ---------------------------------------------------------------------------
# one decode step  -- benchmark/blocktopk_decoder.py:209-225
# ---------------------------------------------------------------------------


def decode_step(q, k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len, topk, sm_scale=None, sink_pages=0,
                local_tokens=1, first_page_offset=0):
    """append -> score -> select -> attend.  Mutates kv_cache / kbar.  Returns
    dict(out, lse, sel_pages, sel_count, sel_logical, scores)."""
    append_paged_kv(k, v, kv_cache, kbar, page_indices, page_indptr, last_page_len)
    sel_pages, sel_count, sel_logical, scores = block_score_topk(q, kbar, page_indices, page_indptr, last_page_len, topk,
                                                                 sink_pages=sink_pages, local_tokens=local_tokens,
                                                                 page_size=kv_cache.shape[2])
    out, lse = sparse_paged_decode(q, kv_cache, sel_pages, sel_count, last_page_len, sm_scale, first_page_offset)
    return dict(out=out, lse=lse, sel_pages=sel_pages, sel_count=sel_count, sel_logical=sel_logical, scores=scores)


# ---------------------------------------------------------------------------
# LiteSys' own formulation on a contiguous cache (mask on full logits)
# ---------------------------------------------------------------------------


def litesys_blockwise_topk_mask(mean_logits, seq_len, topk_block, local, sink=4, block_size=16):
    """LiteSys/litesys/attention/sparsity_utils.py:24-47 for one sequence and one
    KV head.  ``mean_logits`` [seq_len]: the logits averaged over the query group
    (:36).  Returns a bool array [seq_len], True where a token stays attended:
    everything when ``seq_len <= n_full`` (:27-32), otherwise the ``sink`` first
    tokens, the top ``topk_block`` blocks of the dynamic part by block-mean logit
    (:37-45) and the ``_local`` newest tokens (:33-35)."""
    n_full = sink + local + topk_block * block_size
    n_full = (n_full + block_size - 1) // block_size * block_size
    keep = np.ones(seq_len, dtype=bool)
    if seq_len <= n_full:
        return keep
    n_dynamic = (seq_len - local - sink) // block_size * block_size
    n_local = seq_len - n_dynamic - sink
    dyn = np.asarray(mean_logits[sink : seq_len - n_local], dtype=np.float64)
    block_means = dyn.reshape(-1, block_size).mean(axis=1)
    top = select_topk(block_means, topk_block)
    block_keep = np.zeros(len(block_means), dtype=bool)
    block_keep[top] = True
    keep[sink : seq_len - n_local] = np.repeat(block_keep, block_size)
    return keep


def litesys_topk_mask(mean_logits, seq_len, topk, local, sink=4):
    """LiteSys/litesys/attention/sparsity_utils.py:6-21 for one sequence and one
    KV head: everything when ``seq_len <= sink + topk + local`` (:9-12);
    otherwise the ``sink`` first tokens, the ``local`` newest and, of the tokens
    in between, the ``topk`` with the largest group-mean logit (:13-19)."""
    keep = np.ones(seq_len, dtype=bool)
    if seq_len <= sink + topk + local:
        return keep
    dyn = np.asarray(mean_logits[sink : seq_len - local], dtype=np.float64)
    dyn_keep = np.zeros(len(dyn), dtype=bool)
    dyn_keep[select_topk(dyn, topk)] = True
    keep[sink : seq_len - local] = dyn_keep
    return keep


def litesys_strided_mask(mean_logits, seq_len, topk_block, local, sink=4, block_size=16, stride=8):
    """LiteSys/litesys/attention/sparsity_utils.py:49-105 for one sequence and one
    KV head.  Nothing is masked when ``seq_len <= sink + local`` (:56-57) or the
    dynamic part is shorter than a block (:63-64).  Otherwise overlapping blocks
    start every ``stride`` dynamic tokens (:74-77), their mean logit ranks them
    (:80-81), ``min(2 * topk_block, num_blocks)`` are taken (:84-85), their tokens
    united in position order and cut to ``topk_block * block_size`` (:88-95); the
    rest of the dynamic part is masked (:101-103)."""
    keep = np.ones(seq_len, dtype=bool)
    if seq_len <= sink + local:
        return keep
    dyn = np.asarray(mean_logits[sink : seq_len - local], dtype=np.float64)
    L = len(dyn)
    if L < block_size:
        return keep
    num_blocks = (L - block_size) // stride + 1
    starts = np.arange(num_blocks) * stride
    block_means = np.array([dyn[s0 : s0 + block_size].mean() for s0 in starts])
    top = select_topk(block_means, min(2 * topk_block, num_blocks))
    tokens = np.unique(np.concatenate([np.arange(starts[i], starts[i] + block_size) for i in top])) if len(top) else \
        np.zeros(0, dtype=np.int64)
    tokens = tokens[: topk_block * block_size]
    dyn_keep = np.zeros(L, dtype=bool)
    dyn_keep[tokens] = True
    keep[sink : seq_len - local] = dyn_keep
    return keep


def strided_block_means(mean_logits, seq_len, local, sink=4, block_size=16, stride=8):
    """The block means litesys_strided_mask ranks (empty when nothing is masked)."""
    if seq_len <= sink + local or seq_len - sink - local < block_size:
        return np.zeros(0)
    dyn = np.asarray(mean_logits[sink : seq_len - local], dtype=np.float64)
    num_blocks = (len(dyn) - block_size) // stride + 1
    return np.array([dyn[i * stride : i * stride + block_size].mean() for i in range(num_blocks)])


def token_topk_decode(q, kv_cache, page_indices, page_indptr, last_page_len, topk, sink=4, local=1, first_page_offset=0,
                      sm_scale=None, policy="topk", block_size=16, stride=8):
    """Token-level top-k decode on the paged cache: per sequence the cache is
    read back into LiteSys' contiguous form (token t = cache slot t +
    first_page_offset) and litesys_decode (``policy`` "topk" or "strided") does
    the rest.
    Returns (out [B, Hq, D] float64, keep list[b] of bool [Hkv, seq_len],
    mean_logits list[b] of float64 [Hkv, seq_len])."""
    B, Hq, D = q.shape
    ps = kv_cache.shape[2]
    out = np.zeros((B, Hq, D))
    keeps, means = [], []
    qf = elem_to_f32(q).astype(np.float64)
    for b in range(B):
        pages = seq_pages(page_indices, page_indptr, b)
        kv_len = (len(pages) - 1) * ps + int(last_page_len[b]) if len(pages) else 0
        if kv_len - first_page_offset <= 0:
            keeps.append(None)
            means.append(None)
            continue
        K = elem_to_f32(kv_cache[pages, 0]).reshape(len(pages) * ps, -1, D)[first_page_offset:kv_len]
        V = elem_to_f32(kv_cache[pages, 1]).reshape(len(pages) * ps, -1, D)[first_page_offset:kv_len]
        o, keep, mean = litesys_decode(qf[b], K, V, topk, local, sink=sink, sm_scale=sm_scale, policy=policy,
                                       block_size=block_size, stride=stride, return_mean_logits=True)
        out[b] = o
        keeps.append(keep)
        means.append(mean)
    return out, keeps, means


def litesys_decode(q, K, V, topk_block, local, sink=4, block_size=16, sm_scale=None, policy="block",
                   return_mean_logits=False, keep=None, stride=8):
    """One sequence of LiteSys' sparse decode on its contiguous cache
    (LiteSys/litesys/attention/batch_cache.py:154-168): logits of every token
    (cache_utils.py:54-93, scale 1/sqrt(D)), the sparsity policy per KV head on
    the group-mean logits -- blockwise_topk_sparsity (sparsity_utils.py:24-47,
    ``policy="block"``), topk_sparsity (:6-21, ``policy="topk"``, where
    ``topk_block`` counts tokens) or strided_blockwise_topk_sparsity (:49-105,
    ``policy="strided"``) --, softmax over what stays
    (cache_utils.py:216-226), P.V (cache_utils.py:97-169).  q [Hq, D], K / V
    [seq_len, Hkv, D] float (the new token included).  ``topk_block=None`` is the
    dense layer.  ``keep`` [Hkv, seq_len] overrides the policy's choice (to
    price a selection that differs from it only by ties).  Returns (out [Hq, D]
    float64, keep [Hkv, seq_len] bool)."""
    q = np.asarray(q, dtype=np.float64)
    K = np.asarray(K, dtype=np.float64)
    V = np.asarray(V, dtype=np.float64)
    Hq, D = q.shape
    seq_len, Hkv, _ = K.shape
    G = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if sm_scale is None else sm_scale
    out = np.zeros((Hq, D))
    keep_all = np.ones((Hkv, seq_len), dtype=bool)
    mean_all = np.zeros((Hkv, seq_len))
    for h in range(Hkv):
        logits = (q[h * G : (h + 1) * G] @ K[:, h, :].T) * scale  # [G, seq_len]
        mean_all[h] = logits.mean(axis=0)
        if keep is not None:
            keep_all[h] = keep[h]
        elif topk_block is not None and policy == "block":
            keep_all[h] = litesys_blockwise_topk_mask(mean_all[h], seq_len, topk_block, local, sink, block_size)
        elif topk_block is not None and policy == "strided":
            keep_all[h] = litesys_strided_mask(mean_all[h], seq_len, topk_block, local, sink, block_size, stride)
        elif topk_block is not None:
            keep_all[h] = litesys_topk_mask(mean_all[h], seq_len, topk_block, local, sink)
        masked = np.where(keep_all[h][None, :], logits, -np.inf)
        p = np.exp(masked - masked.max(axis=1, keepdims=True))
        out[h * G : (h + 1) * G] = (p / p.sum(axis=1, keepdims=True)) @ V[:, h, :]
    if return_mean_logits:
        return out, keep_all, mean_all
    return out, keep_all


# ---------------------------------------------------------------------------
# Row-wise steps of the decoder layer around the attention path
# ---------------------------------------------------------------------------


def rms_norm(x, weight, eps, residual=None):
    """RMSNorm over the last axis, element bits in and out (bf16, or fp16 inside
    ``element_format("f16")``; "bf16" below then reads "fp16"): x * rsqrt(mean(x^2) + eps)
    * weight, which is flashinfer.rmsnorm as the reference's layer_norm and
    qk_norm call it (benchmark/model_utils.py:4-25).  With ``residual`` the sum
    x + residual, rounded to bf16 as a bf16 tensor add rounds it
    (benchmark/blocktopk_decoder.py:229-232; fused_layer_norm,
    benchmark/model_utils.py:27-41), is normalised instead.  Returns
    (out_bits, new_residual_bits or None)."""
    xf = elem_to_f32(x).astype(np.float64)
    new_res = None
    if residual is not None:
        new_res = f32_to_elem((xf + elem_to_f32(residual).astype(np.float64)).astype(np.float32))
        xf = elem_to_f32(new_res).astype(np.float64)
    w = elem_to_f32(weight).astype(np.float64)
    r = 1.0 / np.sqrt(np.mean(xf * xf, axis=-1, keepdims=True) + float(eps))
    return f32_to_elem((xf * r * w).astype(np.float32)), new_res


def qkv_norm_split(qkv, q_weight, k_weight, eps, num_q_heads, num_kv_heads, head_dim=128):
    """Fused projection rows [Hq*D | Hkv*D | Hkv*D] -> q[B,Hq,D], k[B,Hkv,D] (each
    head RMS-normalised) and v[B,Hkv,D] (benchmark/blocktopk_decoder.py:196-207)."""
    qkv = np.asarray(qkv, dtype=np.uint16)
    B = qkv.shape[0]
    nq, nk = num_q_heads * head_dim, num_kv_heads * head_dim
    q = qkv[:, :nq].reshape(B, num_q_heads, head_dim)
    k = qkv[:, nq:nq + nk].reshape(B, num_kv_heads, head_dim)
    v = qkv[:, nq + nk:nq + 2 * nk].reshape(B, num_kv_heads, head_dim)
    return rms_norm(q, q_weight, eps)[0], rms_norm(k, k_weight, eps)[0], np.ascontiguousarray(v)


def gated_act(gate, up, act="silu"):
    """bf16(bf16(act(gate)) * up): the gated MLP product of
    benchmark/blocktopk_decoder.py:234-237 with the rounding of its two bf16
    tensor operations.  gelu is the erf form."""
    from math import erf

    g = elem_to_f32(gate).astype(np.float64)
    if act == "silu":
        a = g / (1.0 + np.exp(-g))
    elif act == "gelu":
        a = 0.5 * g * (1.0 + np.vectorize(erf)(g / np.sqrt(2.0)))
    elif act == "relu":
        a = np.maximum(g, 0.0)
    else:
        raise ValueError(f"unknown activation {act!r}")
    a = elem_to_f32(f32_to_elem(a.astype(np.float32))).astype(np.float64)
    return f32_to_elem((a * elem_to_f32(up).astype(np.float64)).astype(np.float32))


# ---------------------------------------------------------------------------
# The tie rule of the parity contract
# ---------------------------------------------------------------------------


def selection_matches(got_idx, scores, k, rel_tol=1e-3):
    """True iff ``got_idx`` is an acceptable top-k of ``scores``: the same set
    as the oracle's, except that indices may differ where their scores tie
    with the k-th score within ``rel_tol`` relative.  Returns (ok, message)."""
    scores = np.asarray(scores, dtype=np.float64)
    want = select_topk(scores, k)
    got = np.asarray(got_idx, dtype=np.int64)
    if len(got) != len(want):
        return False, f"length {len(got)} != {len(want)}"
    if len(set(got.tolist())) != len(got):
        return False, "duplicate indices"
    if len(got) and (got.min() < 0 or got.max() >= len(scores)):
        return False, "index out of range"
    if len(want) == 0:
        return True, ""
    kth = scores[want[-1]]
    tol = rel_tol * max(abs(kth), np.finfo(np.float32).tiny)
    diff = set(got.tolist()) ^ set(want.tolist())
    for i in diff:
        if abs(scores[i] - kth) > tol:
            return False, f"index {i} score {scores[i]!r} is not within {rel_tol} rel of k-th score {kth!r}"
    return True, ""
