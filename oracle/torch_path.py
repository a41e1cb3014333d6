"""The reference's torch path for one block top-k decode step, restated for
torch-CPU.  TEST INFRASTRUCTURE: used by tests (cross-checked against
``blocktopk_oracle``) and timed by ``bench.py`` as the ``cpu_baseline``; never
imported by the shipped package.

Op order follows benchmark/blocktopk_decoder.py:209-225:
  append (indexed copy in place of flashinfer.append_paged_kv_cache, :209-213)
  csim = einsum("b g d, b n d -> b g n", q, kbar).mean(dim=1)          (:216)
  topk(csim, k).indices                                                (:217)
  logical -> physical page ids, cat the last page                      (:218-221)
  paged decode attention over the k+1 pages                            (:223-225)
with the attention arithmetic of LiteSys' kernels
(LiteSys/litesys/attention/cache_utils.py:54-169: logits * 1/sqrt(D), -inf mask
past the length, fp32 softmax, P.V) since flashinfer's kernel is not in the
reference tree.  Restrictions (as in the reference, blocktopk_decoder.py:165):
one KV head, every sequence the same page count.
"""
from __future__ import annotations

import math

import torch


@torch.inference_mode()
def blocktopk_decode_step(q, k, v, kv_cache, kbar, page_table, last_page_len, topk, compute_dtype=torch.float32,
                          return_scores=False):
    """q [B,G,D], k/v [B,1,D] bf16; kv_cache [P,2,ps,1,D] bf16; kbar [B,N,D] bf16
    with N = n_pages-1 candidates; page_table [B,n_pages] int64; last_page_len
    [B] int64 (cache state AFTER the append).  Returns (out [B,G,D] bf16,
    topk logical indices [B,k]) and, with ``return_scores``, csim [B,N].
    ``compute_dtype=torch.bfloat16`` is the reference's own score arithmetic: its q
    and compressed_key_cache are bf16 tensors, so the einsum returns bf16, .mean(1)
    returns bf16 and torch.topk ranks those bf16 values
    (benchmark/blocktopk_decoder.py:216-217); float32 is the more exact restatement
    that the HIP path follows."""
    B, G, D = q.shape
    ps = kv_cache.shape[2]
    n_pages = page_table.shape[1]
    # append
    last_page = page_table[:, -1]
    pos = last_page_len - 1
    kv_cache[last_page, 0, pos, 0] = k[:, 0]
    kv_cache[last_page, 1, pos, 0] = v[:, 0]
    # score + select
    csim = torch.einsum("bgd,bnd->bgn", q.to(compute_dtype), kbar.to(compute_dtype)).mean(dim=1)
    kk = min(topk, n_pages - 1)
    idx = torch.topk(csim, kk, dim=-1).indices
    phys = torch.gather(page_table[:, :-1], 1, idx)
    phys = torch.cat([phys, last_page[:, None]], dim=-1)  # [B, kk+1]
    # gather + attention
    K = kv_cache[phys, 0, :, 0].reshape(B, (kk + 1) * ps, D).to(torch.float32)
    V = kv_cache[phys, 1, :, 0].reshape(B, (kk + 1) * ps, D).to(torch.float32)
    logits = torch.einsum("bgd,btd->bgt", q.to(torch.float32), K) * (1.0 / math.sqrt(D))
    tok = torch.arange((kk + 1) * ps)[None, :]
    valid = tok < (kk * ps + last_page_len)[:, None]
    logits = logits.masked_fill(~valid[:, None, :], float("-inf"))
    p = torch.softmax(logits, dim=-1)
    out = torch.einsum("bgt,btd->bgd", p, V).to(torch.bfloat16)
    if return_scores:
        return out, idx, csim
    return out, idx


@torch.inference_mode()
def dense_decode_step(q, k, v, kv_cache, page_table, last_page_len):
    """Dense paged decode over all pages -- benchmark/dense_decoder.py:211-219."""
    B, G, D = q.shape
    ps = kv_cache.shape[2]
    n_pages = page_table.shape[1]
    last_page = page_table[:, -1]
    pos = last_page_len - 1
    kv_cache[last_page, 0, pos, 0] = k[:, 0]
    kv_cache[last_page, 1, pos, 0] = v[:, 0]
    K = kv_cache[page_table, 0, :, 0].reshape(B, n_pages * ps, D).to(torch.float32)
    V = kv_cache[page_table, 1, :, 0].reshape(B, n_pages * ps, D).to(torch.float32)
    logits = torch.einsum("bgd,btd->bgt", q.to(torch.float32), K) * (1.0 / math.sqrt(D))
    tok = torch.arange(n_pages * ps)[None, :]
    valid = tok < ((n_pages - 1) * ps + last_page_len)[:, None]
    logits = logits.masked_fill(~valid[:, None, :], float("-inf"))
    p = torch.softmax(logits, dim=-1)
    return torch.einsum("bgt,btd->bgd", p, V).to(torch.bfloat16)


@torch.inference_mode()
def reference_bf16_scores(q, kbar):
    """csim exactly as the reference forms it: bf16 tensors in, so the einsum's
    [B,G,N] result is bf16 and .mean(1) is bf16 (benchmark/blocktopk_decoder.py:216).
    q [B,G,D] bf16, kbar [B,N,D] bf16 -> [B,N] bf16."""
    assert q.dtype == torch.bfloat16 and kbar.dtype == torch.bfloat16
    return torch.einsum("bgd,bnd->bgn", q, kbar).mean(dim=1)


def _bf16_ulp(x):
    """Spacing of bfloat16 numbers (8 significant bits) around |x| (float64 tensor)."""
    ax = x.abs().clamp_min(2.0 ** -126)
    return torch.pow(2.0, torch.floor(torch.log2(ax)) - 7)


@torch.inference_mode()
def bf16_score_band(q, kbar):
    """How far the reference's bf16 score of a page can lie from the exact one:
    half a bf16 unit for each of the G per-head products the einsum rounds,
    averaged, plus one unit of the mean itself (sum and division each round).
    Returns (exact [B,N] float64, band [B,N] float64)."""
    d = torch.einsum("bgd,bnd->bgn", q.double(), kbar.double())  # exact products of bf16 inputs (float64 holds them)
    exact = d.mean(dim=1)
    band = 0.5 * _bf16_ulp(d).mean(dim=1) + _bf16_ulp(exact)
    return exact, band


@torch.inference_mode()
def compare_with_bf16_reference(q, kbar, got_idx, k):
    """The page indices ``got_idx`` [B,k] (any order) of a selector that ranks by
    exact / fp32 scores, against torch.topk on the reference's bf16 scores.
    For every pair (p picked here but not by the reference, r picked by the
    reference but not here) the reference's own scores must be tied within its
    rounding: ref(r) - ref(p) <= band(r) + band(p).  Returns a dict with the
    overlap fraction, the number of differing picks and the worst violation
    (<= 0 means every disagreement is a tie at the reference's precision)."""
    ref = reference_bf16_scores(q, kbar).double()
    exact, band = bf16_score_band(q, kbar)
    assert bool(((ref - exact).abs() <= band).all()), "the reference's bf16 score left its rounding band"
    ref_idx = torch.topk(ref, k, dim=-1).indices
    B = q.shape[0]
    differing, worst = 0, -float("inf")
    for b in range(B):
        got, want = set(got_idx[b].tolist()), set(ref_idx[b].tolist())
        only_got, only_ref = sorted(got - want), sorted(want - got)
        differing += len(only_got)
        for p in only_got:
            for r in only_ref:
                worst = max(worst, float(ref[b, r] - ref[b, p] - band[b, r] - band[b, p]))
    return dict(overlap=1.0 - differing / float(B * k), differing=differing, picks=B * k, worst_violation=worst, ref_idx=ref_idx)
