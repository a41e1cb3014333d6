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
