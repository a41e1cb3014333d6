"""Seeded synthetic decode problems shared by the CPU and GPU tests.

Everything is numpy so that the oracle and the HIP path see bit-identical
inputs; bfloat16 tensors are uint16 bit arrays (``to_torch`` converts).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np

from oracle import blocktopk_oracle as O

HEAD_DIM = 128
PAGE_SIZE = 16
_head_dim = HEAD_DIM  # what make_problem() builds; see head_dim()


class head_dim:
    """``with head_dim(64): ...`` -- problems made inside have head rows of that many elements."""

    def __init__(self, d: int):
        assert d in (64, 128)
        self.d = d

    def __enter__(self):
        global _head_dim
        self.prev, _head_dim = _head_dim, self.d
        return self.d

    def __exit__(self, *exc):
        global _head_dim
        _head_dim = self.prev
        return False


def current_head_dim() -> int:
    return _head_dim


@dataclass
class Problem:
    q: np.ndarray               # [B, Hq, D] bf16 bits
    k: np.ndarray               # [B, Hkv, D]
    v: np.ndarray               # [B, Hkv, D]
    kv_cache: np.ndarray        # [P, 2, ps, Hkv, D]
    kbar: np.ndarray            # [B, Hkv, kbar_pages, D]  (state BEFORE the append)
    page_indices: np.ndarray    # int32 [nnz]
    page_indptr: np.ndarray     # int32 [B+1]
    last_page_len: np.ndarray   # int32 [B]   (state AFTER the append)
    topk: int
    lengths: np.ndarray         # post-append token counts
    meta: dict = field(default_factory=dict)

    @property
    def B(self):
        return self.q.shape[0]

    @property
    def Hq(self):
        return self.q.shape[1]

    @property
    def Hkv(self):
        return self.kv_cache.shape[3]

    @property
    def num_pages(self):
        return self.kv_cache.shape[0]

    @property
    def max_pages(self):
        return int(np.max(np.diff(self.page_indptr))) if self.B else 0


def randn_bf16(rng, shape, scale=1.0, offset=None):
    x = rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)
    if offset is not None:
        x = x + offset.astype(np.float32)
    return O.f32_to_elem(x)   # bfloat16 bits unless a test is inside O.element_format("f16")


def make_problem(seed: int, lengths, num_kv_heads: int = 1, group: int = 4, topk: int = 8,
                 table: str = "random", extra_pages: int = 3, kbar_slack: int = 2,
                 page_mean_sigma: float = 0.5, build_kbar: bool = True, page_size: int = PAGE_SIZE) -> Problem:
    """``lengths`` are token counts AFTER the append (>= 1 each; 0 = empty sequence).

    table: "random"     physical ids are a seeded permutation of all pages
           "strided"    the reference layout, id = p * B + b (needs equal lengths)
           "fragmented" half the sequences contiguous runs, half scattered
    """
    rng = np.random.default_rng(seed)
    lengths = np.asarray(lengths, dtype=np.int64)
    B = len(lengths)
    ps, D = page_size, _head_dim
    n_pages = (lengths + ps - 1) // ps
    total = int(n_pages.sum()) + extra_pages
    indptr = np.zeros(B + 1, dtype=np.int32)
    indptr[1:] = np.cumsum(n_pages)
    last_len = np.where(lengths > 0, lengths - (n_pages - 1) * ps, 1).astype(np.int32)

    if table == "random":
        perm = rng.permutation(total)[: int(n_pages.sum())]
        indices = perm.astype(np.int32)
    elif table == "strided":
        assert len(set(n_pages.tolist())) == 1, "strided table needs equal page counts"
        n = int(n_pages[0])
        indices = (np.arange(n)[None, :] * B + np.arange(B)[:, None]).reshape(-1).astype(np.int32)
        total = max(total, n * B)
    elif table == "fragmented":
        free = list(rng.permutation(total))
        # contiguous runs first (claimed from a sorted block), scattered ones from what is left
        contiguous = [b for b in range(B) if b % 2 == 0]
        used = set()
        indices = np.zeros(int(n_pages.sum()), dtype=np.int32)
        cursor = 0
        for b in contiguous:
            n = int(n_pages[b])
            indices[indptr[b] : indptr[b] + n] = np.arange(cursor, cursor + n)
            used.update(range(cursor, cursor + n))
            cursor += n
        rest = [p for p in free if p not in used]
        pos = 0
        for b in range(B):
            if b % 2 == 1:
                n = int(n_pages[b])
                indices[indptr[b] : indptr[b] + n] = rest[pos : pos + n]
                pos += n
    else:
        raise ValueError(table)

    # K gets a per-page mean offset so page scores are well separated.
    page_mu = rng.standard_normal((total, 1, 1, num_kv_heads, 1), dtype=np.float32) * np.float32(page_mean_sigma)
    kv = np.empty((total, 2, ps, num_kv_heads, D), dtype=np.uint16)
    kv[:, 0:1] = randn_bf16(rng, (total, 1, ps, num_kv_heads, D), offset=np.broadcast_to(page_mu, (total, 1, ps, num_kv_heads, D)))
    kv[:, 1:2] = randn_bf16(rng, (total, 1, ps, num_kv_heads, D))
    Hq = num_kv_heads * group
    q = randn_bf16(rng, (B, Hq, D))
    k = randn_bf16(rng, (B, num_kv_heads, D))
    v = randn_bf16(rng, (B, num_kv_heads, D))
    kbar_pages = int(n_pages.max()) + kbar_slack if B else 1
    kbar = np.zeros((B, num_kv_heads, kbar_pages, D), dtype=np.uint16)
    if build_kbar:
        # state before the append: the last page is not full yet (its final slot is still unwritten)
        pre_last = np.maximum(last_len - 1, 0).astype(np.int32)
        O.build_kbar(kv, kbar, indices, indptr, pre_last)
    return Problem(q=q, k=k, v=v, kv_cache=kv, kbar=kbar, page_indices=indices, page_indptr=indptr,
                   last_page_len=last_len, topk=topk, lengths=lengths, meta=dict(seed=seed, table=table))


def to_torch(bits: np.ndarray, device="cpu"):
    """uint16 bit patterns -> a bfloat16 tensor (a float16 one inside O.element_format("f16"))."""
    import torch

    dt = torch.float16 if O._ELEMENT_FORMAT == "f16" else torch.bfloat16
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(dt)
    return t.to(device)


def from_torch(t) -> np.ndarray:
    import torch

    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def int_tensor(a: np.ndarray, device="cpu"):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(device)


# Shapes on which the selection is compared with the reference's bf16-scored top-k.
BF16_CASES = [
    # seed, batch, context, topk, group, sigma of the per-page key offset (0: page scores barely separated)
    (0, 8, 4096, 64, 4, 0.5),      # the tiny benchmark configuration
    (1, 6, 32768, 128, 4, 0.5),    # headline shape, a slice of the batch
    (2, 6, 32768, 256, 8, 0.5),    # Qwen3-32B share
    (3, 12, 8192, 64, 3, 0.1),
    (4, 6, 16384, 64, 4, 0.0),
]


def bf16_case(seed, B, L, topk, G, sigma):
    """A uniform problem after its append, as torch tensors for oracle/torch_path.py."""
    pb = make_problem(seed, [L + 1] * B, num_kv_heads=1, group=G, topk=topk, page_mean_sigma=sigma)
    n = L // PAGE_SIZE
    import torch

    table = torch.from_numpy(pb.page_indices.astype(np.int64)).reshape(B, n + 1)
    last = torch.from_numpy(pb.last_page_len.astype(np.int64))
    return pb, n, table, last
