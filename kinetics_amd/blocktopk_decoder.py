"""Attention-layer objects with the buffers and call order of the reference's
``BlockTopkDecoderLayer`` / dense ``DecoderLayer``, backed by the HIP kernels.

``BlockTopkPagedAttention`` owns what the reference layer sets up in its
constructor (benchmark/blocktopk_decoder.py:138-168): the page table
``paged_kv_indices`` (physical id ``p * batch + b``), the CSR ``paged_kv_indptr``,
``last_kv_lens``, the fixed ``topk_page_indices`` buffer, the paged ``kv_cache``
``[pages, 2, page_size, H_kv, D]`` and the ``compressed_key_cache`` of per-page
mean keys.  ``forward(q, k, v)`` runs lines 209-225 of that file: append the new
token, score pages, take the top-k plus the last page, attend.

Differences from the reference file, on purpose: the selected pages are written
into the buffer the attention kernel reads (the reference rebinds the attribute,
so its kernel never sees them, :221 vs :157); the logical->physical translation
is applied once (:218-219 apply it twice); ``last_kv_lens`` follows the
flashinfer contract (1..page_size) instead of zeros (:149); and
``compressed_key_cache`` holds true page means, not random numbers (:166-168).
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import ops


class BlockTopkPagedAttention:
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, batch_size: int, prefix_len: int,
                 max_len: int, page_size: int, topk_page: int, device="cuda", dtype=torch.bfloat16,
                 init_cache: str = "randn", seed: int = 0, fused: Optional[bool] = None, sink_pages: int = 0,
                 local_tokens: int = 1):
        if dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("the HIP kernels are built for bfloat16 and float16")
        if prefix_len % page_size != 0:
            raise ValueError("prefix_len must be a multiple of page_size (as in the reference benchmark)")
        if max_len < prefix_len + page_size:
            raise ValueError("max_len must leave room for at least one page after the prefix")
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.batch_size, self.prefix_len, self.page_size, self.topk_page = batch_size, prefix_len, page_size, topk_page
        self.device = torch.device(device)
        self.dtype = dtype
        B = batch_size
        max_num_pages = max_len // page_size
        self.num_pages_per_req = n = prefix_len // page_size
        self.max_pages_per_req = max_num_pages
        dev = self.device

        # benchmark/blocktopk_decoder.py:141-142: request b owns pages p*B + b, p = 0..n (n full + 1 open).
        table = torch.arange(n + 1, dtype=torch.int32, device=dev) * B + torch.arange(B, dtype=torch.int32, device=dev)[:, None]
        self.paged_kv_indices = table.reshape(-1).contiguous()
        self.paged_kv_indptr = (torch.arange(B + 1, dtype=torch.int32, device=dev) * (n + 1)).contiguous()
        # The open page holds exactly the token being decoded after the append.
        self.last_kv_lens = torch.ones(B, dtype=torch.int32, device=dev)
        # the first sink_pages pages and the pages of the newest local_tokens tokens are always attended
        # (0 / 1: the reference's rule, top-k plus the last page)
        self.sink_pages, self.local_tokens = sink_pages, local_tokens
        self.list_capacity = ops.sel_list_capacity(topk_page, sink_pages, local_tokens)
        self.topk_page_indices = torch.full((B, num_kv_heads, self.list_capacity), -1, dtype=torch.int32, device=dev)
        self.topk_page_count = torch.zeros(B, num_kv_heads, dtype=torch.int32, device=dev)

        shape = (max_num_pages * B, 2, page_size, num_kv_heads, head_dim)
        if init_cache == "randn":
            gen = torch.Generator(device=dev).manual_seed(seed)
            self.kv_cache = torch.empty(shape, dtype=dtype, device=dev)
            # fill page by page range to bound the fp32 temporary
            step = max(1, (1 << 28) // (2 * page_size * num_kv_heads * head_dim))
            for s in range(0, shape[0], step):
                e = min(shape[0], s + step)
                self.kv_cache[s:e] = torch.randn((e - s, *shape[1:]), generator=gen, device=dev, dtype=torch.float32).to(dtype)
        elif init_cache == "empty":
            self.kv_cache = torch.empty(shape, dtype=dtype, device=dev)
        else:
            raise ValueError("init_cache must be 'randn' or 'empty'")
        self.compressed_key_cache = torch.zeros(B, num_kv_heads, max_num_pages, head_dim, dtype=dtype, device=dev)
        self.refresh_compressed_keys()

        self.sm_scale = 1.0 / math.sqrt(head_dim)
        # one launch or three: same results, the faster one for this shape unless told otherwise
        self.fused = ops.prefer_fused_step(B, num_kv_heads, n + 1, topk_page) if fused is None else bool(fused)
        ws = ops.decode_workspace_bytes(B, num_heads, num_kv_heads, self.list_capacity)
        self.workspace: Optional[torch.Tensor] = torch.empty(ws, dtype=torch.uint8, device=dev) if ws else None
        # few, long sequences: the fused step spreads each list's scoring over several workgroups through this
        sws = ops.step_workspace_bytes(B, num_kv_heads, max_num_pages)
        self.step_workspace: Optional[torch.Tensor] = torch.empty(sws, dtype=torch.uint8, device=dev) if sws else None

    # -- the three stages, each a custom op --------------------------------
    def refresh_compressed_keys(self) -> None:
        ops.build_kbar(self.kv_cache, self.compressed_key_cache, self.paged_kv_indices, self.paged_kv_indptr, self.last_kv_lens)

    def update_kv(self, key_states: torch.Tensor, value_states: torch.Tensor) -> None:
        """benchmark/blocktopk_decoder.py:209-213."""
        torch.ops.kinetics.append_paged_kv(key_states, value_states, self.kv_cache, self.compressed_key_cache,
                                           self.paged_kv_indices, self.paged_kv_indptr, self.last_kv_lens)

    def select_pages(self, query_states: torch.Tensor) -> None:
        """benchmark/blocktopk_decoder.py:216-221; result lands in ``topk_page_indices``."""
        torch.ops.kinetics.block_score_topk(query_states, self.compressed_key_cache, self.paged_kv_indices,
                                            self.paged_kv_indptr, self.last_kv_lens, self.topk_page,
                                            self.topk_page_indices, self.topk_page_count, self.sink_pages,
                                            self.local_tokens, self.step_workspace, self.page_size)

    def decode(self, query_states: torch.Tensor) -> torch.Tensor:
        """benchmark/blocktopk_decoder.py:223-225."""
        return torch.ops.kinetics.sparse_paged_decode(query_states, self.kv_cache, self.topk_page_indices,
                                                      self.topk_page_count, self.last_kv_lens, self.workspace,
                                                      self.sm_scale, 0)

    def forward(self, query_states, key_states, value_states) -> torch.Tensor:
        """q [B, H_q, D], k/v [B, H_kv, D] -> [B, H_q, D]."""
        if self.fused:
            return torch.ops.kinetics.blocktopk_decode_step(
                query_states, key_states, value_states, self.kv_cache, self.compressed_key_cache,
                self.paged_kv_indices, self.paged_kv_indptr, self.last_kv_lens, self.topk_page,
                self.topk_page_indices, self.topk_page_count, self.sm_scale, self.sink_pages, self.local_tokens, 0,
                self.step_workspace)
        self.update_kv(key_states, value_states)
        self.select_pages(query_states)
        return self.decode(query_states)

    __call__ = forward


class DensePagedAttention:
    """The dense layer's attention (benchmark/dense_decoder.py:136-170,211-219):
    same cache and table, every page attended."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, batch_size: int, prefix_len: int,
                 max_len: int, page_size: int, device="cuda", dtype=torch.bfloat16,
                 share_cache_with: Optional[BlockTopkPagedAttention] = None, seed: int = 0):
        if share_cache_with is None:
            share_cache_with = BlockTopkPagedAttention(num_heads, num_kv_heads, head_dim, batch_size, prefix_len, max_len,
                                                       page_size, 1, device, dtype, seed=seed)
        s = share_cache_with
        self.state = s
        self.num_heads, self.num_kv_heads, self.head_dim = s.num_heads, s.num_kv_heads, s.head_dim
        self.kv_cache, self.paged_kv_indices, self.paged_kv_indptr, self.last_kv_lens = (
            s.kv_cache, s.paged_kv_indices, s.paged_kv_indptr, s.last_kv_lens)
        self.max_pages = s.num_pages_per_req + 1
        self.sm_scale = s.sm_scale
        ws = ops.decode_workspace_bytes(s.batch_size, s.num_heads, s.num_kv_heads, self.max_pages)
        self.workspace = torch.empty(ws, dtype=torch.uint8, device=s.device) if ws else None

    def update_kv(self, key_states, value_states) -> None:
        torch.ops.kinetics.append_paged_kv(key_states, value_states, self.kv_cache, None, self.paged_kv_indices,
                                           self.paged_kv_indptr, self.last_kv_lens)

    def decode(self, query_states) -> torch.Tensor:
        return torch.ops.kinetics.dense_paged_decode(query_states, self.kv_cache, self.paged_kv_indices,
                                                     self.paged_kv_indptr, self.last_kv_lens, self.max_pages,
                                                     self.workspace, self.sm_scale, 0)

    def forward(self, query_states, key_states, value_states) -> torch.Tensor:
        self.update_kv(key_states, value_states)
        return self.decode(query_states)

    __call__ = forward
