"""A KV manager with the interface of LiteSys' ``BatchKVManager``
(LiteSys/litesys/attention/batch_cache.py) on top of the paged HIP kernels.

LiteSys keeps contiguous per-slot caches ``[max_batch, H_kv, max_len, D]`` and,
for block-sparse decoding, computes full-context logits, masks all but the
top-k blocks and runs softmax and P.V over the whole context
(batch_cache.py:154-168, sparsity_utils.py:24-47).  Here every slot draws
16-token pages of one paged cache per layer from a pool through a free list on
the device (``kv_pool_pages`` pages, by default enough for every slot at
``max_seq_len``; fewer saves memory and serves as many tokens as fit);
``clear_cache`` returns a slot's pages to the pool.  Decode appends the token,
scores the per-page mean keys, selects the top-k pages per KV head and attends
only to those pages plus the pinned ones -- the same result as the mask
formulation, without touching the rest of the context.

Supported configurations (anything else raises at construction):
  * no sparsity arguments                      -> dense paged decode
  * ``attn_block_topk=k`` (+ ``attn_local``)    -> block top-k with ``attn_block_size`` 16 (default),
                                                  32 or 64: the pages are that size
  * ``attn_topk=k`` (+ ``attn_local``)          -> token-level top-k (topk_sparsity,
                                                  sparsity_utils.py:6-21), one launch that
                                                  reads every key of the context once
  * ``attn_block_topk=k, attn_stride=s``        -> overlapping blocks every s tokens
                                                  (strided_blockwise_topk_sparsity,
                                                  sparsity_utils.py:49-105), also one launch
  * ``attn_local`` alone                        -> the 4 sink tokens and the newest attn_local
                                                  tokens only (local_sparsity,
                                                  sparsity_utils.py:107-114): the token-level
                                                  kernel with a budget of 0, which reads no key
                                                  outside that window
LiteSys always attends 4 hard-wired "sink" tokens, starts its 16-token blocks
right after them and always attends the ``_local`` newest tokens that remain
after the last whole block (sparsity_utils.py:24-35,240).  To keep that exact
geometry on pages of one block each, a sparse manager stores every sequence
block_size - 4 slots (12 for blocks of 16) into its first page: the sink tokens
are the last 4 slots of page 0, block j is page j+1, and the kernels are told to
skip the padding slots
(``first_page_offset``), to pin one sink page and to keep the newest
``attn_local`` tokens out of the candidates (``local_tokens``).  The attended
token set is then LiteSys' own, token for token.
``attn_layer_skip`` (default ``[0]``: layer 0 stays dense, sparsity_utils.py:211)
is honoured.
Prefill writes its rows and the mean keys of the pages it completes with the
ragged append kernel; its attention is not the accelerated path and runs on
PyTorch's scaled_dot_product_attention (LiteSys calls flashinfer there,
batch_cache.py:112-145).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from . import _lib, ops

PAGE = 16

_UNSUPPORTED = ("attn_random_select", "attn_random_nsample")


class PagedBatchKVManager:
    def __init__(self, config, max_batch_size: int, max_seq_len: int, device, dtype, **kwargs):
        if dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("the HIP kernels are built for bfloat16 and float16")
        self.config = config
        self.max_length = max_seq_len
        self.device = torch.device(device)
        self.dtype = dtype
        self.max_batch_size = max_batch_size
        self.head_dim = getattr(config, "head_dim", config.hidden_size // config.num_attention_heads)
        import torch.distributed as dist

        self.world_size = dist.get_world_size() if dist.is_available() and dist.is_initialized() else 1
        self.num_layers = config.num_hidden_layers
        self.hidden_size = self.head_dim * config.num_attention_heads // self.world_size
        self.num_key_value_heads = config.num_key_value_heads // self.world_size
        self.num_attention_heads = config.num_attention_heads // self.world_size
        self.num_key_value_groups = config.num_attention_heads // config.num_key_value_heads

        for name in _UNSUPPORTED:
            if kwargs.get(name) is not None:
                raise NotImplementedError(f"{name} is a LiteSys research ablation that the paged kernels do not implement")
        self.block_topk = kwargs.get("attn_block_topk")
        self.token_topk = kwargs.get("attn_topk")
        if self.token_topk is not None:
            # same rules as LiteSys (sparsity_utils.py:203-208)
            assert self.block_topk is None, "Only one of the sparsity parameters can be provided"
            if kwargs.get("attn_local") is None:
                raise AssertionError("attn_local must be provided if use_nonlocal_sparsity is True")
            if not 0 <= int(self.token_topk) <= 4096 or not 0 <= int(kwargs["attn_local"]) <= 1024:
                raise NotImplementedError("attn_topk must be in [0, 4096] and attn_local in [0, 1024]")
        self.strided = None
        if self.block_topk is not None:
            if kwargs.get("attn_local") is None:
                # same rule as LiteSys (sparsity_utils.py:207-208)
                raise AssertionError("attn_local must be provided if use_nonlocal_sparsity is True")
            if kwargs.get("attn_stride") is not None:
                # overlapping blocks (sparsity_utils.py:245-246): a token-granular policy, any block size up to 64
                self.strided = (int(self.block_topk), int(kwargs.get("attn_block_size", PAGE)), int(kwargs["attn_stride"]))
                self.token_local = int(kwargs["attn_local"])
                if not (1 <= self.strided[1] <= 64 and self.strided[2] >= 1 and self.strided[0] * self.strided[1] <= 4096
                        and 0 <= self.token_local <= 1024):
                    raise NotImplementedError("strided blocks: block size <= 64, budget <= 4096 tokens, attn_local <= 1024")
                self.block_topk = None
            elif kwargs.get("attn_block_size", PAGE) not in (16, 32, 64, 128):
                raise NotImplementedError("attn_block_size must be 16, 32, 64 or 128 (a block is one page)")
        elif kwargs.get("attn_stride") is not None:
            raise NotImplementedError("attn_stride needs attn_block_topk")
        if kwargs.get("attn_local") is not None and self.block_topk is None and self.strided is None and self.token_topk is None:
            self.token_topk = 0      # window only (local_sparsity, sparsity_utils.py:107-114): 4 sink + attn_local tokens
            if not 0 <= int(kwargs["attn_local"]) <= 1024:
                raise NotImplementedError("attn_local must be in [0, 1024]")
        self.sparse = self.block_topk is not None
        # tokens per page: LiteSys' block size for the block policy, 16 otherwise
        self.page = int(kwargs.get("attn_block_size", PAGE)) if self.sparse else PAGE
        if self.token_topk is not None:
            self.token_local = int(kwargs["attn_local"])
        if self.head_dim not in ops.HEAD_DIMS:
            raise NotImplementedError(f"head_dim {self.head_dim}: the paged kernels are built for {ops.HEAD_DIMS}")
        self.layer_skip = list(kwargs.get("attn_layer_skip", [0]))
        self.sink_pages = 1 if self.sparse else 0
        self.local_tokens = int(kwargs["attn_local"]) if self.sparse else 1
        if self.sparse and not 1 <= self.local_tokens <= 1009:
            raise NotImplementedError("attn_local must be in [1, 1009]")
        # padding slots in front of every sequence: LiteSys' 4 sink tokens end page 0, its blocks are pages 1, 2, ...
        self.pad = self.page - 4 if self.sparse else 0

        B, Hq, Hkv, D = max_batch_size, self.num_attention_heads, self.num_key_value_heads, self.head_dim
        self.pages_per_slot = P = (max_seq_len + self.pad + self.page - 1) // self.page
        dev = self.device
        # The page pool, shared by all layers (a token position occupies the same page id in every
        # layer's cache): slots take pages as they grow and give them back in clear_cache.
        self.num_pool_pages = int(kwargs.get("kv_pool_pages") or B * P)
        if not 1 <= self.num_pool_pages <= B * P:
            raise ValueError(f"kv_pool_pages must be in [1, max_batch_size * pages_per_slot = {B * P}]")
        self.pool = ops.PagePool(self.num_pool_pages, B, P, self.page, dev)
        self.kv_cache = [torch.zeros(self.num_pool_pages, 2, self.page, Hkv, D, dtype=dtype, device=dev)
                         for _ in range(self.num_layers)]
        # mean keys by SLOT; the kernels find a sequence's row block through slot_ids
        self.kbar = [torch.zeros(B, Hkv, P, D, dtype=dtype, device=dev) for _ in range(self.num_layers)]
        self.kv_offset = [torch.zeros(B, dtype=torch.int32, device=dev) for _ in range(self.num_layers)]
        # Page-table metadata of the ACTIVE batch (sequence b of a launch = the b-th entry of batch_idx),
        # built on the device by the first layer of a decode step and reused by the other layers.
        self.page_indices = torch.zeros(self.num_pool_pages, dtype=torch.int32, device=dev)
        self._indptr = torch.zeros(B + 1, dtype=torch.int32, device=dev)
        self._last = torch.ones(B, dtype=torch.int32, device=dev)
        self._one = torch.ones(B, dtype=torch.int32, device=dev)
        self._slots32 = torch.zeros(B, dtype=torch.int32, device=dev)   # the active slots (fixed address: launch plans keep it)
        self._slots64 = torch.zeros(B, dtype=torch.int64, device=dev)
        self._step_batch_idx = None      # the batch_idx object the current table was built for
        self._step = None                # (n, slots int32, slots int64, indptr view, last view, ones view)
        self._plans = {}                 # (layer, n) -> ops.DecodeStepPlan of the fused step
        self._last_layer = -1
        k = self.block_topk or 0
        self._sel = torch.full((B, Hkv, ops.sel_list_capacity(k, self.sink_pages, self.local_tokens)), -1,
                               dtype=torch.int32, device=dev)
        self._cnt = torch.zeros(B, Hkv, dtype=torch.int32, device=dev)
        # one workspace for every kernel and every number of active sequences
        # (the needs are not monotonic in the number of sequences: few lists are shared by teams of workgroups,
        # lists just above a multiple of the GPU's 256 CUs are split or get teams; asking for every size costs
        # tens of milliseconds, once)
        if B <= 8192:
            sizes = range(1, B + 1)
        else:
            tails = {(m + t) // Hkv + d for m in range(256, B * Hkv + 1, 256) for t in (32, 64, 72, 96) for d in (0, 1)}
            sizes = sorted({1 << i for i in range(B.bit_length())} | {B} | set(range(1, 129)) | {n for n in tails if 1 <= n <= B})
        ws = 16
        for n in sizes:
            ws = max(ws, ops.decode_workspace_bytes(n, Hq, Hkv, P), ops.decode_workspace_bytes(n, Hq, Hkv, self._sel.shape[2]),
                     ops.step_workspace_bytes(n, Hkv, P))
            if self.token_topk is not None:
                ws = max(ws, ops.token_topk_workspace_bytes(n, Hkv, P))
            if self.strided is not None:
                ws = max(ws, ops.strided_topk_workspace_bytes(n, Hkv, P))
        self._ws = torch.empty(ws, dtype=torch.uint8, device=dev)
        # raise at the next decode call, not only in clear_cache, when the pool has flagged trouble (costs a
        # device-to-host copy per decode step)
        self.check_overflow_every_step = bool(kwargs.get("check_overflow_every_step", False))
        self._force_fused = None   # tests: True / False pins the route of the block policy (one launch, or three)

    # ------------------------------------------------------------------ LiteSys interface
    def compute_attention(self, query_states, key_states, value_states, layer_idx, batch_idx):
        """query [B, H_q, s, D], key/value [B, H_kv, s, D] -> [B, s, H_q*D]
        (batch_cache.py:86-110).  s > 1 is a prefill of one request."""
        bsz, seq_len = query_states.shape[0], query_states.shape[2]
        if seq_len > 1:
            return self.prefill_or_append(query_states, key_states, value_states, layer_idx, batch_idx)
        out = self.decode(query_states, key_states, value_states, batch_idx, layer_idx)
        return out.reshape(bsz, seq_len, self.hidden_size)

    def clear_cache(self, batch_idx: int):
        """batch_cache.py:147-152.  The slot's pages go back to the pool; they need no
        zeroing (an empty page list hides them).  Also the place where trouble that the
        kernels could only flag is raised, once: an exhausted pool, a sequence beyond
        max_seq_len (such a sequence had an empty page list from then on: nothing was
        written for it and its output was zero)."""
        for i in range(self.num_layers):
            self.kv_offset[i][batch_idx] = 0
        self.pool.release(torch.tensor([int(batch_idx)], dtype=torch.int32, device=self.device))
        self._step_batch_idx = None
        self.pool.raise_on_overflow()

    # ------------------------------------------------------------------ decode
    def _begin_step(self, batch_idx, layer_idx):
        """Page table of the active sequences.  The first layer of a decode step grows the slots
        and builds it (four small launches, no host synchronisation); the other layers of the step
        -- called in increasing order with the same batch_idx object, as LiteSys' layer loop does
        (LiteSys/litesys/models/qwen3.py:134-135) -- find every layer's kv_offset at the same value
        and reuse it."""
        fresh = (self._step_batch_idx is not batch_idx) or layer_idx <= self._last_layer
        self._last_layer = layer_idx
        if fresh:
            n = batch_idx.numel()
            self._step_batch_idx = batch_idx
            self._slots32[:n].copy_(batch_idx, non_blocking=True)
            self._slots64[:n].copy_(batch_idx, non_blocking=True)
            self._step = (n, self._slots32[:n], self._slots64[:n], self._indptr[: n + 1], self._last[:n], self._one[:n])
        n, slots, slots_long, indptr, last, ones = self._step
        if fresh:
            if self.check_overflow_every_step:
                self.pool.raise_on_overflow()
            lens = self.kv_offset[layer_idx][slots_long] + (self.pad + 1)   # after this step's append
            # a slot that crossed a page boundary takes a page from the pool
            self.pool.reserve(lens, slots)
            self.pool.build_page_table(lens, self.page_indices, indptr, last, slots)
        return n, slots, indptr, last

    def _advance(self, layer_idx):
        """kv_offset[layer][batch_idx] += 1 (batch_cache.py:83) for the routes whose kernels do not do it themselves."""
        self.kv_offset[layer_idx].index_add_(0, self._step[2], self._step[5])

    def decode(self, query, key, value, batch_idx, layer_idx):
        """append -> (select ->) attend for the active slots (batch_cache.py:154-168): q, k, v and
        the output are indexed by position in the active batch, the caches by slot (through the
        page table, and slot_ids for the mean keys), as in the reference's kernels
        (LiteSys/litesys/attention/cache_utils.py:40-51,67-70).  Launches are planned for the active
        sequences, whatever max_batch_size is."""
        n, slots, indptr, last = self._begin_step(batch_idx, layer_idx)
        Hkv = self.num_key_value_heads
        q, k, v = query[:, :, 0, :], key[:, :, 0, :], value[:, :, 0, :]
        if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
            q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        out = torch.empty_like(q)
        idx = self.page_indices
        kv, kbar = self.kv_cache[layer_idx], self.kbar[layer_idx]
        sparse = self.sparse and layer_idx not in self.layer_skip
        if self.token_topk is not None and layer_idx not in self.layer_skip:
            # token-level top-k: LiteSys' 4 sink tokens, the top tokens of the middle, the newest attn_local tokens
            self._advance(layer_idx)
            ops.append_paged_kv(k, v, kv, None, idx, indptr, last)
            ops.token_topk_decode(q, kv, idx, indptr, last, self.token_topk, self.pages_per_slot, sink_tokens=4,
                                  local_tokens=self.token_local, out=out, workspace=self._ws)
        elif self.strided is not None and layer_idx not in self.layer_skip:
            self._advance(layer_idx)
            ops.append_paged_kv(k, v, kv, None, idx, indptr, last)
            ops.strided_topk_decode(q, kv, idx, indptr, last, self.strided[0], self.pages_per_slot,
                                    block_size=self.strided[1], stride=self.strided[2], sink_tokens=4,
                                    local_tokens=self.token_local, out=out, workspace=self._ws)
        elif sparse and (self._force_fused if self._force_fused is not None
                         else ops.prefer_fused_step(n, Hkv, self.pages_per_slot, self.block_topk)):
            plan = self._plans.get((layer_idx, n))
            if plan is None:   # everything but q, k, v, out is the manager's own and stays where it is: bound once
                plan = self._plans[(layer_idx, n)] = ops.DecodeStepPlan(
                    kv, kbar, idx, indptr, last, self.block_topk, self.num_attention_heads, sink_pages=self.sink_pages,
                    local_tokens=self.local_tokens, first_page_offset=self.pad, workspace=self._ws, slot_ids=slots,
                    slot_lens=self.kv_offset[layer_idx])     # the kernel advances the slots' offsets itself
            plan(q, k, v, out)
        else:
            self._advance(layer_idx)
            ops.append_paged_kv(k, v, kv, kbar, idx, indptr, last, slot_ids=slots)
            if sparse:
                sel, cnt = self._sel[:n], self._cnt[:n]
                ops.block_score_topk(q, kbar, idx, indptr, last, self.block_topk, sel, cnt, sink_pages=self.sink_pages,
                                     local_tokens=self.local_tokens, workspace=self._ws, page_size=self.page, slot_ids=slots)
                ops.sparse_paged_decode(q, kv, sel, cnt, last, out=out, workspace=self._ws, first_page_offset=self.pad)
            else:
                ops.dense_paged_decode(q, kv, idx, indptr, last, self.pages_per_slot, out=out, workspace=self._ws,
                                       first_page_offset=self.pad)
        return out

    # ------------------------------------------------------------------ prefill (not the accelerated path)
    def prefill_or_append(self, query_states, key_states, value_states, layer_idx, batch_idx):
        """One request: write its K/V rows into the slot's pages and refresh the
        mean keys of the pages that are now full (one ragged append), then causal
        attention over the slot's whole context (batch_cache.py:112-145)."""
        bsz, seq_len = query_states.shape[0], query_states.shape[2]
        slot = int(batch_idx.item())
        offset = int(self.kv_offset[layer_idx][slot].item())
        total = offset + seq_len
        pad = self.pad                                   # token t lives in cache slot t + pad
        if total + pad > self.pages_per_slot * self.page:
            raise ValueError(f"sequence of {total} tokens exceeds max_seq_len")
        Hkv, D = self.num_key_value_heads, self.head_dim
        n_pages = (total + pad + self.page - 1) // self.page
        self._step_batch_idx = None   # the next decode step builds its table afresh
        self.pool.reserve(torch.tensor([total + pad], dtype=torch.int32, device=self.device),
                          torch.tensor([slot], dtype=torch.int32, device=self.device))
        free, bits = self.pool.status()
        if bits & ops.PagePool.EXHAUSTED:
            # nothing was reserved and nothing is recorded: the request can be retried after a clear_cache
            self.pool.acknowledge()
            raise _lib.KineticsError(f"page pool exhausted ({free} pages free): cannot hold {total} tokens in slot {slot}")
        self.kv_offset[layer_idx][slot] += seq_len
        idx = self.pool.slot_table[slot, :n_pages].contiguous()
        ptr = torch.tensor([0, n_pages], dtype=torch.int32, device=self.device)
        last = torch.tensor([total + pad - (n_pages - 1) * self.page], dtype=torch.int32, device=self.device)
        # rows to their page slots, mean keys of the pages that are now full
        ops.append_paged_kv_ragged(key_states[0].transpose(0, 1).contiguous(), value_states[0].transpose(0, 1).contiguous(),
                                   torch.tensor([0, seq_len], dtype=torch.int32, device=self.device),
                                   self.kv_cache[layer_idx], self.kbar[layer_idx][slot:slot + 1], idx, ptr, last)
        pages = self.kv_cache[layer_idx][idx.long()]                                           # [n_pages, 2, self.page, Hkv, D]
        k_all = pages[:, 0].reshape(n_pages * self.page, Hkv, D)[pad:total + pad].transpose(0, 1)   # [Hkv, total, D]
        v_all = pages[:, 1].reshape(n_pages * self.page, Hkv, D)[pad:total + pad].transpose(0, 1)
        G = self.num_attention_heads // Hkv
        q = query_states[0]                                                                    # [Hq, s, D]
        pos_q = torch.arange(offset, total, device=self.device)[:, None]
        mask = torch.arange(total, device=self.device)[None, :] <= pos_q                       # causal with history
        o = F.scaled_dot_product_attention(q[None], k_all.repeat_interleave(G, dim=0)[None],
                                           v_all.repeat_interleave(G, dim=0)[None], attn_mask=mask[None, None],
                                           scale=1.0 / math.sqrt(D))[0]                       # [Hq, s, D]
        return o.transpose(0, 1).reshape(bsz, seq_len, self.hidden_size)
